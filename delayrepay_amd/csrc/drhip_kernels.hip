// Static gfx950 kernels of libdrhip: pattern fill and the plain streaming copy
// used as the measured ceiling of the memory system.  Generated expression
// kernels are not here; they are emitted as source at run time.
#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>
#include <stdint.h>

namespace {

constexpr unsigned kBlock = 256;  // 4 wave64 per workgroup

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename W>
__global__ __launch_bounds__(kBlock) void fill_kernel(W* __restrict__ dst, W v, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (; i < n; i += stride) dst[i] = v;
}

// 128-bit non-temporal loads and stores.  A block copies runs of 256 consecutive
// vectors and advances by gridDim.x runs; launched with one run per block, which is
// the fastest read+write pattern measured on MI355X (the DRAM access stream stays
// nearly sequential).
__global__ __launch_bounds__(kBlock) void copy_kernel(u32x4* __restrict__ dst,
                                                      const u32x4* __restrict__ src, size_t nvec) {
    const size_t nrun = nvec / kBlock;
    for (size_t r = blockIdx.x; r < nrun; r += gridDim.x) {
        const size_t i = r * kBlock + threadIdx.x;
        u32x4 a = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(a, dst + i);
    }
    for (size_t i = nrun * kBlock + (size_t)blockIdx.x * kBlock + threadIdx.x; i < nvec;
         i += (size_t)gridDim.x * kBlock) {
        u32x4 a = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(a, dst + i);
    }
}

// C[M,N] = A[M,K] * B[K,N], row-major with leading dimensions.  64x64 output tile
// per 256-thread block, 4x4 outputs per thread, K staged through LDS 16 deep.
// Serves the eager `dot` of the array namespace; it is not on the fused path.
template <typename T>
__global__ __launch_bounds__(kBlock) void matmul_kernel(const T* __restrict__ A,
                                                        const T* __restrict__ B,
                                                        T* __restrict__ C, long M, long N, long K,
                                                        long lda, long ldb, long ldc) {
    constexpr int TM = 64, TN = 64, TK = 16;
    __shared__ T As[TK][TM + 1];
    __shared__ T Bs[TK][TN + 1];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const long row0 = (long)blockIdx.y * TM, col0 = (long)blockIdx.x * TN;
    T acc[4][4] = {};
    for (long k0 = 0; k0 < K; k0 += TK) {
        for (int i = threadIdx.x; i < TM * TK; i += kBlock) {
            const int r = i / TK, k = i % TK;
            const long gr = row0 + r, gk = k0 + k;
            As[k][r] = (gr < M && gk < K) ? A[gr * lda + gk] : T(0);
        }
        for (int i = threadIdx.x; i < TK * TN; i += kBlock) {
            const int k = i / TN, c = i % TN;
            const long gk = k0 + k, gc = col0 + c;
            Bs[k][c] = (gk < K && gc < N) ? B[gk * ldb + gc] : T(0);
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < TK; ++k) {
            T a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const long r = row0 + ty * 4 + i, c = col0 + tx + 16 * j;
            if (r < M && c < N) C[r * ldc + c] = acc[i][j];
        }
}

unsigned fill_grid(size_t n) {
    size_t b = (n + kBlock - 1) / kBlock;
    const size_t cap = 256u * 16u;
    return (unsigned)(b < cap ? b : cap);
}

}  // namespace

extern "C" void drhip_k_launch_fill32(void* dst, uint32_t v, size_t n, hipStream_t s) {
    hipLaunchKernelGGL(fill_kernel<uint32_t>, dim3(fill_grid(n)), dim3(kBlock), 0, s,
                       (uint32_t*)dst, v, n);
}

extern "C" void drhip_k_launch_fill64(void* dst, uint64_t v, size_t n, hipStream_t s) {
    hipLaunchKernelGGL(fill_kernel<uint64_t>, dim3(fill_grid(n)), dim3(kBlock), 0, s,
                       (uint64_t*)dst, v, n);
}

extern "C" void drhip_k_launch_copy(void* dst, const void* src, size_t nvec, unsigned grid,
                                    hipStream_t s) {
    hipLaunchKernelGGL(copy_kernel, dim3(grid), dim3(kBlock), 0, s, (u32x4*)dst,
                       (const u32x4*)src, nvec);
}

extern "C" void drhip_k_launch_matmul(int is_double, const void* A, const void* B, void* C, long M,
                                      long N, long K, long lda, long ldb, long ldc,
                                      hipStream_t s) {
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
    if (is_double)
        hipLaunchKernelGGL(matmul_kernel<double>, grid, dim3(kBlock), 0, s, (const double*)A,
                           (const double*)B, (double*)C, M, N, K, lda, ldb, ldc);
    else
        hipLaunchKernelGGL(matmul_kernel<float>, grid, dim3(kBlock), 0, s, (const float*)A,
                           (const float*)B, (float*)C, M, N, K, lda, ldb, ldc);
}

// Inclusive prefix sum of n elements (hipCUB device scan).  Two-phase protocol:
// with temp == nullptr only *temp_bytes is set.
template <typename T>
static hipError_t scan_sum(void* temp, size_t* temp_bytes, const void* in, void* out, size_t n,
                           hipStream_t s) {
    return hipcub::DeviceScan::InclusiveSum(temp, *temp_bytes, (const T*)in, (T*)out, (int)n, s);
}

extern "C" int drhip_k_cumsum(int kind, void* temp, size_t* temp_bytes, const void* in, void* out,
                              size_t n, hipStream_t s) {
    switch (kind) {
        case 0: return (int)scan_sum<float>(temp, temp_bytes, in, out, n, s);
        case 1: return (int)scan_sum<double>(temp, temp_bytes, in, out, n, s);
        case 2: return (int)scan_sum<int32_t>(temp, temp_bytes, in, out, n, s);
        case 3: return (int)scan_sum<int64_t>(temp, temp_bytes, in, out, n, s);
    }
    return (int)hipErrorInvalidValue;
}
