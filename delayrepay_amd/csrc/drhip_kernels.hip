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

// ---- the same product on the matrix cores -----------------------------------------
// A 256-thread block owns a 128x128 tile of C; its four waves own 64x64 quarters and
// keep them in MFMA accumulators (float: 2x2 tiles of v_mfma_f32_32x32x2f32, double:
// 4x4 tiles of v_mfma_f64_16x16x4f64).  A and B pass through LDS TK deep, A stored
// k-major so that both operands are read with consecutive lanes on consecutive
// addresses; the next k-slab is fetched from global memory into registers while the
// current one is multiplied (two LDS buffers, one barrier per slab).
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef double f64x2u __attribute__((ext_vector_type(2), aligned(8)));

template <typename T> struct Mfma;
template <> struct Mfma<float> {
    static constexpr int MT = 32, MK = 2, TILES = 2, NACC = 16, V = 4, TK = 16;
    using acc_t = f32x16;
    using vec_t = f32x4;
    using vecu_t = f32x4u;
    static __device__ __forceinline__ acc_t mac(float a, float b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    // accumulator register v of lane l holds C[row(v, l)][l % 32]
    static __device__ __forceinline__ int row(int v, int lane) {
        return (v / 4) * 8 + (lane / 32) * 4 + (v % 4);
    }
};
template <> struct Mfma<double> {
    static constexpr int MT = 16, MK = 4, TILES = 4, NACC = 4, V = 2, TK = 8;
    using acc_t = f64x4;
    using vec_t = f64x2;
    using vecu_t = f64x2u;
    static __device__ __forceinline__ acc_t mac(double a, double b, acc_t c) {
        return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ int row(int v, int lane) { return 4 * v + lane / 16; }
};

template <typename T>
__global__ __launch_bounds__(kBlock) void matmul_mfma_kernel(const T* __restrict__ A,
                                                             const T* __restrict__ B,
                                                             T* __restrict__ C, long M, long N,
                                                             long K, long lda, long ldb,
                                                             long ldc) {
    using P = Mfma<T>;
    constexpr int MT = P::MT, MK = P::MK, TI = P::TILES, V = P::V, TK = P::TK;
    constexpr int BM = 2 * TI * MT, BN = BM, PAD = 4;      // 128 x 128
    constexpr int A_VECS = BM * TK / V / kBlock;            // vectors per thread and slab: 2
    constexpr int B_VECS = TK * BN / V / kBlock;
    __shared__ __attribute__((aligned(16))) T As[2][TK][BM + PAD];
    __shared__ __attribute__((aligned(16))) T Bs[2][TK][BN + PAD];   // rows are 16-byte multiples
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long row0 = (long)blockIdx.y * BM, col0 = (long)blockIdx.x * BN;
    const int wrow = (wave >> 1) * TI * MT, wcol = (wave & 1) * TI * MT;
    typename P::acc_t acc[TI][TI];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TI; ++j)
#pragma unroll
            for (int v = 0; v < P::NACC; ++v) acc[i][j][v] = T(0);

    typename P::vec_t ra[A_VECS], rb[B_VECS];
    auto fetch = [&](long k0) {
#pragma unroll
        for (int p = 0; p < A_VECS; ++p) {
            const int idx = threadIdx.x + p * kBlock;
            const int r = idx / (TK / V), kq = (idx % (TK / V)) * V;
            const long gr = row0 + r, gk = k0 + kq;
            if (gr < M && gk + V <= K) {
                ra[p] = *(const typename P::vecu_t*)(A + gr * lda + gk);
            } else {
#pragma unroll
                for (int q = 0; q < V; ++q)
                    ra[p][q] = (gr < M && gk + q < K) ? A[gr * lda + gk + q] : T(0);
            }
        }
#pragma unroll
        for (int p = 0; p < B_VECS; ++p) {
            const int idx = threadIdx.x + p * kBlock;
            const int k = idx / (BN / V), c = (idx % (BN / V)) * V;
            const long gk = k0 + k, gc = col0 + c;
            if (gk < K && gc + V <= N) {
                rb[p] = *(const typename P::vecu_t*)(B + gk * ldb + gc);
            } else {
#pragma unroll
                for (int q = 0; q < V; ++q)
                    rb[p][q] = (gk < K && gc + q < N) ? B[gk * ldb + gc + q] : T(0);
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int p = 0; p < A_VECS; ++p) {
            const int idx = threadIdx.x + p * kBlock;
            const int r = idx / (TK / V), kq = (idx % (TK / V)) * V;
#pragma unroll
            for (int q = 0; q < V; ++q) As[buf][kq + q][r] = ra[p][q];
        }
#pragma unroll
        for (int p = 0; p < B_VECS; ++p) {
            const int idx = threadIdx.x + p * kBlock;
            const int k = idx / (BN / V), c = (idx % (BN / V)) * V;
            *(typename P::vec_t*)&Bs[buf][k][c] = rb[p];
        }
    };

    const long slabs = (K + TK - 1) / TK;
    fetch(0);
    stage(0);
    __syncthreads();
    for (long s = 0; s < slabs; ++s) {
        const int buf = (int)(s & 1);
        if (s + 1 < slabs) fetch((s + 1) * TK);
#pragma unroll
        for (int ks = 0; ks < TK / MK; ++ks) {
            const int k = ks * MK + lane / MT;
            T a[TI], b[TI];
#pragma unroll
            for (int i = 0; i < TI; ++i) a[i] = As[buf][k][wrow + i * MT + lane % MT];
#pragma unroll
            for (int j = 0; j < TI; ++j) b[j] = Bs[buf][k][wcol + j * MT + lane % MT];
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < TI; ++j) acc[i][j] = P::mac(a[i], b[j], acc[i][j]);
        }
        if (s + 1 < slabs) stage(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TI; ++j)
#pragma unroll
            for (int v = 0; v < P::NACC; ++v) {
                const long r = row0 + wrow + i * MT + P::row(v, lane);
                const long c = col0 + wcol + j * MT + lane % MT;
                if (r < M && c < N) C[r * ldc + c] = acc[i][j][v];
            }
}

unsigned fill_grid(size_t n) {
    size_t b = (n + kBlock - 1) / kBlock;
    const size_t cap = 256u * 16u;
    return (unsigned)(b < cap ? b : cap);
}

}  // namespace

// ---- static scratch memory ----------------------------------------------------------
// Device memory for drhip_launch_scratch: partial results of reductions for callers that
// cannot allocate.  One array per GPU (each device that loads this code object holds its
// own copy at its own address) until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress, never a device address: the address is looked up
// once per device and everything else works with that pointer.
#define DRHIP_SCRATCH_BYTES (4u << 20)
static __device__ __align__(256) unsigned char scratch[DRHIP_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// Look up the address of `scratch` on `device`, which must be the current device.
extern "C" int drhip_k_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
    if (g_scratch_ptr[device]) return 0;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[device] = ptr;
    return 0;
}

// Device address of the scratch array on `device` (null before drhip_k_scratch_init).
extern "C" void* drhip_k_scratch_ptr(int device) {
    return (device >= 0 && device < kMaxDevices) ? g_scratch_ptr[device] : nullptr;
}

extern "C" size_t drhip_k_scratch_bytes(void) { return DRHIP_SCRATCH_BYTES; }

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
    if (M >= 64 && N >= 64 && K >= 8) {   // enough of a 128x128 tile to be worth the matrix cores
        dim3 grid((unsigned)((N + 127) / 128), (unsigned)((M + 127) / 128));
        if (is_double)
            hipLaunchKernelGGL(matmul_mfma_kernel<double>, grid, dim3(kBlock), 0, s,
                               (const double*)A, (const double*)B, (double*)C, M, N, K, lda, ldb,
                               ldc);
        else
            hipLaunchKernelGGL(matmul_mfma_kernel<float>, grid, dim3(kBlock), 0, s,
                               (const float*)A, (const float*)B, (float*)C, M, N, K, lda, ldb,
                               ldc);
        return;
    }
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
