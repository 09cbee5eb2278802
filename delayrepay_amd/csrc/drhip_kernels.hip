// Static gfx950 kernels of libdrhip: pattern fill and the plain streaming copy
// used as the measured ceiling of the memory system.  Generated expression
// kernels are not here; they are emitted as source at run time.
#include <hip/hip_runtime.h>
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

// 128-bit loads and stores, grid-stride, four independent vectors in flight
// per thread and iteration.
__global__ __launch_bounds__(kBlock) void copy_kernel(u32x4* __restrict__ dst,
                                                      const u32x4* __restrict__ src, size_t nvec) {
    const size_t stride = (size_t)gridDim.x * kBlock;
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    for (; i + 3 * stride < nvec; i += 4 * stride) {
        u32x4 a = __builtin_nontemporal_load(src + i);
        u32x4 b = __builtin_nontemporal_load(src + i + stride);
        u32x4 c = __builtin_nontemporal_load(src + i + 2 * stride);
        u32x4 d = __builtin_nontemporal_load(src + i + 3 * stride);
        __builtin_nontemporal_store(a, dst + i);
        __builtin_nontemporal_store(b, dst + i + stride);
        __builtin_nontemporal_store(c, dst + i + 2 * stride);
        __builtin_nontemporal_store(d, dst + i + 3 * stride);
    }
    for (; i < nvec; i += stride) {
        u32x4 a = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(a, dst + i);
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
