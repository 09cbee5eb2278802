/*
 * drhip.h -- C ABI of libdrhip.so, the device runtime under the DelayRepay
 * HIP fusion backend for AMD Instinct MI355X (gfx950).
 *
 * The reference's GPU backend (delayrepay/cuda.py) has no FFI of its own: it
 * reaches the device through CuPy (cupy.ElementwiseKernel -> NVRTC -> CUDA
 * driver launch, CuPy's memory pool, cupy.ndarray.get()).  This library is the
 * set of entry points a backend module needs in place of those CuPy services.
 * Each declaration names the reference call site whose CuPy service it
 * replaces.
 *
 * Conventions
 *   - plain C types only; device memory is passed as void* device addresses;
 *   - every function returning int returns 0 on success, otherwise a non-zero
 *     code (hipError_t, or 10000 + hiprtcResult for compiler errors, or a
 *     DRHIP_E* value below); drhip_last_error() then holds a message;
 *   - all work is issued on one library-owned stream, in order; a call
 *     returns once the work is queued unless stated otherwise;
 *   - not thread-safe: one host thread drives the library (the reference is
 *     single threaded as well: delayrepay/delayarray.py:27-32 keeps unguarded
 *     module globals).
 */
#ifndef DRHIP_H
#define DRHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DRHIP_ENOTINIT 20001 /* drhip_init has not succeeded yet          */
#define DRHIP_EINVAL   20002 /* argument rejected before touching the GPU */
#define DRHIP_ERTC     10000 /* + hiprtcResult                            */

/* ---- life cycle --------------------------------------------------------- */

/* Select the device, create the stream, read device properties.  Idempotent.
 * Replaces the implicit CUDA context creation done by `import cupy`
 * (delayrepay/cuda.py:17). */
int drhip_init(int device);

/* Fixed facts about the device chosen by drhip_init. */
typedef struct drhip_device_info {
    char     name[128];
    char     arch[64];       /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"  */
    int32_t  compute_units;
    int32_t  wavefront_size;
    int32_t  max_lds_bytes;  /* per workgroup                                */
    int32_t  l2_bytes;
    int64_t  total_mem;
    int32_t  clock_khz;
    int32_t  mem_clock_khz;
    int32_t  mem_bus_bits;
    int32_t  hiprtc_version; /* major * 1000 + minor of the run-time compiler   */
} drhip_device_info;
int drhip_device_info_get(drhip_device_info* out);

/* Thread-local message for the last non-zero return on this thread. */
const char* drhip_last_error(void);

/* ---- pooled device memory ----------------------------------------------
 * Replaces CuPy's default memory pool, from which cuda.py:96 `kern(*inputs)`
 * takes its output array and which frees on garbage collection.
 * Blocks are rounded up to a size class and recycled through per-class free
 * lists; nothing is returned to the driver until drhip_pool_trim().  Reuse is
 * safe without synchronisation because every kernel and copy runs on the one
 * library stream, in order. */
int drhip_malloc(void** dptr, size_t nbytes);
int drhip_free(void* dptr);

typedef struct drhip_pool_stats_t {
    uint64_t bytes_in_use;     /* handed out, class-rounded                 */
    uint64_t bytes_cached;     /* sitting in free lists                     */
    uint64_t bytes_peak;       /* high-water mark of in_use + cached        */
    uint64_t n_driver_allocs;  /* hipMalloc calls so far                    */
    uint64_t n_pool_hits;      /* drhip_malloc served from a free list      */
    uint64_t n_mallocs;        /* drhip_malloc calls so far                 */
} drhip_pool_stats_t;
int drhip_pool_stats(drhip_pool_stats_t* out);
/* Give every cached block back to the driver (synchronises first). */
int drhip_pool_trim(void);

/* ---- copies -------------------------------------------------------------
 * h2d replaces cupy.asarray / cupy.array on host data (delayarray.py:620-623
 * through cuda.fallback); d2h replaces cupy.ndarray.get() (delayarray.py:104)
 * and blocks until the bytes are in host memory; d2d is queued. */
int drhip_memcpy_h2d(void* dst_dev, const void* src_host, size_t nbytes);
int drhip_memcpy_d2h(void* dst_host, const void* src_dev, size_t nbytes);
int drhip_memcpy_d2d(void* dst_dev, const void* src_dev, size_t nbytes);
/* Fill nwords 32-bit (or 64-bit) words with a pattern, using a fill kernel
 * (no memset node, so the call is safe to record into a HIP graph). */
int drhip_fill32(void* dst_dev, uint32_t pattern, size_t nwords);
int drhip_fill64(void* dst_dev, uint64_t pattern, size_t nwords);
/* Plain streaming copy kernel (128-bit non-temporal loads and stores); used as
 * the measured ceiling of the memory system next to generated kernels and to
 * calibrate profiler byte counters.  nbytes must be a multiple of 16;
 * grid_blocks = 0 picks one run of 256 vectors per block. */
int drhip_copy_kernel(void* dst_dev, const void* src_dev, size_t nbytes,
                      unsigned grid_blocks);

/* Row-major C[m,n] = A[m,k] * B[k,n] in float (is_double = 0) or double, leading
 * dimensions in elements.  Replaces `_backend.fallback.dot` = cupy.dot -> cuBLAS
 * (delayarray.py:85) for matrix operands; eager, not part of the fused path.
 * Products with at least 64 rows and columns run on the matrix cores (128x128 tiles
 * of MFMA accumulators), smaller ones on a 64x64 vector-ALU tile. */
int drhip_matmul(int is_double, const void* a, const void* b, void* c, int64_t m, int64_t n,
                 int64_t k, int64_t lda, int64_t ldb, int64_t ldc);

/* Inclusive prefix sum of n contiguous elements; kind 0 float, 1 double, 2 int32,
 * 3 int64.  Replaces `_backend.fallback.cumsum` = cupy.cumsum (delayarray.py:558);
 * eager, not part of the fused path. */
int drhip_cumsum(int kind, const void* in_dev, void* out_dev, size_t n);

/* ---- run-time compilation ----------------------------------------------
 * Replaces cupy.ElementwiseKernel(...) construction (cuda.py:35-43), i.e.
 * NVRTC + module load.  `src` is HIP C++ text holding one or more
 * `extern "C" __global__` functions.  The library always passes
 * --offload-arch=<device arch or DRHIP_ARCH>; `opts` are added after it.
 * On success *module is an opaque handle.  drhip_compile needs no GPU when
 * `module` is NULL: it then only compiles, which lets a build machine check
 * generated source; the code object can be fetched with drhip_code_get. */
int drhip_compile(const char* src, const char* name, const char* const* opts,
                  int nopts, void** module);
/* Code object of the most recent successful drhip_compile on this thread
 * (valid until the next compile).  For the on-disk kernel cache. */
int drhip_code_get(const void** code, size_t* nbytes);
/* Load a code object produced earlier by drhip_compile (disk-cache hit). */
int drhip_load_code(const void* code, size_t nbytes, void** module);
int drhip_module_unload(void* module);
int drhip_get_function(void* module, const char* kernel_name, void** func);
/* Compiler diagnostics of the most recent drhip_compile on this thread. */
const char* drhip_compile_log(void);

/* ---- launch -------------------------------------------------------------
 * Replaces `kern(*inputs)` (cuda.py:95-96).  `args` is the kernel's argument
 * block laid out exactly as the kernel's parameters (natural alignment, as a
 * C struct), `args_bytes` its size.  1-D grid of `grid_x` blocks of `block_x`
 * threads, `lds_bytes` of dynamic LDS. */
int drhip_launch(void* func, unsigned grid_x, unsigned block_x,
                 unsigned lds_bytes, const void* args, size_t args_bytes);

/* drhip_launch for a kernel that needs device scratch memory (the partial results a
 * reduction kernel hands to its finalising kernel), for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference (whose reductions are CuPy library calls,
 * delayarray.py:516-518).  The call allocates nothing: the scratch memory is one static
 * device array of drhip_scratch_bytes() bytes (4 MiB) that every GPU the library runs on
 * holds until the process ends.  Its address on the current device is written into the
 * pointer slot at byte offset `scratch_arg_offset` of the argument block (a multiple of
 * 8; the slot's previous contents are ignored), then the kernel is launched exactly as
 * drhip_launch would.  The kernel may use the first `scratch_bytes` bytes; a request
 * above drhip_scratch_bytes(), or an argument block above DRHIP_MAX_ARGS_BYTES, is
 * refused with DRHIP_EINVAL.  All calls on a GPU share the array and it keeps the last
 * call's contents: a kernel must write what it later reads (nothing is cleared), work
 * queued through this library is ordered by its one stream, and users of the array that
 * overlap on one GPU by any other route race. */
#define DRHIP_MAX_ARGS_BYTES 4096
int drhip_launch_scratch(void* func, unsigned grid_x, unsigned block_x, unsigned lds_bytes,
                         const void* args, size_t args_bytes, size_t scratch_arg_offset,
                         size_t scratch_bytes);
size_t drhip_scratch_bytes(void);

/* ---- HIP graphs -----------------------------------------------------------
 * Capture the launches issued between begin and end into a graph and replay
 * them with one call: for launch-bound loops (small arrays, many sweeps).  The
 * reference has no counterpart (it launches kernel by kernel, cuda.py:96).
 * Between begin and end only drhip_launch, drhip_fill32/64 and
 * drhip_copy_kernel may be called (no allocation, copy or synchronisation);
 * captured kernels keep the device addresses they were recorded with. */
int drhip_graph_begin(void);
int drhip_graph_end(void** graph_exec);
int drhip_graph_launch(void* graph_exec);
int drhip_graph_destroy(void* graph_exec);

/* ---- synchronisation and timing ---------------------------------------- */
int drhip_sync(void);
int drhip_event_create(void** ev);
int drhip_event_destroy(void* ev);
int drhip_event_record(void* ev);            /* on the library stream      */
int drhip_event_sync(void* ev);
int drhip_event_elapsed_ms(void* start, void* stop, float* ms);

/* Counters for the bench harness. */
typedef struct drhip_counters_t {
    uint64_t n_compiles;
    uint64_t n_code_loads;
    uint64_t n_launches;
    uint64_t compile_ns;     /* wall time spent inside hiprtc              */
} drhip_counters_t;
int drhip_counters(drhip_counters_t* out);

#ifdef __cplusplus
}
#endif
#endif /* DRHIP_H */
