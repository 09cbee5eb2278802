// libdrhip: device runtime under the DelayRepay HIP fusion backend (gfx950).
//
// Owns one HIP stream, a pooled allocator over hipMalloc, the hiprtc
// compile/load path for generated kernels, and launch/timing helpers.
// Interface and conventions: include/drhip.h.
#include "../../include/drhip.h"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

// static kernels, defined in drhip_kernels.hip
extern "C" void drhip_k_launch_fill32(void* dst, uint32_t v, size_t n, hipStream_t s);
extern "C" void drhip_k_launch_fill64(void* dst, uint64_t v, size_t n, hipStream_t s);
extern "C" void drhip_k_launch_copy(void* dst, const void* src, size_t nvec,
                                    unsigned grid, hipStream_t s);

extern "C" void drhip_k_launch_matmul(int is_double, const void* A, const void* B, void* C, long M,
                                      long N, long K, long lda, long ldb, long ldc,
                                      hipStream_t s);

extern "C" int drhip_k_cumsum(int kind, void* temp, size_t* temp_bytes, const void* in, void* out,
                              size_t n, hipStream_t s);

extern "C" int drhip_k_scratch_init(int device);
extern "C" void* drhip_k_scratch_ptr(int device);
extern "C" size_t drhip_k_scratch_bytes(void);

namespace {

thread_local std::string t_err;
thread_local std::string t_log;
thread_local std::vector<char> t_code;

bool g_init = false;
bool g_capturing = false;
int g_device = -1;
hipStream_t g_stream = nullptr;
hipDeviceProp_t g_prop;
std::string g_arch;

struct Pool {
    std::unordered_map<size_t, std::vector<void*>> free_lists;
    std::unordered_map<void*, size_t> live;  // ptr -> class size
    drhip_pool_stats_t st{};
} g_pool;

drhip_counters_t g_cnt{};

int fail(int code, const char* what, const char* detail) {
    char buf[512];
    snprintf(buf, sizeof buf, "%s: %s (code %d)", what, detail ? detail : "", code);
    t_err = buf;
    return code;
}

#define HIP_TRY(expr)                                                     \
    do {                                                                  \
        hipError_t e_ = (expr);                                           \
        if (e_ != hipSuccess) return fail((int)e_, #expr, hipGetErrorString(e_)); \
    } while (0)

#define NEED_INIT()                                                       \
    do {                                                                  \
        if (!g_init) return fail(DRHIP_ENOTINIT, "drhip", "drhip_init has not been called"); \
    } while (0)

// Size classes: powers of two up to 1 MiB, then multiples of 2 MiB.  Large
// arrays of equal shape (the common case for expression temporaries and
// outputs) land in the same class and recycle exactly.
size_t size_class(size_t n) {
    if (n == 0) n = 1;
    const size_t small_max = size_t(1) << 20;
    if (n <= small_max) {
        size_t c = 256;
        while (c < n) c <<= 1;
        return c;
    }
    const size_t gran = size_t(2) << 20;
    return (n + gran - 1) / gran * gran;
}

}  // namespace

extern "C" {

const char* drhip_last_error(void) { return t_err.c_str(); }
const char* drhip_compile_log(void) { return t_log.c_str(); }

int drhip_init(int device) {
    if (g_init) {
        if (device == g_device) return 0;
        return fail(DRHIP_EINVAL, "drhip_init", "already initialised on another device");
    }
    int n = 0;
    HIP_TRY(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) return fail(DRHIP_EINVAL, "drhip_init", "no such device");
    HIP_TRY(hipSetDevice(device));
    HIP_TRY(hipGetDeviceProperties(&g_prop, device));
    HIP_TRY(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
    // address of the static scratch array on this device (drhip_launch_scratch)
    if (int rc = drhip_k_scratch_init(device))
        return fail(rc, "hipGetSymbolAddress(scratch)", hipGetErrorString((hipError_t)rc));
    g_arch = g_prop.gcnArchName;
    g_device = device;
    g_init = true;
    return 0;
}

int drhip_device_info_get(drhip_device_info* out) {
    NEED_INIT();
    if (!out) return fail(DRHIP_EINVAL, "drhip_device_info_get", "null out");
    memset(out, 0, sizeof *out);
    snprintf(out->name, sizeof out->name, "%s", g_prop.name);
    snprintf(out->arch, sizeof out->arch, "%s", g_prop.gcnArchName);
    out->compute_units = g_prop.multiProcessorCount;
    out->wavefront_size = g_prop.warpSize;
    out->max_lds_bytes = (int32_t)g_prop.sharedMemPerBlock;
    out->l2_bytes = g_prop.l2CacheSize;
    out->total_mem = (int64_t)g_prop.totalGlobalMem;
    out->clock_khz = g_prop.clockRate;
    out->mem_clock_khz = g_prop.memoryClockRate;
    out->mem_bus_bits = g_prop.memoryBusWidth;
    int major = 0, minor = 0;
    if (hiprtcVersion(&major, &minor) == HIPRTC_SUCCESS) out->hiprtc_version = major * 1000 + minor;
    return 0;
}

// ---- pool ------------------------------------------------------------------
// One host thread drives the library, but an array's finaliser may run on whichever
// thread happens to collect it, while the driving thread is inside another call (a
// Python caller drops its interpreter lock for the duration of a foreign call): the
// pool's tables are therefore guarded.  Recursive: an out-of-memory drhip_malloc trims.
static std::recursive_mutex g_pool_mutex;
#define POOL_LOCK() std::lock_guard<std::recursive_mutex> pool_lock_(g_pool_mutex)

int drhip_malloc(void** dptr, size_t nbytes) {
    NEED_INIT();
    if (!dptr) return fail(DRHIP_EINVAL, "drhip_malloc", "null dptr");
    POOL_LOCK();
    const size_t c = size_class(nbytes);
    g_pool.st.n_mallocs++;
    auto it = g_pool.free_lists.find(c);
    void* p = nullptr;
    if (g_capturing && (it == g_pool.free_lists.end() || it->second.empty()))
        return fail(DRHIP_EINVAL, "drhip_malloc", "would call hipMalloc while capturing a graph");
    if (it != g_pool.free_lists.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        g_pool.st.bytes_cached -= c;
        g_pool.st.n_pool_hits++;
    } else {
        hipError_t e = hipMalloc(&p, c);
        if (e != hipSuccess) {
            // Out of memory with blocks parked in the pool: release them and retry once.
            (void)hipGetLastError();
            if (drhip_pool_trim() != 0) return (int)e;
            e = hipMalloc(&p, c);
            if (e != hipSuccess) return fail((int)e, "hipMalloc", hipGetErrorString(e));
        }
        g_pool.st.n_driver_allocs++;
    }
    g_pool.live[p] = c;
    g_pool.st.bytes_in_use += c;
    const uint64_t tot = g_pool.st.bytes_in_use + g_pool.st.bytes_cached;
    if (tot > g_pool.st.bytes_peak) g_pool.st.bytes_peak = tot;
    *dptr = p;
    return 0;
}

int drhip_free(void* dptr) {
    if (!dptr) return 0;
    NEED_INIT();
    POOL_LOCK();
    auto it = g_pool.live.find(dptr);
    if (it == g_pool.live.end())
        return fail(DRHIP_EINVAL, "drhip_free", "pointer was not returned by drhip_malloc");
    const size_t c = it->second;
    g_pool.live.erase(it);
    g_pool.free_lists[c].push_back(dptr);
    g_pool.st.bytes_in_use -= c;
    g_pool.st.bytes_cached += c;
    return 0;
}

int drhip_pool_stats(drhip_pool_stats_t* out) {
    if (!out) return fail(DRHIP_EINVAL, "drhip_pool_stats", "null out");
    POOL_LOCK();
    *out = g_pool.st;
    return 0;
}

int drhip_pool_trim(void) {
    NEED_INIT();
    POOL_LOCK();
    HIP_TRY(hipStreamSynchronize(g_stream));
    for (auto& kv : g_pool.free_lists) {
        for (void* p : kv.second) {
            HIP_TRY(hipFree(p));
            g_pool.st.bytes_cached -= kv.first;
        }
        kv.second.clear();
    }
    return 0;
}

// ---- copies ----------------------------------------------------------------

int drhip_memcpy_h2d(void* dst, const void* src, size_t n) {
    NEED_INIT();
    if (g_capturing) return fail(DRHIP_EINVAL, "drhip_memcpy_h2d", "not allowed while capturing a graph");
    if (n == 0) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, g_stream));
    // pageable source: the caller may reuse it as soon as we return
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int drhip_memcpy_d2h(void* dst, const void* src, size_t n) {
    NEED_INIT();
    if (g_capturing) return fail(DRHIP_EINVAL, "drhip_memcpy_d2h", "not allowed while capturing a graph");
    if (n == 0) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, g_stream));
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int drhip_memcpy_d2d(void* dst, const void* src, size_t n) {
    NEED_INIT();
    if (g_capturing) return fail(DRHIP_EINVAL, "drhip_memcpy_d2d", "not allowed while capturing a graph");
    if (n == 0) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, g_stream));
    return 0;
}

int drhip_fill32(void* dst, uint32_t pattern, size_t nwords) {
    NEED_INIT();
    if (nwords == 0) return 0;
    if ((uintptr_t)dst % 4) return fail(DRHIP_EINVAL, "drhip_fill32", "dst not 4-byte aligned");
    drhip_k_launch_fill32(dst, pattern, nwords, g_stream);
    HIP_TRY(hipGetLastError());
    g_cnt.n_launches++;
    return 0;
}

int drhip_fill64(void* dst, uint64_t pattern, size_t nwords) {
    NEED_INIT();
    if (nwords == 0) return 0;
    if ((uintptr_t)dst % 8) return fail(DRHIP_EINVAL, "drhip_fill64", "dst not 8-byte aligned");
    drhip_k_launch_fill64(dst, pattern, nwords, g_stream);
    HIP_TRY(hipGetLastError());
    g_cnt.n_launches++;
    return 0;
}

int drhip_copy_kernel(void* dst, const void* src, size_t nbytes, unsigned grid) {
    NEED_INIT();
    if (nbytes % 16 || (uintptr_t)dst % 16 || (uintptr_t)src % 16)
        return fail(DRHIP_EINVAL, "drhip_copy_kernel", "size and pointers must be multiples of 16");
    if (nbytes == 0) return 0;
    if (grid == 0) {  // one run of 256 vectors per block
        size_t runs = nbytes / 16 / 256;
        if (runs == 0) runs = 1;
        grid = (unsigned)(runs < (size_t(1) << 23) ? runs : (size_t(1) << 23));
    }
    drhip_k_launch_copy(dst, src, nbytes / 16, grid, g_stream);
    HIP_TRY(hipGetLastError());
    g_cnt.n_launches++;
    return 0;
}

int drhip_matmul(int is_double, const void* a, const void* b, void* c, int64_t m, int64_t n,
                 int64_t k, int64_t lda, int64_t ldb, int64_t ldc) {
    NEED_INIT();
    if (!a || !b || !c) return fail(DRHIP_EINVAL, "drhip_matmul", "null operand");
    if (m < 0 || n < 0 || k < 0 || lda < k || ldb < n || ldc < n)
        return fail(DRHIP_EINVAL, "drhip_matmul", "bad dimensions");
    if (m == 0 || n == 0) return 0;
    // the launch counts 64-row tiles in the grid's second dimension (at most 65535):
    // taller products go in slabs of rows
    const int64_t slab = 65535LL * 64;
    const size_t item = is_double ? sizeof(double) : sizeof(float);
    for (int64_t r0 = 0; r0 < m; r0 += slab) {
        const int64_t rows = m - r0 < slab ? m - r0 : slab;
        drhip_k_launch_matmul(is_double, (const char*)a + (size_t)r0 * lda * item, b,
                              (char*)c + (size_t)r0 * ldc * item, rows, n, k, lda, ldb, ldc, g_stream);
        HIP_TRY(hipGetLastError());
        g_cnt.n_launches++;
    }
    return 0;
}

int drhip_cumsum(int kind, const void* in, void* out, size_t n) {
    NEED_INIT();
    if (kind < 0 || kind > 3) return fail(DRHIP_EINVAL, "drhip_cumsum", "kind must be 0..3");
    if (n == 0) return 0;
    if (!in || !out) return fail(DRHIP_EINVAL, "drhip_cumsum", "null operand");
    if (n > (size_t)0x7fffffff) return fail(DRHIP_EINVAL, "drhip_cumsum", "more than 2^31-1 elements");
    size_t bytes = 0;
    int rc = drhip_k_cumsum(kind, nullptr, &bytes, in, out, n, g_stream);
    if (rc) return fail(rc, "hipcub::DeviceScan (size query)", hipGetErrorString((hipError_t)rc));
    void* temp = nullptr;
    rc = drhip_malloc(&temp, bytes ? bytes : 1);
    if (rc) return rc;
    rc = drhip_k_cumsum(kind, temp, &bytes, in, out, n, g_stream);
    drhip_free(temp);  // stream-ordered reuse
    if (rc) return fail(rc, "hipcub::DeviceScan", hipGetErrorString((hipError_t)rc));
    g_cnt.n_launches++;
    return 0;
}

// ---- compile / load --------------------------------------------------------

int drhip_compile(const char* src, const char* name, const char* const* opts, int nopts,
                  void** module) {
    if (!src) return fail(DRHIP_EINVAL, "drhip_compile", "null source");
    if (module && !g_init) return fail(DRHIP_ENOTINIT, "drhip_compile", "loading a module needs drhip_init");
    t_log.clear();
    t_code.clear();
    hiprtcProgram prog = nullptr;
    hiprtcResult r = hiprtcCreateProgram(&prog, src, name ? name : "dr_kernel.hip", 0, nullptr, nullptr);
    if (r != HIPRTC_SUCCESS) return fail(DRHIP_ERTC + (int)r, "hiprtcCreateProgram", hiprtcGetErrorString(r));

    std::string arch = "--offload-arch=";
    if (const char* env = getenv("DRHIP_ARCH")) arch += env;
    else if (g_init) arch += g_arch;
    else arch += "gfx950";
    std::vector<const char*> o;
    o.push_back(arch.c_str());
    for (int i = 0; i < nopts; i++) o.push_back(opts[i]);

    const auto t0 = std::chrono::steady_clock::now();
    r = hiprtcCompileProgram(prog, (int)o.size(), o.data());
    const auto t1 = std::chrono::steady_clock::now();
    g_cnt.compile_ns += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(t1 - t0).count();
    g_cnt.n_compiles++;

    size_t ls = 0;
    if (hiprtcGetProgramLogSize(prog, &ls) == HIPRTC_SUCCESS && ls > 1) {
        t_log.resize(ls);
        hiprtcGetProgramLog(prog, &t_log[0]);
        while (!t_log.empty() && t_log.back() == '\0') t_log.pop_back();
    }
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail(DRHIP_ERTC + (int)r, "hiprtcCompileProgram", hiprtcGetErrorString(r));
    }
    size_t cs = 0;
    r = hiprtcGetCodeSize(prog, &cs);
    if (r == HIPRTC_SUCCESS) {
        t_code.resize(cs);
        r = hiprtcGetCode(prog, t_code.data());
    }
    hiprtcDestroyProgram(&prog);
    if (r != HIPRTC_SUCCESS) return fail(DRHIP_ERTC + (int)r, "hiprtcGetCode", hiprtcGetErrorString(r));
    if (module) return drhip_load_code(t_code.data(), t_code.size(), module);
    return 0;
}

int drhip_code_get(const void** code, size_t* nbytes) {
    if (!code || !nbytes) return fail(DRHIP_EINVAL, "drhip_code_get", "null out");
    if (t_code.empty()) return fail(DRHIP_EINVAL, "drhip_code_get", "no compiled code on this thread");
    *code = t_code.data();
    *nbytes = t_code.size();
    return 0;
}

int drhip_load_code(const void* code, size_t nbytes, void** module) {
    NEED_INIT();
    if (!code || !nbytes || !module) return fail(DRHIP_EINVAL, "drhip_load_code", "null argument");
    hipModule_t m = nullptr;
    HIP_TRY(hipModuleLoadData(&m, code));
    g_cnt.n_code_loads++;
    *module = (void*)m;
    return 0;
}

int drhip_module_unload(void* module) {
    NEED_INIT();
    if (!module) return 0;
    HIP_TRY(hipModuleUnload((hipModule_t)module));
    return 0;
}

int drhip_get_function(void* module, const char* kernel_name, void** func) {
    NEED_INIT();
    if (!module || !kernel_name || !func) return fail(DRHIP_EINVAL, "drhip_get_function", "null argument");
    hipFunction_t f = nullptr;
    HIP_TRY(hipModuleGetFunction(&f, (hipModule_t)module, kernel_name));
    *func = (void*)f;
    return 0;
}

// ---- launch ----------------------------------------------------------------

int drhip_launch(void* func, unsigned grid_x, unsigned block_x, unsigned lds_bytes,
                 const void* args, size_t args_bytes) {
    NEED_INIT();
    if (!func) return fail(DRHIP_EINVAL, "drhip_launch", "null function");
    if (grid_x == 0 || block_x == 0 || block_x > 1024)
        return fail(DRHIP_EINVAL, "drhip_launch", "bad launch geometry");
    if (lds_bytes > (unsigned)g_prop.sharedMemPerBlock)
        return fail(DRHIP_EINVAL, "drhip_launch", "LDS request exceeds the per-workgroup limit");
    size_t sz = args_bytes;
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(args),
                     HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
    HIP_TRY(hipModuleLaunchKernel((hipFunction_t)func, grid_x, 1, 1, block_x, 1, 1, lds_bytes,
                                  g_stream, nullptr, extra));
    g_cnt.n_launches++;
    return 0;
}

size_t drhip_scratch_bytes(void) { return drhip_k_scratch_bytes(); }

int drhip_launch_scratch(void* func, unsigned grid_x, unsigned block_x, unsigned lds_bytes,
                         const void* args, size_t args_bytes, size_t scratch_arg_offset,
                         size_t scratch_bytes) {
    NEED_INIT();
    unsigned char block[DRHIP_MAX_ARGS_BYTES];
    if (!args || args_bytes > sizeof block)
        return fail(DRHIP_EINVAL, "drhip_launch_scratch", "argument block missing or larger than DRHIP_MAX_ARGS_BYTES");
    // (compared without adding to the offset: an offset close to SIZE_MAX must not wrap)
    if (scratch_arg_offset % sizeof(void*) || args_bytes < sizeof(void*) ||
        scratch_arg_offset > args_bytes - sizeof(void*))
        return fail(DRHIP_EINVAL, "drhip_launch_scratch", "scratch pointer slot outside the argument block or misaligned");
    if (scratch_bytes > drhip_k_scratch_bytes())
        return fail(DRHIP_EINVAL, "drhip_launch_scratch", "request exceeds the static scratch array (drhip_scratch_bytes())");
    void* ptr = drhip_k_scratch_ptr(g_device);
    if (!ptr) return fail(DRHIP_ENOTINIT, "drhip_launch_scratch", "scratch address was not resolved");
    memcpy(block, args, args_bytes);
    memcpy(block + scratch_arg_offset, &ptr, sizeof ptr);
    return drhip_launch(func, grid_x, block_x, lds_bytes, block, args_bytes);
}

// ---- graphs ----------------------------------------------------------------

int drhip_graph_begin(void) {
    NEED_INIT();
    if (g_capturing) return fail(DRHIP_EINVAL, "drhip_graph_begin", "a capture is already open");
    HIP_TRY(hipStreamBeginCapture(g_stream, hipStreamCaptureModeThreadLocal));
    g_capturing = true;
    return 0;
}

int drhip_graph_end(void** graph_exec) {
    NEED_INIT();
    if (!g_capturing) return fail(DRHIP_EINVAL, "drhip_graph_end", "no capture is open");
    g_capturing = false;
    hipGraph_t graph = nullptr;
    HIP_TRY(hipStreamEndCapture(g_stream, &graph));
    if (!graph_exec) {
        (void)hipGraphDestroy(graph);
        return fail(DRHIP_EINVAL, "drhip_graph_end", "null out");
    }
    hipGraphExec_t exec = nullptr;
    hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail((int)e, "hipGraphInstantiate", hipGetErrorString(e));
    *graph_exec = (void*)exec;
    return 0;
}

int drhip_graph_launch(void* graph_exec) {
    NEED_INIT();
    if (!graph_exec) return fail(DRHIP_EINVAL, "drhip_graph_launch", "null graph");
    HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, g_stream));
    g_cnt.n_launches++;
    return 0;
}

int drhip_graph_destroy(void* graph_exec) {
    NEED_INIT();
    if (!graph_exec) return 0;
    HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
    return 0;
}

// ---- sync / events ---------------------------------------------------------

int drhip_sync(void) {
    NEED_INIT();
    if (g_capturing) return fail(DRHIP_EINVAL, "drhip_sync", "not allowed while capturing a graph");
    HIP_TRY(hipStreamSynchronize(g_stream));
    return 0;
}

int drhip_event_create(void** ev) {
    NEED_INIT();
    if (!ev) return fail(DRHIP_EINVAL, "drhip_event_create", "null out");
    hipEvent_t e;
    HIP_TRY(hipEventCreate(&e));
    *ev = (void*)e;
    return 0;
}

int drhip_event_destroy(void* ev) {
    NEED_INIT();
    if (!ev) return 0;
    HIP_TRY(hipEventDestroy((hipEvent_t)ev));
    return 0;
}

int drhip_event_record(void* ev) {
    NEED_INIT();
    HIP_TRY(hipEventRecord((hipEvent_t)ev, g_stream));
    return 0;
}

int drhip_event_sync(void* ev) {
    NEED_INIT();
    HIP_TRY(hipEventSynchronize((hipEvent_t)ev));
    return 0;
}

int drhip_event_elapsed_ms(void* start, void* stop, float* ms) {
    NEED_INIT();
    if (!ms) return fail(DRHIP_EINVAL, "drhip_event_elapsed_ms", "null out");
    HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

int drhip_counters(drhip_counters_t* out) {
    if (!out) return fail(DRHIP_EINVAL, "drhip_counters", "null out");
    *out = g_cnt;
    return 0;
}

}  // extern "C"
