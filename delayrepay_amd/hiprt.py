"""ctypes binding of libdrhip.so (C ABI: include/drhip.h).

This is the only module that talks to the device.  It plays the part CuPy's
runtime plays under the reference's GPU backend (delayrepay/cuda.py:17,38,96):
device memory, run-time compilation, launch, copies.  There is no host
fall-back: if the library is not built, or no GPU answers, every entry point
raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdrhip.so")


class DrhipError(RuntimeError):
    """A libdrhip call returned a non-zero code."""

    def __init__(self, code, msg, log=""):
        super().__init__(f"[drhip {code}] {msg}" + (f"\n{log}" if log else ""))
        self.code = code
        self.log = log


class DeviceInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("max_lds_bytes", C.c_int32),
        ("l2_bytes", C.c_int32),
        ("total_mem", C.c_int64),
        ("clock_khz", C.c_int32),
        ("mem_clock_khz", C.c_int32),
        ("mem_bus_bits", C.c_int32),
        ("hiprtc_version", C.c_int32),
    ]


class PoolStats(C.Structure):
    _fields_ = [
        ("bytes_in_use", C.c_uint64),
        ("bytes_cached", C.c_uint64),
        ("bytes_peak", C.c_uint64),
        ("n_driver_allocs", C.c_uint64),
        ("n_pool_hits", C.c_uint64),
        ("n_mallocs", C.c_uint64),
    ]


class Counters(C.Structure):
    _fields_ = [
        ("n_compiles", C.c_uint64),
        ("n_code_loads", C.c_uint64),
        ("n_launches", C.c_uint64),
        ("compile_ns", C.c_uint64),
    ]


# name -> (restype, argtypes); every symbol include/drhip.h declares
_SIGNATURES = {
    "drhip_init": (C.c_int, [C.c_int]),
    "drhip_device_info_get": (C.c_int, [C.POINTER(DeviceInfo)]),
    "drhip_last_error": (C.c_char_p, []),
    "drhip_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "drhip_free": (C.c_int, [C.c_void_p]),
    "drhip_pool_stats": (C.c_int, [C.POINTER(PoolStats)]),
    "drhip_pool_trim": (C.c_int, []),
    "drhip_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "drhip_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "drhip_memcpy_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "drhip_fill32": (C.c_int, [C.c_void_p, C.c_uint32, C.c_size_t]),
    "drhip_fill64": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t]),
    "drhip_copy_kernel": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint]),
    "drhip_matmul": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int64] * 6),
    "drhip_cumsum": (C.c_int, [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]),
    "drhip_compile": (C.c_int, [C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_int,
                                C.POINTER(C.c_void_p)]),
    "drhip_code_get": (C.c_int, [C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]),
    "drhip_load_code": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "drhip_module_unload": (C.c_int, [C.c_void_p]),
    "drhip_get_function": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "drhip_compile_log": (C.c_char_p, []),
    "drhip_launch": (C.c_int, [C.c_void_p, C.c_uint, C.c_uint, C.c_uint, C.c_void_p, C.c_size_t]),
    "drhip_launch_scratch": (C.c_int, [C.c_void_p, C.c_uint, C.c_uint, C.c_uint, C.c_void_p,
                                       C.c_size_t, C.c_size_t, C.c_size_t]),
    "drhip_scratch_bytes": (C.c_size_t, []),
    "drhip_graph_begin": (C.c_int, []),
    "drhip_graph_end": (C.c_int, [C.POINTER(C.c_void_p)]),
    "drhip_graph_launch": (C.c_int, [C.c_void_p]),
    "drhip_graph_destroy": (C.c_int, [C.c_void_p]),
    "drhip_sync": (C.c_int, []),
    "drhip_event_create": (C.c_int, [C.POINTER(C.c_void_p)]),
    "drhip_event_destroy": (C.c_int, [C.c_void_p]),
    "drhip_event_record": (C.c_int, [C.c_void_p]),
    "drhip_event_sync": (C.c_int, [C.c_void_p]),
    "drhip_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "drhip_counters": (C.c_int, [C.POINTER(Counters)]),
}

_lib = None
_initialised = False


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {_HERE}/csrc` "
                "(or __graft_entry__.build()); the HIP backend has no host fall-back")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def _check(code):
    if code != 0:
        l = lib()
        msg = (l.drhip_last_error() or b"").decode(errors="replace")
        log = ""
        if code >= 10000 and code < 20000:
            log = (l.drhip_compile_log() or b"").decode(errors="replace")
        raise DrhipError(code, msg, log)


def init(device=None):
    """Initialise the device once; later calls are free."""
    global _initialised
    if _initialised:
        return
    if device is None:
        device = int(os.environ.get("DRHIP_DEVICE", "0"))
    _check(lib().drhip_init(device))
    _initialised = True


def device_info():
    init()
    info = DeviceInfo()
    _check(lib().drhip_device_info_get(C.byref(info)))
    return {f: (getattr(info, f).decode() if isinstance(getattr(info, f), bytes) else getattr(info, f))
            for f, _ in DeviceInfo._fields_}


def malloc(nbytes):
    p = C.c_void_p()
    _check(_lib.drhip_malloc(C.byref(p), nbytes))
    return p.value


def free(ptr):
    # called from finalisers: never raise during interpreter shutdown
    lib_ = _lib
    if lib_ is not None and ptr:
        lib_.drhip_free(ptr)


def pool_stats():
    st = PoolStats()
    _check(lib().drhip_pool_stats(C.byref(st)))
    return {f: getattr(st, f) for f, _ in PoolStats._fields_}


def pool_trim():
    _check(lib().drhip_pool_trim())


def memcpy_h2d(dst, host_ptr, nbytes):
    _check(_lib.drhip_memcpy_h2d(dst, host_ptr, nbytes))


def memcpy_d2h(host_ptr, src, nbytes):
    _check(_lib.drhip_memcpy_d2h(host_ptr, src, nbytes))


def memcpy_d2d(dst, src, nbytes):
    _check(_lib.drhip_memcpy_d2d(dst, src, nbytes))


def fill32(dst, pattern, nwords):
    _check(_lib.drhip_fill32(dst, pattern, nwords))


def fill64(dst, pattern, nwords):
    _check(_lib.drhip_fill64(dst, pattern, nwords))


def copy_kernel(dst, src, nbytes, grid_blocks=0):
    _check(_lib.drhip_copy_kernel(dst, src, nbytes, grid_blocks))


def matmul(is_double, a, b, c, m, n, k, lda, ldb, ldc):
    _check(_lib.drhip_matmul(int(is_double), a, b, c, m, n, k, lda, ldb, ldc))


def cumsum(kind, src, dst, n):
    _check(_lib.drhip_cumsum(kind, src, dst, n))


def _opts_array(opts):
    arr = (C.c_char_p * len(opts))(*[o.encode() for o in opts])
    return arr, len(opts)


def compile_only(src, name, opts):
    """Compile without loading (works on a machine with no GPU); returns the code object."""
    arr, n = _opts_array(opts)
    _check(lib().drhip_compile(src.encode(), name.encode(), arr, n, None))
    code = C.c_void_p()
    size = C.c_size_t()
    _check(lib().drhip_code_get(C.byref(code), C.byref(size)))
    return C.string_at(code.value, size.value)


def compile_module(src, name, opts):
    """Compile and load; returns (module handle, code object bytes)."""
    init()
    arr, n = _opts_array(opts)
    mod = C.c_void_p()
    _check(_lib.drhip_compile(src.encode(), name.encode(), arr, n, C.byref(mod)))
    code = C.c_void_p()
    size = C.c_size_t()
    _check(_lib.drhip_code_get(C.byref(code), C.byref(size)))
    return mod.value, C.string_at(code.value, size.value)


def load_code(code_bytes):
    init()
    mod = C.c_void_p()
    _check(_lib.drhip_load_code(code_bytes, len(code_bytes), C.byref(mod)))
    return mod.value


def get_function(module, name):
    fn = C.c_void_p()
    _check(_lib.drhip_get_function(module, name.encode(), C.byref(fn)))
    return fn.value


def compile_log():
    return (lib().drhip_compile_log() or b"").decode(errors="replace")


def launch(func, grid, block, lds_bytes, argbuf, nbytes):
    rc = _lib.drhip_launch(func, grid, block, lds_bytes, argbuf, nbytes)
    if rc:
        _check(rc)


def launch_scratch(func, grid, block, lds_bytes, argbuf, nbytes, slot_offset, scratch_bytes):
    """`launch` with the library's static scratch array in the pointer slot at
    `slot_offset` of the argument block; allocates nothing."""
    rc = _lib.drhip_launch_scratch(func, grid, block, lds_bytes, argbuf, nbytes, slot_offset,
                                   scratch_bytes)
    if rc:
        _check(rc)


def scratch_bytes():
    return lib().drhip_scratch_bytes()


def sync():
    _check(lib().drhip_sync())


class Graph:
    """Instantiated HIP graph of the launches issued inside `with Graph.capture()`."""

    def __init__(self, handle):
        self.h = handle

    @staticmethod
    def begin():
        init()
        _check(_lib.drhip_graph_begin())

    @staticmethod
    def end():
        h = C.c_void_p()
        _check(_lib.drhip_graph_end(C.byref(h)))
        return Graph(h.value)

    def launch(self):
        _check(_lib.drhip_graph_launch(self.h))

    def __del__(self):
        if _lib is not None and self.h:
            _lib.drhip_graph_destroy(self.h)
            self.h = None


class Event:
    """A hipEvent recorded on the library stream."""

    __slots__ = ("h",)

    def __init__(self):
        init()
        h = C.c_void_p()
        _check(_lib.drhip_event_create(C.byref(h)))
        self.h = h.value

    def record(self):
        _check(_lib.drhip_event_record(self.h))
        return self

    def synchronize(self):
        _check(_lib.drhip_event_sync(self.h))

    def elapsed_ms(self, later):
        ms = C.c_float()
        _check(_lib.drhip_event_elapsed_ms(self.h, later.h, C.byref(ms)))
        return ms.value

    def __del__(self):
        if _lib is not None and self.h:
            _lib.drhip_event_destroy(self.h)
            self.h = None


def counters():
    c = Counters()
    _check(lib().drhip_counters(C.byref(c)))
    return {f: getattr(c, f) for f, _ in Counters._fields_}
