"""Shared test helpers: ulp distance, the C oracle binding, golden fixtures."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def golden(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def ulp_distance(a, b):
    """Distance in units in the last place between same-dtype float arrays
    (0 where both are NaN or both the same infinity)."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == b.dtype and a.dtype.kind == "f"
    itype = np.int32 if a.dtype.itemsize == 4 else np.int64
    ia = a.view(itype).astype(np.int64)
    ib = b.view(itype).astype(np.int64)
    top = np.int64(np.iinfo(itype).min)
    ia = np.where(ia < 0, top - ia, ia)   # map to a monotone integer line
    ib = np.where(ib < 0, top - ib, ib)
    dist = np.abs(ia - ib).astype(np.float64)
    both_nan = np.isnan(a) & np.isnan(b)
    one_nan = np.isnan(a) ^ np.isnan(b)
    dist = np.where(both_nan, 0.0, dist)
    dist = np.where(one_nan, np.inf, dist)
    return dist


def bits_equal(a, b):
    """Same dtype, shape and bit patterns.  NaNs must sit at the same positions, but
    their sign and payload are not compared: IEEE 754 leaves both unspecified for
    invalid operations (x86 SSE returns the negative quiet NaN, gfx950 the positive)."""
    a = np.asarray(a)
    b = np.asarray(b)
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    if a.dtype.kind == "f":
        na, nb = np.isnan(a), np.isnan(b)
        if na.any() or nb.any():
            if not np.array_equal(na, nb):
                return False
            a, b = np.where(na, 0, a), np.where(nb, 0, b)
    return a.tobytes() == b.tobytes()


_C_ORACLE = None


def c_oracle():
    """ctypes handle of oracle/libdr_oracle.so (built on demand with gcc)."""
    global _C_ORACLE
    if _C_ORACLE is None:
        path = os.path.join(ROOT, "oracle", "libdr_oracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True)
        lib = ctypes.CDLL(path)
        f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
        f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
        lib.dro_saxpy_f32.argtypes = [ctypes.c_float, f32p, f32p, f32p, ctypes.c_size_t]
        lib.dro_horner_f32.argtypes = [f32p, ctypes.c_int, f32p, f32p, ctypes.c_size_t]
        lib.dro_jacobi_sweep_f32.argtypes = [f32p, f32p, ctypes.c_size_t, ctypes.c_size_t]
        lib.dro_black_scholes_f64.argtypes = [f64p, f64p, f64p, ctypes.c_double, ctypes.c_double,
                                              f64p, f64p, ctypes.c_size_t]
        lib.dro_sumsq_terms_f64.argtypes = [f64p, f64p, f64p, f64p, ctypes.c_size_t]
        for fn in (lib.dro_saxpy_f32, lib.dro_horner_f32, lib.dro_jacobi_sweep_f32,
                   lib.dro_black_scholes_f64, lib.dro_sumsq_terms_f64):
            fn.restype = None
        _C_ORACLE = lib
    return _C_ORACLE
