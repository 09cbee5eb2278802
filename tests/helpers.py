"""Shared test helpers: ulp distance, the C oracle binding, golden fixtures."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def golden(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


from oracle.accuracy import ulp_distance  # noqa: E402,F401


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
