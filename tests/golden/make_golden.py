"""Writes the golden fixtures in this directory.

The vectors come from NumPy and SciPy alone (the libraries the reference's CPU
backend evaluates with, delayrepay/cpu.py:19-26); nothing of the reference is
imported or run.  Each expression is written out operation by operation, in the
order the front end's rewrites produce (delayrepay/delayarray.py:316-336).

    python tests/golden/make_golden.py
"""
import os

import numpy as np
from scipy.special import erf, erfc

HERE = os.path.dirname(os.path.abspath(__file__))
INV_SQRT2 = 0.7071067811865476


def configs(n=1024):
    out = {}
    rs = np.random.RandomState(0)
    x = rs.uniform(-1, 1, n).astype(np.float32)
    y = rs.uniform(-1, 1, n).astype(np.float32)
    out["saxpy_x"], out["saxpy_y"] = x, y
    out["saxpy_z"] = np.float32(2.0) * x + y

    rs = np.random.RandomState(0)
    c = rs.uniform(-1, 1, 9).astype(np.float32)
    x = rs.uniform(-2, 2, n).astype(np.float32)
    acc = c[8] * x + c[7]
    for i in range(6, -1, -1):
        acc = acc * x + c[i]
    out["horner_c"], out["horner_x"], out["horner_y"] = c, x, acc

    for tag, dt in (("bs64", np.float64), ("bs32", np.float32)):
        rs = np.random.RandomState(0)
        S = rs.uniform(5, 30, n).astype(dt)
        K = rs.uniform(1, 100, n).astype(dt)
        T = rs.uniform(0.25, 10, n).astype(dt)
        r, sigma = 0.02, 0.30
        sqT = np.sqrt(T)
        vs = sigma * sqT
        d1 = (np.log(S / K) + (r + 0.5 * sigma * sigma) * T) / vs
        d2 = d1 - vs
        N1 = 0.5 * (1 + erf(d1 * INV_SQRT2))
        N2 = 0.5 * (1 + erf(d2 * INV_SQRT2))
        disc = K * np.exp((-r) * T)
        out[tag + "_S"], out[tag + "_K"], out[tag + "_T"] = S, K, T
        out[tag + "_call"] = S * N1 - disc * N2
        out[tag + "_put"] = disc * (1 - N2) - S * (1 - N1)
        assert out[tag + "_call"].dtype == dt

    rs = np.random.RandomState(0)
    u = np.zeros((34, 50), np.float32)
    u[1:-1, 1:-1] = rs.uniform(0, 1, (32, 48))
    out["jacobi_u0"] = u.copy()
    for sweep in range(1, 11):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        if sweep in (1, 10):
            out[f"jacobi_u{sweep}"] = u.copy()

    rs = np.random.RandomState(0)
    x = rs.standard_normal(4 * n)
    y = rs.standard_normal(4 * n)
    w = rs.uniform(0, 1, 4 * n)
    d = x - y
    out["sumsq_x"], out["sumsq_y"], out["sumsq_w"] = x, y, w
    out["sumsq_s"] = np.sum(d * d * w)
    return out


UNARY = {
    "negative": np.negative, "absolute": np.absolute, "sin": np.sin, "cos": np.cos, "tan": np.tan,
    "arcsin": np.arcsin, "arccos": np.arccos, "arctan": np.arctan, "sinh": np.sinh,
    "cosh": np.cosh, "tanh": np.tanh, "exp": np.exp, "exp2": np.exp2, "expm1": np.expm1,
    "log": np.log, "log2": np.log2, "log10": np.log10, "log1p": np.log1p, "sqrt": np.sqrt,
    "cbrt": np.cbrt, "erf": erf, "erfc": erfc, "floor": np.floor, "ceil": np.ceil,
    "trunc": np.trunc, "rint": np.rint, "reciprocal": np.reciprocal,
}
BINARY = {
    "add": np.add, "subtract": np.subtract, "multiply": np.multiply, "divide": np.divide,
    "power": np.power, "arctan2": np.arctan2, "hypot": np.hypot, "maximum": np.maximum,
    "minimum": np.minimum, "fmax": np.fmax, "fmin": np.fmin, "copysign": np.copysign,
    "fmod": np.fmod,
}


def special_values():
    """Every mapped function on a table of special and ordinary arguments."""
    out = {}
    for tag, dt in (("f32", np.float32), ("f64", np.float64)):
        fi = np.finfo(dt)
        base = [0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 2.0, -2.0, 3.5, -3.5, 1e-3, -1e-3, 10.0, -10.0,
                88.0, -88.0, 700.0, -700.0, np.pi, -np.pi, np.e, 0.1, 0.9999999, 1.0000001,
                fi.tiny, -fi.tiny, fi.tiny / 8, -fi.tiny / 8, fi.max, -fi.max, fi.eps,
                np.inf, -np.inf, np.nan, 1e10, -1e10, 2.5, -2.5, 1.5, -1.5]
        rs = np.random.RandomState(1)
        x = np.concatenate([np.array(base, dtype=dt),
                            rs.uniform(-4, 4, 88).astype(dt)])
        y = np.concatenate([np.array(base[::-1], dtype=dt),
                            rs.uniform(-4, 4, 88).astype(dt)])
        out[f"{tag}_x"], out[f"{tag}_y"] = x, y
        with np.errstate(all="ignore"):
            for name, fn in UNARY.items():
                out[f"{tag}_{name}"] = fn(x)
            for name, fn in BINARY.items():
                out[f"{tag}_{name}"] = fn(x, y)
    return out


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "configs_small.npz"), **configs())
    np.savez_compressed(os.path.join(HERE, "special_values.npz"), **special_values())
    for name in ("configs_small.npz", "special_values.npz"):
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")
