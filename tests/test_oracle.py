"""Pins the NumPy oracle (oracle/numpy_oracle.py) before anything is compared with it.

The reference ships no golden vectors (its tests compare a backend with NumPy at
six decimals on 64 elements), so the oracle is pinned by:
  * the reference's own test expressions against closed-form answers;
  * an independent C restatement (oracle/dr_oracle.c), bit-exact for + - * /;
  * what the mathematics fixes: put-call parity, mpmath at 50 digits, Jacobi
    invariants and a pure-Python loop, math.fsum for the reduction;
  * the committed fixtures in tests/golden (generated from NumPy/SciPy alone).
"""
import math

import numpy as np
import pytest

from oracle import numpy_oracle as orc
from oracle.numpy_oracle import OracleArray
from tests.helpers import bits_equal, c_oracle, golden, ulp_distance

SIZE = 64


# ---- the reference's test expressions (tests/test.py) against closed forms ----

def test_reference_elementwise_cases():
    arr = OracleArray(np.ones(SIZE))
    assert np.all((arr + 1).get() == 2.0)                       # test.py:21-23
    assert np.all((arr * 3).get() == 3.0)                       # test.py:25-27
    assert np.all((7 * arr).get() == 7.0)                       # test.py:29-32
    assert np.all((8 * arr + 9).get() == 17.0)                  # test.py:34-38
    assert np.all((arr + arr * 3 + 9).get() == 13.0)            # test.py:40-45
    assert np.all(np.cos(arr).get() == math.cos(1.0))           # test.py:51-53
    assert np.all((arr ** 2).get() == 1.0)                      # test.py:55-57
    a32 = arr.astype(np.float32)                                # test.py:59-62
    assert (a32 ** 2).get().dtype == np.float32
    fused = (np.sin(arr) ** 2 + np.cos(arr) ** 2).get()         # test.py:64-67
    assert np.all(np.abs(fused - 1.0) < 1e-15)


def test_reference_vector_cases():
    a = OracleArray(np.full((SIZE,), 7).astype(np.float32))
    b = OracleArray(np.full((SIZE,), 3).astype(np.float32))
    assert np.all((a + b).get() == 10.0)                        # test.py:79-81
    assert np.all((a * b).get() == 21.0)                        # test.py:83-85
    assert a.sum() == 7.0 * SIZE                                # test.py:102-106
    at = np.arctan2(a, b).get()                                 # test.py:108-111
    assert at.dtype == np.float32
    assert np.all(ulp_distance(at, np.full(SIZE, np.float32(math.atan2(7.0, 3.0)))) <= 1)
    m = OracleArray(np.full((SIZE, SIZE), 7).astype(np.float32))
    assert np.all((m * 3).get() == 21.0)                        # test.py:122-124


def test_power_rewrite_is_left_associated_product():
    rs = np.random.RandomState(3)
    x = rs.uniform(-3, 3, 4096).astype(np.float32)
    cube = (OracleArray(x) ** 3).get()
    assert bits_equal(cube, (x * x) * x)                        # delayarray.py:316-324
    # and it is NOT what numpy.power computes, which is why the rewrite matters
    assert not bits_equal(cube, np.power(x, 3))
    assert bits_equal((OracleArray(x) ** 1).get(), x)
    assert bits_equal(np.square(OracleArray(x)).get(), x * x)   # delayarray.py:330-331
    assert bits_equal((OracleArray(x) ** 2.0).get(), np.power(x, 2.0))  # float exponent: pow


def test_weak_python_scalars_keep_float32():
    x = np.linspace(-1, 1, 257, dtype=np.float32)
    z = (0.3 * OracleArray(x)).get()
    assert z.dtype == np.float32
    assert bits_equal(z, np.float32(0.3) * x)


# ---- bit-exact against the C restatement ---------------------------------------

@pytest.mark.parametrize("n", [1, 7, 1000, 65537])
def test_saxpy_matches_c(n):
    inp = orc.make_inputs("saxpy", n)
    z = np.empty(n, np.float32)
    c_oracle().dro_saxpy_f32(inp["a"], inp["x"], inp["y"], z, n)
    assert bits_equal(orc.saxpy(inp["a"], inp["x"], inp["y"]), z)
    assert bits_equal((inp["a"] * OracleArray(inp["x"]) + OracleArray(inp["y"])).get(), z)


@pytest.mark.parametrize("n", [1, 1000, 65537])
def test_horner_matches_c(n):
    inp = orc.make_inputs("horner", n)
    y = np.empty(n, np.float32)
    c_oracle().dro_horner_f32(np.array(inp["c"], np.float32), 8, inp["x"], y, n)
    assert bits_equal(orc.horner(inp["c"], inp["x"]), y)
    x = OracleArray(inp["x"])
    c = inp["c"]
    acc = c[8] * x + c[7]
    for i in range(6, -1, -1):
        acc = acc * x + c[i]
    assert bits_equal(acc.get(), y)


def test_horner_against_exact_rational_arithmetic():
    """Closed form: the float32 Horner value is within a few ulp-of-the-largest-term
    of the exactly evaluated polynomial."""
    from fractions import Fraction
    inp = orc.make_inputs("horner", 64)
    y = orc.horner(inp["c"], inp["x"])
    for xi, yi in zip(inp["x"][:16], y[:16]):
        exact = Fraction(0)
        for c in reversed(inp["c"]):
            exact = exact * Fraction(float(xi)) + Fraction(c)
        mag = sum(abs(c) * abs(float(xi)) ** k for k, c in enumerate(inp["c"]))
        assert abs(float(exact) - float(yi)) <= 16 * np.finfo(np.float32).eps * mag


@pytest.mark.parametrize("shape", [(3, 3), (8, 8), (34, 50), (65, 129)])
def test_jacobi_matches_c_and_python_loop(shape):
    rs = np.random.RandomState(5)
    u0 = np.zeros(shape, np.float32)
    u0[1:-1, 1:-1] = rs.uniform(0, 1, (shape[0] - 2, shape[1] - 2))
    got = orc.jacobi(u0, 3)
    a, b = u0.copy(), np.empty_like(u0)
    for _ in range(3):
        c_oracle().dro_jacobi_sweep_f32(a, b, shape[0], shape[1])
        a, b = b, a
    assert bits_equal(got, a)
    if shape[0] <= 8:   # brute force in pure Python, float32 rounding after every operation
        f = np.float32
        cur = u0.copy()
        for _ in range(3):
            nxt = cur.copy()
            for i in range(1, shape[0] - 1):
                for j in range(1, shape[1] - 1):
                    s = f(f(f(cur[i - 1, j] + cur[i + 1, j]) + cur[i, j - 1]) + cur[i, j + 1])
                    nxt[i, j] = f(f(0.25) * s)
            cur = nxt
        assert bits_equal(got, cur)


def test_jacobi_invariants():
    u = np.zeros((40, 56), np.float32)
    u[1:-1, 1:-1] = np.random.RandomState(1).uniform(0, 1, (38, 54))
    out = orc.jacobi(u, 10)
    assert np.all(out[0] == 0) and np.all(out[-1] == 0)          # boundary untouched
    assert np.all(out[:, 0] == 0) and np.all(out[:, -1] == 0)
    assert out.max() <= u.max() and out.min() >= 0               # discrete maximum principle
    const = np.full((20, 20), np.float32(0.75))
    assert bits_equal(orc.jacobi(const, 5), const)               # constant field is a fixed point
    assert np.all(orc.jacobi(u, 0) == u)
    # Jacobi, not Gauss-Seidel: one sweep of a single spike touches only its 4 neighbours
    spike = np.zeros((7, 7), np.float32)
    spike[3, 3] = 1
    one = orc.jacobi(spike, 1)
    assert one[3, 3] == 0 and one[2, 3] == one[4, 3] == one[3, 2] == one[3, 4] == 0.25
    assert np.count_nonzero(one) == 4


# ---- Black-Scholes ---------------------------------------------------------------

def test_black_scholes_put_call_parity():
    inp = orc.make_inputs("bs64", 20000)
    call, put = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    parity = inp["S"] - inp["K"] * np.exp(-inp["r"] * inp["T"])
    assert np.max(np.abs((call - put) - parity) / np.maximum(inp["S"], inp["K"])) < 5e-16
    assert np.all(call >= -1e-12) and np.all(put >= -1e-12)
    assert np.all(call <= inp["S"] + 1e-12)


def test_black_scholes_against_mpmath():
    mpmath = pytest.importorskip("mpmath")
    mpmath.mp.dps = 50
    inp = orc.make_inputs("bs64", 200)
    call, put = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    r, sg = mpmath.mpf(inp["r"]), mpmath.mpf(inp["sigma"])
    for i in range(0, 200, 4):
        S, K, T = (mpmath.mpf(float(inp[k][i])) for k in "SKT")
        vs = sg * mpmath.sqrt(T)
        d1 = (mpmath.log(S / K) + (r + sg * sg / 2) * T) / vs
        d2 = d1 - vs
        N = lambda d: (1 + mpmath.erf(d / mpmath.sqrt(2))) / 2   # noqa: E731
        disc = K * mpmath.exp(-r * T)
        c = S * N(d1) - disc * N(d2)
        p = disc * (1 - N(d2)) - S * (1 - N(d1))
        scale = max(float(S), float(K))
        assert abs(float(c) - call[i]) <= 2e-15 * scale
        assert abs(float(p) - put[i]) <= 2e-15 * scale


def test_black_scholes_matches_c_libm():
    inp = orc.make_inputs("bs64", 5000)
    call, put = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    cc, cp = np.empty(5000), np.empty(5000)
    c_oracle().dro_black_scholes_f64(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"],
                                     cc, cp, 5000)
    scale = np.maximum(inp["S"], inp["K"])
    assert np.max(np.abs(call - cc) / scale) <= 1e-13
    assert np.max(np.abs(put - cp) / scale) <= 1e-13


def test_black_scholes_f32_stays_f32():
    inp = orc.make_inputs("bs32", 1000)
    call, put = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    assert call.dtype == np.float32 and put.dtype == np.float32
    c64, p64 = orc.black_scholes(*(inp[k].astype(np.float64) for k in "SKT"), inp["r"], inp["sigma"])
    scale = np.maximum(inp["S"], inp["K"])
    assert np.max(np.abs(call - c64) / scale) < 1e-6


# ---- fused reduction ---------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 129, 1 << 16, (1 << 20) + 3])
def test_sumsq_against_fsum_and_c_terms(n):
    inp = orc.make_inputs("sumsq", n)
    s = orc.sumsq(inp["x"], inp["y"], inp["w"])
    terms = np.empty(n)
    c_oracle().dro_sumsq_terms_f64(inp["x"], inp["y"], inp["w"], terms, n)
    d = inp["x"] - inp["y"]
    assert bits_equal(terms, d * d * inp["w"])                 # element-wise part bit-exact
    exact = math.fsum(terms.tolist())
    assert abs(s - exact) <= 1e-13 * abs(exact)


# ---- committed fixtures --------------------------------------------------------------

def test_oracle_reproduces_golden_configs():
    g = golden("configs_small.npz")
    assert bits_equal(orc.saxpy(2.0, g["saxpy_x"], g["saxpy_y"]), g["saxpy_z"])
    assert bits_equal(orc.horner([float(c) for c in g["horner_c"]], g["horner_x"]), g["horner_y"])
    for tag in ("bs64", "bs32"):
        call, put = orc.black_scholes(g[tag + "_S"], g[tag + "_K"], g[tag + "_T"], 0.02, 0.30)
        assert bits_equal(call, g[tag + "_call"]) and bits_equal(put, g[tag + "_put"])
    assert bits_equal(orc.jacobi(g["jacobi_u0"], 1), g["jacobi_u1"])
    assert bits_equal(orc.jacobi(g["jacobi_u0"], 10), g["jacobi_u10"])
    assert orc.sumsq(g["sumsq_x"], g["sumsq_y"], g["sumsq_w"]) == g["sumsq_s"]


def test_oracle_array_reproduces_golden_special_values():
    g = golden("special_values.npz")
    from tests.golden.make_golden import UNARY, BINARY
    for tag in ("f32", "f64"):
        x, y = OracleArray(g[f"{tag}_x"]), OracleArray(g[f"{tag}_y"])
        with np.errstate(all="ignore"):
            for name, fn in UNARY.items():
                assert bits_equal(fn(x).get(), g[f"{tag}_{name}"]), name
            for name, fn in BINARY.items():
                assert bits_equal(fn(x, y).get(), g[f"{tag}_{name}"]), name


def test_accuracy_report_measures_what_it_says():
    """oracle/accuracy.py: the 50-digit price agrees with the float64 oracle where nothing
    cancels, the ulp distance counts representable numbers, and a planted error shows up
    at the right index, in the right subset, with the right size."""
    from oracle import accuracy
    inp = orc.make_inputs("bs64", 4096)
    call, put = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    scale = np.maximum(inp["S"], inp["K"])
    for i in np.flatnonzero(call >= 0.25 * scale)[:5]:
        truth = float(accuracy.bs_truth(inp["S"][i], inp["K"][i], inp["T"][i], 0.02, 0.30, "call"))
        assert abs(call[i] - truth) <= 1e-14 * truth
        parity = float(accuracy.bs_truth(inp["S"][i], inp["K"][i], inp["T"][i], 0.02, 0.30, "put"))
        assert abs((truth - parity) - (inp["S"][i] - inp["K"][i] * np.exp(-0.02 * inp["T"][i]))) \
            <= 1e-13 * scale[i]
    one = np.float32(1.0)
    assert accuracy.ulp_distance(np.array([one]), np.array([np.nextafter(one, np.float32(2))]))[0] == 1
    assert accuracy.ulp_distance(np.array([-0.0]), np.array([0.0]))[0] == 0
    assert accuracy.ulp_distance(np.array([np.nan]), np.array([1.0]))[0] == np.inf
    bent = call.copy()
    i = int(np.flatnonzero(call >= 0.5 * scale)[0])
    for _ in range(5):
        bent[i] = np.nextafter(bent[i], np.inf)
    rep = accuracy.bs_report(bent, put, call, put, inp)
    assert rep["call"]["subsets"][1]["max_ulp"] == 5 and rep["call"]["subsets"][1]["max_ulp_index"] == i
    assert rep["call"]["subsets"][1]["max_ulp_at"]["oracle_err_ulp_vs_truth"] < 16
    assert rep["put"]["subsets"][16]["max_ulp"] == 0 and rep["put"]["scaled"]["max_eps"] == 0
    assert "5 ulp" in accuracy.format_report("bs64", rep)


def test_philox_restatement_against_numpy_and_the_published_vectors():
    """oracle/philox.py: known-answer vectors of Philox-4x64-10 (all-zero and all-ones
    counter and key, from the generator's reference distribution), NumPy's generator for
    keys and counters that exercise every word and the carry out of the counter, and the
    53-bit doubles across two calls of one Generator."""
    from oracle import philox
    assert philox.block(0, 0) == [0x16554d9eca36314c, 0xdb20fe9d672d0fdc,
                                  0xd7e772cee186176b, 0x7e68b68aec7ba23b]
    assert philox.block((1 << 256) - 1, (1 << 128) - 1) == [
        0x87b092c3013fe90b, 0x438c3c67be8d0224, 0x9cc7d7c69cd777b6, 0xa09caebf594f0ba0]
    for key, ctr in ((0, 0), (12345, 0), ((1 << 128) - 5, (1 << 256) - 2),
                     (987654321 << 70, 3 << 190), (1, (1 << 64) - 2), (2, (1 << 128) - 1)):
        ref = np.random.Philox(key=key, counter=ctr).random_raw(23)
        assert [int(v) for v in ref] == philox.stream(key, ctr, 23), (key, ctr)
    gen = np.random.Generator(np.random.Philox(key=7))
    drawn = list(gen.random(10)) + list(gen.random(7))          # 17 outputs: not a multiple of 4
    assert drawn == philox.doubles(philox.stream(7, 0, 17))
    assert philox.stream(7, 0, 5, skip=9) == philox.stream(7, 0, 14)[9:]
