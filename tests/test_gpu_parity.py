"""Parity of the HIP fusion backend with the oracle, through libdrhip's C ABI.

Bars (written out where they are applied):
  + - * / and sqrt expressions          bit-exact
  transcendental functions               <= 2 ulp in float32; <= 1e-13 relative in float64
  Black-Scholes call/put                 result-relative: <= 1e-13 (float64) wherever the price
                                         is >= 2^-8 max(S, K); float32: within 8 ulp of the
                                         oracle where the price is >= max(S, K)/2 and no
                                         farther from the true price than NumPy is (the
                                         stated 2 ulp is beyond NumPy's own float32 error,
                                         see `bs_bars`).  Everywhere, including options whose
                                         terms cancel:
                                         |gpu - oracle| <= 4 eps(float32) resp. 1e-13 (float64)
                                         times max(S, K).  The price is a difference of
                                         terms of that size, so ulps of the (possibly tiny)
                                         result would only measure cancellation, in NumPy as
                                         well; and the 27-node expression chains five
                                         functions that each may differ by 2 ulp, so the
                                         compound bound is wider than the per-function one
                                         (measured: 2.4 eps at n = 2^25).  The float32 result
                                         must also be as close to the float64 value as
                                         NumPy's own float32 result is.
  sum / max / min                        rtol 1e-13 (float64), 1e-6 (float32); max/min exact
"""
import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import hip, lowering
from delayrepay_amd.delayarray import ReduceEx
from oracle import numpy_oracle as orc
from oracle.numpy_oracle import OracleArray
from tests.helpers import bits_equal, golden, ulp_distance

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 4, 5, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4099, 100003, (1 << 20) + 1]


# ---- C1 SAXPY ---------------------------------------------------------------------------

@pytest.mark.parametrize("n", SIZES)
def test_saxpy_bit_exact(n):
    inp = orc.make_inputs("saxpy", n)
    z = inp["a"] * dr.array(inp["x"]) + dr.array(inp["y"])
    assert bits_equal(z.get(), orc.saxpy(inp["a"], inp["x"], inp["y"]))


def test_saxpy_golden():
    g = golden("configs_small.npz")
    z = 2.0 * dr.array(g["saxpy_x"]) + dr.array(g["saxpy_y"])
    assert bits_equal(z.get(), g["saxpy_z"])


def test_saxpy_full_size():
    inp = orc.make_inputs("saxpy")          # n = 2^24
    z = inp["a"] * dr.array(inp["x"]) + dr.array(inp["y"])
    assert bits_equal(z.get(), orc.saxpy(inp["a"], inp["x"], inp["y"]))


@pytest.mark.parametrize("lo,hi", [(1, None), (0, -1), (3, -5), (2, 2 + 4096)])
def test_saxpy_on_misaligned_contiguous_views(lo, hi):
    inp = orc.make_inputs("saxpy", 10000)
    x, y = dr.array(inp["x"]), dr.array(inp["y"])
    z = 2.0 * x[lo:hi] + y[lo:hi]
    assert bits_equal(z.get(), orc.saxpy(2.0, inp["x"][lo:hi], inp["y"][lo:hi]))


def test_denormals_infinities_and_nans_pass_through():
    tiny = np.finfo(np.float32).tiny
    x = np.array([tiny / 4, -tiny / 2, tiny, 0.0, -0.0, np.inf, -np.inf, np.nan, 1e38, 3e38] * 13,
                 np.float32)
    y = x[::-1].copy()
    with np.errstate(all="ignore"):
        for fn in (lambda a, b: a * 0.5 + b, lambda a, b: a / b, lambda a, b: (a - b) * a,
                   lambda a, b: a * a * a):
            got = fn(dr.array(x), dr.array(y)).get()
            assert bits_equal(got, fn(OracleArray(x), OracleArray(y)).get())


# ---- C2 Horner --------------------------------------------------------------------------

def horner_expr(c, x):
    acc = c[8] * x + c[7]
    for i in range(6, -1, -1):
        acc = acc * x + c[i]
    return acc


@pytest.mark.parametrize("n", [1, 1000, 4097, (1 << 20) + 3])
def test_horner_bit_exact(n):
    inp = orc.make_inputs("horner", n)
    y = horner_expr(inp["c"], dr.array(inp["x"]))
    assert bits_equal(y.get(), orc.horner(inp["c"], inp["x"]))


def test_horner_golden_and_kernel_reuse():
    g = golden("configs_small.npz")
    c = [float(v) for v in g["horner_c"]]
    y = horner_expr(c, dr.array(g["horner_x"]))
    assert bits_equal(y.get(), g["horner_y"])
    compiles = hip.STATS["compiles"] + hip.STATS["disk_hits"]
    other = [v * 0.5 - 0.1 for v in c]                     # new coefficients, same structure
    y2 = horner_expr(other, dr.array(g["horner_x"]))
    assert bits_equal(y2.get(), orc.horner(other, g["horner_x"]))
    assert hip.STATS["compiles"] + hip.STATS["disk_hits"] == compiles


def test_horner_full_size():
    inp = orc.make_inputs("horner")         # n = 2^26
    y = horner_expr(inp["c"], dr.array(inp["x"]))
    assert bits_equal(y.get(), orc.horner(inp["c"], inp["x"]))


# ---- C3 Black-Scholes -------------------------------------------------------------------

def bs_check(cfg, n):
    inp = orc.make_inputs(cfg, n)
    S, K, T = (dr.array(inp[k]) for k in "SKT")
    call, put = orc.black_scholes_expr(dr, S, K, T, inp["r"], inp["sigma"])
    launches = hip.STATS["launches"]
    dr.evaluate(call, put)
    assert hip.STATS["launches"] == launches + 1           # both roots from ONE kernel
    ocall, oput = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    scale = np.maximum(inp["S"], inp["K"])
    dt = inp["S"].dtype
    tol = 4 * np.finfo(np.float32).eps if dt == np.float32 else 1e-13
    for got, ref in ((call.get(), ocall), (put.get(), oput)):
        assert got.dtype == dt
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64)) / scale
        assert err.max() <= tol, (cfg, err.max(), int(err.argmax()))
    if dt == np.float32:     # accuracy against the float64 evaluation of the same inputs
        t_call, t_put = orc.black_scholes(*(inp[k].astype(np.float64) for k in "SKT"),
                                          inp["r"], inp["sigma"])
        for got, ref, truth in ((call.get(), ocall, t_call), (put.get(), oput, t_put)):
            e_gpu = np.max(np.abs(got - truth) / scale)
            e_np = np.max(np.abs(ref - truth) / scale)
            assert e_gpu <= 1.5 * e_np + np.finfo(np.float32).eps, (e_gpu, e_np)
    return call.get(), put.get(), inp


@pytest.mark.parametrize("cfg", ["bs64", "bs32"])
@pytest.mark.parametrize("n", [1, 1000, 65537])
def test_black_scholes_within_tolerance(cfg, n):
    call, put, inp = bs_check(cfg, n)
    if n > 1:
        bs_bars(cfg, call, put, inp)


def bs_bars(cfg, call, put, inp):
    """The result-relative bars, on the options where a result-relative figure means
    something, and the table that shows where they stop meaning something.

    float64: <= 1e-13 relative (the stated bar, literally) on every option whose price is
    at least 2^-8 of max(S, K): 62 % of the calls and 95 % of the puts at n = 2^25,
    measured maximum 4.9e-14.  Below that the two terms of the price cancel and the
    figure grows in the CPU evaluation exactly as on the device (at 2^-16: 7e-12, with
    the oracle itself 57 000 ulp from the 50-digit value); those are held by the bar
    scaled with max(S, K) in `bs_check`.
    float32: the stated 2 ulp cannot be met by any implementation, a correctly rounded
    one included: on the best-conditioned options (price >= max(S, K) / 2) NumPy's own
    float32 result is up to 4.6 (call) and 6.3 (put) ulp from the true price, so a perfect
    device result would still be 4-6 ulp from the oracle.  What is asserted instead: the
    device is within 8 / 16 / 40 ulp of the oracle on the subsets 2^-1 / 2^-2 / 2^-4
    (measured 8 / 16 / 40: each is the sum of the two sides' own errors), and it is at
    least as close to the true price (the float64 evaluation of the same inputs) as
    NumPy's float32 result is, plus one ulp."""
    from oracle import accuracy
    ocall, oput = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
    rep = accuracy.bs_report(call, put, ocall, oput, inp, detail=call.size >= 1 << 20)
    print("\n" + accuracy.format_report(cfg, rep), flush=True)
    for which in ("call", "put"):
        sub = rep[which]["subsets"]
        if cfg == "bs64":
            for k in (1, 2, 4, 8):
                if sub[k]["count"]:
                    assert sub[k]["max_rel"] <= 1e-13, (which, k, sub[k])
        else:
            for k, bound in ((1, 8), (2, 16), (4, 40)):
                if sub[k]["count"]:
                    assert sub[k]["max_ulp"] <= bound, (which, k, sub[k])
    if cfg == "bs32":
        truth = orc.black_scholes(*(inp[k].astype(np.float64) for k in "SKT"), inp["r"], inp["sigma"])
        scale = np.maximum(inp["S"], inp["K"]).astype(np.float64)
        for which, got, ref, t in (("call", call, ocall, truth[0]), ("put", put, oput, truth[1])):
            ulp = np.spacing(np.abs(t).astype(np.float32)).astype(np.float64)
            for k in (1, 2, 4):
                m = np.abs(t) >= scale * 2.0 ** -k
                if m.any():
                    e_dev = float(np.max(np.abs(got - t)[m] / ulp[m]))
                    e_np = float(np.max(np.abs(ref - t)[m] / ulp[m]))
                    print(f"  {which}, price >= 2^-{k} max(S,K): device {e_dev:.2f} ulp, NumPy float32 "
                          f"{e_np:.2f} ulp from the float64 value", flush=True)
                    assert e_dev <= e_np + 1.0, (which, k, e_dev, e_np)
    return rep


@pytest.mark.parametrize("cfg", ["bs64", "bs32"])
def test_black_scholes_full_size_and_put_call_parity(cfg):
    call, put, inp = bs_check(cfg, 1 << 25)
    bs_bars(cfg, call, put, inp)
    parity = inp["S"].astype(np.float64) - inp["K"] * np.exp(-inp["r"] * inp["T"].astype(np.float64))
    scale = np.maximum(inp["S"], inp["K"])
    tol = 8 * np.finfo(inp["S"].dtype).eps
    assert np.max(np.abs((call.astype(np.float64) - put) - parity) / scale) <= tol


@pytest.mark.parametrize("cfg", ["bs64", "bs32"])
def test_black_scholes_golden(cfg):
    g = golden("configs_small.npz")
    S, K, T = (dr.array(g[f"{cfg}_{k}"]) for k in "SKT")
    call, put = dr.evaluate(*orc.black_scholes_expr(dr, S, K, T, 0.02, 0.30))
    scale = np.maximum(g[f"{cfg}_S"], g[f"{cfg}_K"])
    tol = 4 * np.finfo(np.float32).eps if cfg == "bs32" else 1e-13
    assert np.max(np.abs(call.get() - g[f"{cfg}_call"]) / scale) <= tol
    assert np.max(np.abs(put.get() - g[f"{cfg}_put"]) / scale) <= tol


EXACT = ("negative", "absolute", "sqrt", "floor", "ceil", "trunc", "rint", "reciprocal",
         "add", "subtract", "multiply", "divide", "maximum", "minimum", "fmax", "fmin",
         "copysign", "fmod")


@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_every_function_on_the_special_value_table(tag):
    """Per-function accuracy against the golden table (NumPy/SciPy values)."""
    from tests.golden.make_golden import UNARY, BINARY
    g = golden("special_values.npz")
    x, y = dr.array(g[f"{tag}_x"]), dr.array(g[f"{tag}_y"])
    worst = {}
    for name, fn in list(UNARY.items()) + list(BINARY.items()):
        got = (fn(x) if name in UNARY else fn(x, y)).get()
        ref = g[f"{tag}_{name}"]
        assert got.dtype == ref.dtype, name
        assert np.array_equal(np.isnan(got), np.isnan(ref)), name
        if name in EXACT:
            assert bits_equal(got, ref), name
            continue
        finite = np.isfinite(ref)
        assert np.array_equal(got[~finite & ~np.isnan(ref)], ref[~finite & ~np.isnan(ref)]), name
        if tag == "f32":
            d = ulp_distance(got[finite], ref[finite])
            worst[name] = d.max() if d.size else 0
            assert worst[name] <= 2, (name, worst[name])          # <= 2 ulp in float32
        else:
            denom = np.maximum(np.abs(ref[finite]), np.finfo(np.float64).tiny)
            rel = np.abs(got[finite] - ref[finite]) / denom
            worst[name] = rel.max() if rel.size else 0
            assert worst[name] <= 1e-13, (name, worst[name])      # <= 1e-13 relative in float64
    print(tag, "worst:", {k: float(v) for k, v in sorted(worst.items(), key=lambda kv: -kv[1])[:6]})


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_transcendentals_on_dense_random_arguments(dtype):
    from scipy.special import erf
    rs = np.random.RandomState(11)
    n = 1 << 18
    cases = {
        "exp": (np.exp, rs.uniform(-20, 20, n)), "log": (np.log, rs.uniform(1e-6, 1e6, n)),
        "erf": (erf, rs.uniform(-6, 6, n)), "sin": (np.sin, rs.uniform(-100, 100, n)),
        "cos": (np.cos, rs.uniform(-100, 100, n)), "tanh": (np.tanh, rs.uniform(-10, 10, n)),
        "sqrt": (np.sqrt, rs.uniform(0, 1e6, n)), "arctan": (np.arctan, rs.uniform(-50, 50, n)),
    }
    for name, (fn, arg) in cases.items():
        arg = arg.astype(dtype)
        got, ref = fn(dr.array(arg)).get(), fn(arg)
        if dtype == np.float32:
            assert ulp_distance(got, ref).max() <= (0 if name == "sqrt" else 2), name
        else:
            assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-300)) <= 1e-13, name


def test_float64_sqrt_is_ieee_on_the_device():
    """The short float64 square root (reciprocal square root estimate by hardware, then
    the compiler's own correction steps) must give IEEE sqrt's bits: random arguments over
    every exponent, neighbours of perfect squares, and the arguments that take the guarded
    path (below 2^-767, denormals, zeros, infinity, NaN, negative)."""
    rs = np.random.RandomState(12)
    m = rs.uniform(1, 4, 1 << 22)
    exact = np.floor(rs.uniform(1, 2 ** 26, 1 << 18)) ** 2
    x = np.concatenate([m, np.ldexp(m, rs.randint(-1074, 1020, m.size)), exact, np.nextafter(exact, 0),
                        np.nextafter(exact, np.inf), rs.uniform(0, 1e-300, 1 << 12),
                        rs.randint(0, 1 << 62, 1 << 22).astype(np.uint64).view(np.float64),
                        [0.0, -0.0, np.inf, -np.inf, np.nan, -1.0, 4.0, 2.0, 1e-320, 5e-324, 2.0 ** -767,
                         np.nextafter(2.0 ** -767, 0), 1.7976931348623157e308]])
    with np.errstate(invalid="ignore"):
        want = np.sqrt(x)
    assert bits_equal(np.sqrt(dr.array(x)).get(), want)
    # inside a larger expression (the packed form) and in the general-stride kernel
    y = rs.uniform(0.5, 2, x.size)
    with np.errstate(invalid="ignore"):
        assert bits_equal((np.sqrt(dr.array(x)) * dr.array(y) + 1.0).get(), np.sqrt(x) * y + 1.0)
        x2 = x[:1 << 20].reshape(1 << 10, 1 << 10)
        assert bits_equal(np.sqrt(dr.array(x2)[::2, 1::3]).get(), np.sqrt(x2[::2, 1::3]))


@pytest.mark.parametrize("name", ["erf", "exp", "log"])
def test_float32_functions_over_the_bit_patterns(name):
    """The device's own float32 `erf`, `exp`, `log` (hardware 2^x and log2 inside) against
    SciPy / NumPy evaluated in float64 and rounded: every 7th float32 bit pattern (613
    million arguments, denormals, infinities and NaNs among them) plus every float32 of
    the intervals where the method changes.  Bar: 2 ulp of the correctly rounded result
    (exp, log: 1 ulp on denormal results, which have fewer bits)."""
    from scipy.special import erf
    fn = {"erf": erf, "exp": np.exp, "log": np.log}[name]
    worst = 0.0

    def check(bits):
        nonlocal worst
        x = bits.view(np.float32)
        got = fn(dr.array(x)).get()
        with np.errstate(all="ignore"):
            exact = fn(x.astype(np.float64))
            want = exact.astype(np.float32)
        fin = np.isfinite(want)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])   # infinities
        err = ulp_distance(got[fin], want[fin])
        k = int(err.argmax()) if err.size else 0
        assert err.size == 0 or err[k] <= 2, (name, x[fin][k], got[fin][k], want[fin][k])
        worst = max(worst, float(err.max()) if err.size else 0.0)

    step = 7
    for lo in range(0, 1 << 32, 1 << 29):
        check(np.arange(lo, lo + (1 << 29), step, dtype=np.uint64).astype(np.uint32))
    dense = {"erf": [(0.86, 0.89), (3.9, 4.1), (0.0, 1e-6)],
             "exp": [(86.0, 89.0), (-104.5, -86.0), (-1e-3, 1e-3)],
             "log": [(0.99, 1.01), (1e-39, 2e-38)]}[name]
    for a, b in dense:
        for sign in ((1, -1) if name != "log" else (1,)):
            lo, hi = sorted(np.array([a, b], np.float32).view(np.uint32).astype(np.int64))
            span = np.arange(lo, min(hi, lo + (1 << 25)), dtype=np.int64).astype(np.uint32)
            check(span if sign > 0 else span | np.uint32(1 << 31))
    print(f"\n  float32 {name}: worst {worst:.0f} ulp from the correctly rounded result", flush=True)


# ---- C4 Jacobi and other shifted-slice stencils --------------------------------------------

def jacobi_sweeps(u, sweeps):
    for _ in range(sweeps):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
    return u


@pytest.mark.parametrize("shape", [(3, 3), (4, 7), (8, 8), (17, 130), (18, 131), (130, 257),
                                   (129, 1000), (514, 514), (1000, 37)])
@pytest.mark.parametrize("sweeps", [1, 10])
def test_jacobi_bit_exact(shape, sweeps):
    rs = np.random.RandomState(7)
    u0 = np.zeros(shape, np.float32)
    u0[1:-1, 1:-1] = rs.uniform(0, 1, (shape[0] - 2, shape[1] - 2))
    u = jacobi_sweeps(dr.array(u0), sweeps)
    assert bits_equal(u.get(), orc.jacobi(u0, sweeps))


def test_jacobi_golden():
    g = golden("configs_small.npz")
    u = dr.array(g["jacobi_u0"])
    assert bits_equal(jacobi_sweeps(u, 1).get(), g["jacobi_u1"])
    assert bits_equal(jacobi_sweeps(u, 9).get(), g["jacobi_u10"])


def test_jacobi_full_size():
    inp = orc.make_inputs("jacobi")          # 8192 x 8192, 10 sweeps
    u = jacobi_sweeps(dr.array(inp["u"]), inp["sweeps"])
    got = u.get()
    assert bits_equal(got, orc.jacobi(inp["u"], inp["sweeps"]))
    assert not got[0].any() and not got[-1].any() and not got[:, 0].any() and not got[:, -1].any()


def test_jacobi_uses_the_lds_kernel_once_compiled():
    u = dr.array(np.zeros((64, 64), np.float32))
    jacobi_sweeps(u, 1)
    compiles = hip.STATS["compiles"] + hip.STATS["disk_hits"]
    launches = hip.STATS["launches"]
    jacobi_sweeps(u, 5)                       # new view objects every sweep, same structure
    assert hip.STATS["compiles"] + hip.STATS["disk_hits"] == compiles
    assert hip.STATS["launches"] == launches + 5      # one kernel per sweep, no copy-back


def test_stencil_result_into_fresh_array_and_all_views_see_updates():
    rs = np.random.RandomState(2)
    a0 = rs.uniform(-1, 1, (70, 90)).astype(np.float32)
    a = dr.array(a0)
    inner = a[1:-1, 1:-1]                     # a view taken BEFORE the update
    lap = a[:-2, 1:-1] + a[2:, 1:-1] + a[1:-1, :-2] + a[1:-1, 2:] - 4.0 * a[1:-1, 1:-1]
    oa = OracleArray(a0.copy())
    olap = oa[:-2, 1:-1] + oa[2:, 1:-1] + oa[1:-1, :-2] + oa[1:-1, 2:] - 4.0 * oa[1:-1, 1:-1]
    assert bits_equal(lap.get(), olap.get())  # fresh (70-2, 90-2) output
    a[1:-1, 1:-1] = 0.5 * (a[:-2, 1:-1] + a[2:, 1:-1])
    oa[1:-1, 1:-1] = 0.5 * (oa[:-2, 1:-1] + oa[2:, 1:-1])
    assert bits_equal(a.get(), oa.get())
    assert bits_equal(inner.get(), oa.get()[1:-1, 1:-1])      # old view follows the buffer


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_wide_and_asymmetric_stencils(dtype):
    rs = np.random.RandomState(4)
    a0 = rs.uniform(-1, 1, (61, 203)).astype(dtype)

    def nine_point(a):
        return (a[:-2, :-2] + a[:-2, 1:-1] + a[:-2, 2:] + a[1:-1, :-2] + a[1:-1, 1:-1]
                + a[1:-1, 2:] + a[2:, :-2] + a[2:, 1:-1] + a[2:, 2:]) / 9

    def skewed(a):
        return a[3:, 5:] * 2.0 - a[:-3, :-5] + a[1:-2, 2:-3]

    for fn in (nine_point, skewed):
        assert bits_equal(fn(dr.array(a0)).get(), fn(OracleArray(a0)).get()), fn.__name__


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_stencils_written_to_fresh_arrays_store_vectors_at_element_alignment(dtype):
    """The grid's rows are 16-byte periodic, the fresh result's rows (a few elements shorter)
    are not: LDS window along the grid's boundaries, stores at element alignment; another
    operand beside the window, a grid that starts off 16 bytes."""
    rs = np.random.RandomState(43)
    for shape in [(67, 200), (130, 1032), (9, 4100)]:
        a0 = rs.uniform(-1, 1, shape).astype(dtype)
        w0 = rs.uniform(-1, 1, (shape[0] - 2, shape[1] - 2)).astype(dtype)

        def nine(a, w):
            return (a[:-2, :-2] + a[:-2, 1:-1] + a[:-2, 2:] + a[1:-1, :-2] + a[1:-1, 1:-1]
                    + a[1:-1, 2:] + a[2:, :-2] + a[2:, 1:-1] + a[2:, 2:]) * w
        a, w = dr.array(a0), dr.array(w0)
        low = hip.lower_only(nine(a, w))[0]
        vw = 16 // np.dtype(dtype).itemsize
        assert low.key[0] == "tile2dv" and low.key[-1] is ((shape[1] - 2) % vw != 0), shape
        assert bits_equal(nine(a, w).get(), nine(OracleArray(a0), OracleArray(w0)).get()), shape
        sub, osub = a[1:, 4:], OracleArray(a0)[1:, 4:]        # still 16-byte periodic rows
        assert bits_equal(nine(sub, w[1:, 4:]).get(), nine(osub, OracleArray(w0)[1:, 4:]).get()), shape


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_shifted_views_of_a_vector_go_through_the_lds_window(dtype):
    """Differences and 1-D stencils: the vector is tiled as a matrix of one row; lengths
    around the tile width, views that start off 16 bytes, an operand beside the window,
    results written back into the vector."""
    rs = np.random.RandomState(44)
    for n in (4099, 5120, 100003, (1 << 20) + 5):
        a0 = rs.uniform(-1, 1, n).astype(dtype)
        b0 = rs.uniform(-1, 1, n).astype(dtype)
        a, b, oa, ob = dr.array(a0), dr.array(b0), OracleArray(a0), OracleArray(b0)
        low = hip.lower_only(a[2:] + a[:-2] - 2.0 * a[1:-1])[0]
        assert low.key[0] == "tile2dv" and low.tail[0] == 1, n
        assert bits_equal((a[1:] - a[:-1]).get(), (oa[1:] - oa[:-1]).get()), n
        assert bits_equal((a[2:] + a[:-2] - 2.0 * a[1:-1]).get(), (oa[2:] + oa[:-2] - 2.0 * oa[1:-1]).get()), n
        assert bits_equal(((a[5:] - a[:-5]) * b[3:-2]).get(), ((oa[5:] - oa[:-5]) * ob[3:-2]).get()), n
        s, os_ = a[3:-1], oa[3:-1]
        assert bits_equal((s[1:] * s[:-1]).get(), (os_[1:] * os_[:-1]).get()), n
    u0 = rs.uniform(0, 1, 50001).astype(dtype)
    u, ou = dr.array(u0), OracleArray(u0.copy())
    for _ in range(3):
        for arr in (u, ou):
            arr[1:-1] = 0.5 * (arr[:-2] + arr[2:])
    assert bits_equal(u.get(), ou.get())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_flipped_views_are_read_as_reversed_vectors(dtype):
    """`a[::-1]`, `m[:, ::-1]`, `m[::-1, ::-1]`: 16-byte loads from the mirrored place,
    reversed in registers; widths around the vector and tile sizes, a flipped operand beside
    a straight one, flips of interior views, a flipped 3-D array; narrow and mixed-width
    cases keep the element-wise kernel."""
    rs = np.random.RandomState(46)
    mk = (lambda s: rs.randint(-99, 99, s).astype(dtype)) if dtype == np.int32 else \
        (lambda s: rs.uniform(-1, 1, s).astype(dtype))
    for n in (17, 1000, 4099, 100003):
        a0, b0 = mk(n), mk(n)
        a, b = dr.array(a0), dr.array(b0)
        assert hip.lower_only(a[::-1] * 2)[0].key[0] == "tile2dv", n
        assert np.array_equal((a[::-1] * 2).get(), a0[::-1] * 2), n
        assert np.array_equal((a[::-1] + b).get(), a0[::-1] + b0), n
        assert np.array_equal((a[3:-2][::-1] - b[:-5]).get(), a0[3:-2][::-1] - b0[:-5]), n
    for shape in [(5, 16), (33, 1030), (257, 4100)]:
        m0, k0 = mk(shape), mk(shape)
        m, k = dr.array(m0), dr.array(k0)
        low = hip.lower_only(m[:, ::-1] * 2)[0]
        assert low.key[0] == "tile2dv" and ("dr",) in low.key[2], shape
        assert np.array_equal((m[:, ::-1] * 2).get(), m0[:, ::-1] * 2), shape
        assert np.array_equal((m[:, ::-1] + k).get(), m0[:, ::-1] + k0), shape
        assert np.array_equal((m[::-1, ::-1] - k).get(), m0[::-1, ::-1] - k0), shape
        assert np.array_equal((m[::-1, ::-1] + m[:, ::-1] + m[::-1]).get(),
                              m0[::-1, ::-1] + m0[:, ::-1] + m0[::-1]), shape
        assert np.array_equal((m[1:-1, 2:-1][:, ::-1] * k[1:-1, :-3]).get(),
                              m0[1:-1, 2:-1][:, ::-1] * k0[1:-1, :-3]), shape
        row0 = mk(shape[1])
        assert np.array_equal((m[:, ::-1] + dr.array(row0)).get(), m0[:, ::-1] + row0), shape
    v0 = mk((6, 7, 300))
    assert np.array_equal((dr.array(v0)[:, :, ::-1] * 3).get(), v0[:, :, ::-1] * 3)
    assert np.array_equal((dr.array(v0)[::-1, ::-1, ::-1] * 3).get(), v0[::-1, ::-1, ::-1] * 3)
    n0 = mk((40, 3))                                            # rows shorter than four vectors
    assert np.array_equal((dr.array(n0)[:, ::-1] * 2).get(), n0[:, ::-1] * 2)
    d0 = rs.uniform(-1, 1, (9, 200))                            # float64 beside the flipped operand
    m0 = mk((9, 200))
    assert np.array_equal((dr.array(m0)[:, ::-1] * dr.array(d0)).get(), m0[:, ::-1] * d0)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.uint8])
def test_every_kth_element_of_a_vector_takes_the_flat_kernel(dtype):
    """`a[::2]`: the vectors that hold a thread's elements are loaded whole and the elements
    picked out of the registers; `a[1::3]`, `a[5:-3:4]` and float64 go one element per lane;
    lengths around the vector and run sizes, views that end on the buffer's last element
    (the last vector is left to the element-wise tail), strided beside dense operands, a
    reduction, a float64 result."""
    rs = np.random.RandomState(47)
    mk = (lambda n: rs.randint(0, 99, n).astype(dtype)) if np.dtype(dtype).kind in "iu" else \
        (lambda n: rs.uniform(-1, 1, n).astype(dtype))
    for n in (64, 1000, 4096, 8192, 100003, 1 << 20):
        a0 = mk(n)
        a = dr.array(a0)
        for k in (2, 3, 4, 5, 8):
            for lo in (0, 1, k - 1):
                assert np.array_equal((a[lo::k] * 2).get(), a0[lo::k] * 2), (n, k, lo)
            low = hip.lower_only(a[::k] * 3)[0]          # not yet evaluated
            if k == 2 and np.dtype(dtype).itemsize <= 4:
                assert low.kind == "flat" and low.key[2] == ("s2",), (n, k)
            else:       # wider strides and types: one element per lane in the general kernel
                assert low.kind == "nd", (n, k)
        m = a0[::2].size
        b0 = mk(m)
        assert np.array_equal((a[::2] + dr.array(b0)).get(), a0[::2] + b0), n
        assert np.array_equal((a[1::2] - a[::2][:a0[1::2].size]).get(), a0[1::2] - a0[::2][:a0[1::2].size]), n
        assert np.array_equal((a[5:-3:4] * 3).get(), a0[5:-3:4] * 3), n
        d0 = rs.uniform(-1, 1, m)
        assert np.array_equal((a[::2] * dr.array(d0)).get(), a0[::2] * d0), n
    a0 = mk(1 << 16)
    a = dr.array(a0)
    if np.dtype(dtype).itemsize <= 4:
        # the view's last vector would end past the buffer: left to the tail
        assert hip.lower_only(a[1::2] * 2)[0].key[-2] is True
        assert hip.lower_only(a[::2] * 5)[0].key[-2] is False
    got, want = dr.sum(a[::2] * a[1::2]), np.sum(a0[::2] * a0[1::2])
    if np.dtype(dtype).kind == "f":
        assert abs(float(got) - float(want)) <= 1e-5 * (1 << 15)
    else:
        assert int(got) == int(want)
    m0 = mk(300 * 64).reshape(300, 64)
    assert np.array_equal((dr.array(m0)[:, ::2] * 2).get(), m0[:, ::2] * 2)     # rows merge: one stride
    assert np.array_equal((dr.array(m0)[:, 1::3] * 2).get(), m0[:, 1::3] * 2)   # they do not: general kernel


def test_boundary_change_between_sweeps_is_seen():
    """The ping-pong copy is refreshed when something else writes the buffer."""
    u0 = np.zeros((20, 24), np.float32)
    u0[1:-1, 1:-1] = np.random.RandomState(3).uniform(0, 1, (18, 22))
    u, ou = dr.array(u0), OracleArray(u0.copy())
    for step in range(4):
        for arr in (u, ou):
            arr[1:-1, 1:-1] = 0.25 * (arr[:-2, 1:-1] + arr[2:, 1:-1] + arr[1:-1, :-2] + arr[1:-1, 2:])
            arr[0, :] = float(step + 1)       # heat the top edge
    assert bits_equal(u.get(), ou.get())


def test_in_place_elementwise_update_of_a_view():
    a0 = np.random.RandomState(5).uniform(-1, 1, (33, 65)).astype(np.float32)
    a, oa = dr.array(a0), OracleArray(a0.copy())
    for arr in (a, oa):
        arr[1:-1, 1:-1] = 2.0 * arr[1:-1, 1:-1] + 1.0
        arr[5] = arr[6] * 3.0                 # rows: distinct memory, direct write
        arr[:, 0] = 9
    assert bits_equal(a.get(), oa.get())


def test_overlapping_1d_shift_assignment():
    a0 = np.arange(1000, dtype=np.float64)
    a, oa = dr.array(a0), OracleArray(a0.copy())
    for arr in (a, oa):
        arr[1:] = arr[:-1] + arr[1:]          # reads what it overwrites: needs the temporary
    assert bits_equal(a.get(), oa.get())


# ---- C5 fused element-wise + reduction ------------------------------------------------------

@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 1000, 4097, (1 << 20) + 3])
def test_sumsq_within_rtol(n):
    inp = orc.make_inputs("sumsq", n)
    x, y, w = (dr.array(inp[k]) for k in "xyw")
    launches = hip.STATS["launches"]
    s = dr.sum((x - y) ** 2 * w)
    assert hip.STATS["launches"] == launches + 2           # fused body+partials, finalize
    ref = orc.sumsq(inp["x"], inp["y"], inp["w"])
    assert abs(float(s) - ref) <= 1e-13 * abs(ref)         # documented rtol for the reduction


def test_sumsq_golden():
    g = golden("configs_small.npz")
    s = dr.sum((dr.array(g["sumsq_x"]) - dr.array(g["sumsq_y"])) ** 2 * dr.array(g["sumsq_w"]))
    assert abs(float(s) - float(g["sumsq_s"])) <= 1e-13 * float(g["sumsq_s"])


def test_sumsq_full_size_and_sum_of_partial_sums():
    inp = orc.make_inputs("sumsq")           # n = 2^27
    x, y, w = (dr.array(inp[k]) for k in "xyw")
    s = float(dr.sum((x - y) ** 2 * w))
    ref = float(orc.sumsq(inp["x"], inp["y"], inp["w"]))
    assert abs(s - ref) <= 1e-13 * abs(ref)
    n = x.shape[0]
    parts = [float(dr.sum((x[a:a + n // 8] - y[a:a + n // 8]) ** 2 * w[a:a + n // 8]))
             for a in range(0, n, n // 8)]
    assert abs(sum(parts) - s) <= 1e-13 * abs(s)
    assert s == float(dr.sum((x - y) ** 2 * w))            # deterministic: no atomics


def test_other_reductions_and_dtypes():
    rs = np.random.RandomState(9)
    a64 = rs.standard_normal(70001)
    a32 = a64.astype(np.float32)
    ai = rs.randint(-1000, 1000, 70001)
    assert float(dr.max(dr.array(a64))) == a64.max()
    assert float(dr.min(dr.array(a64) * 2.0)) == (a64 * 2.0).min()
    assert float(dr.max(dr.array(a32))) == a32.max()
    assert int(dr.sum(dr.array(ai))) == int(ai.sum())
    assert int(dr.sum(dr.array(ai.astype(np.int32)))) == int(ai.sum())
    s32 = dr.sum(dr.array(a32) * dr.array(a32))
    assert s32.dtype == np.float32
    assert abs(float(s32) - float(np.sum(a32 * a32))) <= 1e-6 * float(np.sum(a32 * a32))
    nan = a64.copy()
    nan[1234] = np.nan
    assert np.isnan(float(dr.max(dr.array(nan))))           # NaN propagates, like numpy.max
    m = dr.mean(dr.array(a64))
    assert abs(float(m) - a64.mean()) <= 1e-13 * abs(a64.mean()) + 1e-16
    v = dr.var(dr.array(a64))
    assert abs(float(v) - a64.var()) <= 1e-12 * a64.var()
    d = dr.array(a64).dot(dr.array(a64))
    assert abs(float(d) - a64.dot(a64)) <= 1e-13 * a64.dot(a64)
    strided = dr.array(rs.standard_normal((300, 70)))
    sub = strided[::3, 5:60:2]
    assert abs(float(dr.sum(sub * 2.0)) - float(np.sum(sub.get() * 2.0))) <= 1e-12 * 1e4


# ---- fused == un-fused; broadcasting; mixed dtypes -------------------------------------------

def test_unfused_mode_gives_identical_bits():
    inp = orc.make_inputs("horner", 50000)
    x = dr.array(inp["x"])
    fused = horner_expr(inp["c"], x).get()
    hip.set_fused(False)
    try:
        launches = hip.STATS["launches"]
        y = horner_expr([c + 0.0 for c in inp["c"]], dr.array(inp["x"]))
        unfused = y.get()
        assert hip.STATS["launches"] == launches + 16       # one kernel per DAG node
    finally:
        hip.set_fused(True)
    assert bits_equal(fused, unfused)


def test_broadcasting_and_mixed_dtypes_follow_numpy():
    rs = np.random.RandomState(6)
    a = rs.standard_normal((17, 1, 33))
    b = rs.standard_normal((1, 29, 33)).astype(np.float32)
    c = rs.randint(-5, 5, (29, 1))
    got = (dr.array(a) * dr.array(b) + dr.array(c) / 3).get()
    ref = (OracleArray(a) * OracleArray(b) + OracleArray(c) / 3).get()
    assert bits_equal(got, ref)
    row = rs.standard_normal(40).astype(np.float32)
    mat = rs.standard_normal((25, 40)).astype(np.float32)
    assert bits_equal((dr.array(mat) - dr.array(row)).get(), mat - row)
    assert bits_equal((dr.array(mat).T * 2.0).get(), mat.T * np.float32(2.0))
    cmp = (dr.array(mat) > 0.25).get()
    assert cmp.dtype == np.bool_ and np.array_equal(cmp, mat > 0.25)


def test_astype_is_fused_and_exact():
    x64 = np.random.RandomState(8).standard_normal(5000)
    x = dr.array(x64)
    got = ((x * 1.5).astype(np.float32) + 1).get()
    ref = (x64 * 1.5).astype(np.float32) + np.float32(1)
    assert bits_equal(got, ref)
    i = dr.full((64,), 7).astype(np.float32)               # reference tests/test.py:74
    assert i.dtype == np.float32 and bits_equal(i.get(), np.full((64,), 7).astype(np.float32))


# ---- plan reuse -------------------------------------------------------------------------------

def test_repeated_expression_reuses_its_plan_and_stays_correct():
    inp = orc.make_inputs("saxpy", 5000)
    x, y = dr.array(inp["x"]), dr.array(inp["y"])
    first = hip.run(2.0 * x + y)
    hits = hip.STATS["plan_hits"]
    again = hip.run(2.0 * x + y)              # same nodes from the hash-cons table
    assert hip.STATS["plan_hits"] == hits + 1
    assert bits_equal(first.get(), again.get()) and first.ptr != again.ptr
    x[:] = x * 3.0                            # leaves change: same plan, new values
    ref = orc.saxpy(2.0, inp["x"] * np.float32(3.0), inp["y"])
    assert bits_equal((2.0 * x + y).get(), ref)
    x64 = x.astype(np.float64)                # a new leaf; expressions on x are untouched
    assert x.dtype == np.float32 and bits_equal((2.0 * x + y).get(), ref)
    assert bits_equal((2.0 * x64 + y).get(),
                      2.0 * (inp["x"] * np.float32(3.0)).astype(np.float64) + inp["y"])


def test_sweeps_reuse_one_plan():
    u0 = np.zeros((40, 72), np.float32)
    u0[1:-1, 1:-1] = np.random.RandomState(1).uniform(0, 1, (38, 70))
    u = dr.array(u0)
    jacobi_sweeps(u, 2)
    hits = hip.STATS["plan_hits"]
    jacobi_sweeps(u, 6)
    assert hip.STATS["plan_hits"] == hits + 6
    assert bits_equal(u.get(), orc.jacobi(u0, 8))
    dr.reset()
    jacobi_sweeps(u, 1)
    assert bits_equal(u.get(), orc.jacobi(u0, 9))


# ---- edges: empty, 0-d, more than 2^31 elements -------------------------------------------------

def test_empty_and_zero_dimensional_arrays():
    e = dr.array(np.zeros((0,), np.float32))
    assert (e * 2.0 + 1).get().shape == (0,)
    assert float(dr.sum(e)) == 0.0 and dr.sum(e).dtype == np.float32
    with pytest.raises(ValueError):
        dr.max(e)
    e2 = dr.array(np.zeros((3, 0, 5)))
    assert (e2 + e2).get().shape == (3, 0, 5)
    e[:] = 1.0                                       # writes nothing, must not launch
    s = dr.array(np.float64(3.0))                    # 0-d leaf
    assert s.shape == () and float(s * 2 + 1) == 7.0
    v = dr.array(np.arange(5.0))
    assert np.array_equal((v * s).get(), np.arange(5.0) * 3.0)
    one = dr.array(np.array([2.5], np.float32))
    assert np.array_equal((one + one).get(), np.array([5.0], np.float32))


def test_more_than_2_to_31_elements():
    """64-bit indexing: n = 2^31 + 5 float32 (8 GiB per array)."""
    n = (1 << 31) + 5
    x = dr.zeros(n, dtype=np.float32)
    x[:] = 1.5
    x[n - 3:] = 2.5
    z = 2.0 * x + 1.0
    tail = z[n - 6:].get()
    assert np.array_equal(tail, np.array([4, 4, 4, 6, 6, 6], np.float32))
    assert float(z[1 << 31]) == 4.0 and float(z[0]) == 4.0
    total = float(dr.sum(z.astype(np.float64)))
    assert total == 4.0 * (n - 3) + 6.0 * 3
    strided = z[::3]                                  # > 2^31 / 3 elements through the nd kernel
    assert float(dr.max(strided * 1.0)) == 6.0 or float(dr.max(strided * 1.0)) == 4.0
    assert float(dr.sum((strided * 0.0 + 1.0).astype(np.float64))) == float(len(range(0, n, 3)))


# ---- reductions along axes -------------------------------------------------------------------------

@pytest.mark.parametrize("axis", [0, 1, 2, -1, (0, 1), (0, 2), (1, 2), (0, 1, 2)])
def test_axis_reductions_match_numpy(axis):
    rs = np.random.RandomState(12)
    a = rs.standard_normal((37, 70, 129))
    b = rs.standard_normal((70, 1)).astype(np.float32)
    da, db = dr.array(a), dr.array(b)
    got = dr.sum(da * db + 1.0, axis=axis)
    ref = np.sum(a * b + 1.0, axis=axis)
    got = np.asarray(got.get() if hasattr(got, "get") else got)
    assert got.shape == ref.shape and got.dtype == ref.dtype
    np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-12)
    mx = dr.max(da, axis=axis)
    mx = np.asarray(mx.get() if hasattr(mx, "get") else mx)
    assert np.array_equal(mx, np.max(a, axis=axis))
    kd = dr.sum(da, axis=axis, keepdims=True)
    assert kd.get().shape == np.sum(a, axis=axis, keepdims=True).shape


def test_axis_mean_var_on_views_and_integers():
    rs = np.random.RandomState(13)
    a = rs.standard_normal((64, 300))
    da = dr.array(a)
    np.testing.assert_allclose(dr.mean(da, axis=0).get(), a.mean(axis=0), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(dr.mean(da, axis=1).get(), a.mean(axis=1), rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(dr.var(da, axis=1).get(), a.var(axis=1), rtol=1e-11)
    np.testing.assert_allclose(dr.var(da, axis=0, ddof=1).get(), a.var(axis=0, ddof=1), rtol=1e-11)
    np.testing.assert_allclose(float(dr.var(da)), a.var(), rtol=1e-11)
    t = da.T[5:200:3]                                   # strided, transposed view
    np.testing.assert_allclose(dr.sum(t, axis=0).get(), a.T[5:200:3].sum(axis=0), rtol=1e-12)
    np.testing.assert_allclose(dr.sum(t * 2.0, axis=1).get(), (a.T[5:200:3] * 2.0).sum(axis=1),
                               rtol=1e-12)
    i = rs.randint(-50, 50, (33, 17)).astype(np.int32)
    s = dr.sum(dr.array(i), axis=0).get()
    assert s.dtype == np.int64 and np.array_equal(s, i.sum(axis=0))
    assert dr.mean(dr.array(i), axis=1).get().dtype == np.float64
    np.testing.assert_allclose(dr.mean(dr.array(i), axis=1).get(), i.mean(axis=1), rtol=1e-14)
    with pytest.raises(np.exceptions.AxisError):
        dr.sum(da, axis=2)


# ---- every tunable code path gives the same bits ------------------------------------------------------

TUNE_VARIANTS = [
    {"unroll": 2}, {"unroll": 4, "flat_cap": 512}, {"red_unroll": 1, "red_blocks": 64},
    {"ntl": 0, "nts": 0}, {"cache_mib": 0}, {"svec": 0}, {"lds": 0}, {"gpr": 32, "rpt": 4},
    {"gpr": 128, "rpt": 1}, {"tw": 64, "th": 8, "svec": 0}, {"sntl": 1, "snts": 0},
]


@pytest.mark.parametrize("variant", TUNE_VARIANTS, ids=lambda v: ",".join(f"{k}={x}" for k, x in v.items()))
def test_tunables_do_not_change_results(variant):
    saved = dict(hip.TUNE)
    hip.set_tune(**variant)
    try:
        inp = orc.make_inputs("horner", 70001)
        assert bits_equal(horner_expr(inp["c"], dr.array(inp["x"])).get(),
                          orc.horner(inp["c"], inp["x"]))
        u0 = np.zeros((67, 301), np.float32)
        u0[1:-1, 1:-1] = np.random.RandomState(7).uniform(0, 1, (65, 299))
        assert bits_equal(jacobi_sweeps(dr.array(u0), 3).get(), orc.jacobi(u0, 3))
        g = golden("configs_small.npz")
        s = dr.sum((dr.array(g["sumsq_x"]) - dr.array(g["sumsq_y"])) ** 2 * dr.array(g["sumsq_w"]))
        assert abs(float(s) - float(g["sumsq_s"])) <= 1e-13 * float(g["sumsq_s"])
        bs_check("bs64", 5000)
    finally:
        hip.set_tune(**saved)


def test_where_clip_sign_and_predicates():
    rs = np.random.RandomState(14)
    a0 = rs.standard_normal(4099).astype(np.float32)
    a0[::97] = np.nan
    a0[5::131] = np.inf
    a0[7::113] = -np.inf
    a0[11::89] = 0.0
    b0 = rs.standard_normal(4099).astype(np.float32)
    a, b = dr.array(a0), dr.array(b0)
    with np.errstate(all="ignore"):
        assert bits_equal(np.where(a > b, a * 2.0, b).get(), np.where(a0 > b0, a0 * np.float32(2.0), b0))
        assert bits_equal(np.where(a > 0, a, 0.0).get(), np.where(a0 > 0, a0, np.float32(0.0)))
        assert bits_equal(np.where(np.isnan(a), b, a).get(), np.where(np.isnan(a0), b0, a0))
        assert bits_equal(np.clip(a, -0.5, 0.75).get(), np.clip(a0, -0.5, 0.75))
        assert bits_equal(np.sign(a).get(), np.sign(a0))
        for fn in (np.isnan, np.isinf, np.isfinite, np.logical_not):
            got = fn(a).get()
            assert got.dtype == np.bool_ and np.array_equal(got, fn(a0)), fn.__name__
        assert np.array_equal(np.logical_and(a > 0, b > 0).get(), np.logical_and(a0 > 0, b0 > 0))
        assert np.array_equal(np.logical_or(a, b > 1).get(), np.logical_or(a0, b0 > 1))
        cnt = dr.sum(a > b)
        assert int(cnt) == int(np.sum(a0 > b0)) and cnt.dtype == np.int64
    i0 = rs.randint(-3, 4, 1000)
    assert np.array_equal(np.sign(dr.array(i0)).get(), np.sign(i0))
    assert np.array_equal(np.where(dr.array(i0) > 0, dr.array(i0), -1).get(), np.where(i0 > 0, i0, -1))


@pytest.mark.parametrize("dtype,tol", [(np.float32, 2e-5), (np.float64, 1e-13)])
def test_matrix_vector_products_are_fused_reductions(dtype, tol):
    """`A @ x` and `x @ A` read the matrix once as a reduction along / over its rows, fused
    with the expressions that make their operands; transposed and lazy operands, `np.dot`,
    mismatched shapes."""
    rs = np.random.RandomState(45)
    for m, k in [(600, 777), (33, 5000), (3000, 64), (1, 300), (257, 1)]:
        a0, x0, y0 = (rs.standard_normal(s).astype(dtype) for s in ((m, k), (k,), (m,)))
        a, x, y = dr.array(a0), dr.array(x0), dr.array(y0)
        ref = a0.astype(np.float64) @ x0.astype(np.float64)
        scale = np.abs(a0.astype(np.float64)) @ np.abs(x0.astype(np.float64))
        for got in (a @ x, np.dot(a, x), a.dot(x)):
            got = got.get()
            assert got.shape == (m,) and got.dtype == dtype
            assert np.all(np.abs(got - ref) <= tol * scale), (m, k)
        refl = y0.astype(np.float64) @ a0.astype(np.float64)
        scalel = np.abs(y0.astype(np.float64)) @ np.abs(a0.astype(np.float64))
        got = (y @ a).get()
        assert got.shape == (k,) and got.dtype == dtype and np.all(np.abs(got - refl) <= tol * scalel), (m, k)
        got = (a.T @ y).get()
        assert np.all(np.abs(got - refl) <= tol * scalel), (m, k)
        got = ((a * 2.0) @ (x + 1.0) - y).get()                   # fuses on both sides
        ref2 = (a0.astype(np.float64) * 2.0) @ (x0.astype(np.float64) + 1.0) - y0
        assert np.all(np.abs(got - ref2) <= tol * (2 * scale + 2 * np.abs(a0).sum(axis=1) + 1)), (m, k)
    with pytest.raises(ValueError):
        dr.array(np.zeros((4, 5), dtype)) @ dr.array(np.zeros(4, dtype))
    with pytest.raises(ValueError):
        dr.array(np.zeros(5, dtype)) @ dr.array(np.zeros((4, 5), dtype))
    i = dr.array(np.arange(12).reshape(3, 4)) @ dr.array(np.arange(4))     # integers: as before
    assert np.array_equal(np.asarray(i.get(), dtype=np.int64), np.arange(12).reshape(3, 4) @ np.arange(4))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_rows_that_share_an_operand_take_several_rows_per_block(dtype):
    """Row reductions with an operand that is the same for every row (`A @ x`): several rows
    per block, the shared vectors loaded once; the same sums to the bit as a block per row,
    row counts that are not multiples of the group, ragged row lengths, a per-row weight."""
    rs = np.random.RandomState(47)
    for m, k in [(4096, 4096), (4099, 5001), (5000, 4100)]:
        a0, x0, w0 = (rs.standard_normal(s).astype(dtype) for s in ((m, k), (k,), (m, 1)))
        a, x, w = dr.array(a0), dr.array(x0), dr.array(w0)
        results = {}
        default = lowering.TUNE["ax_block_rows"]
        for rows in (2, 3, 4, 1):
            hip.set_tune(ax_block_rows=rows)
            try:
                low = hip.lower_only(ReduceEx(np.add, a * x, (1,)))[0]
                assert low.kind == "axis_block" and (low.key[-1] == rows) == (rows > 1), (m, k, rows)
                results[rows] = (hip.run(ReduceEx(np.add, a * x, (1,))).get(),
                                 hip.run(ReduceEx(np.maximum, a * x * w, (1,))).get())
            finally:
                hip.set_tune(ax_block_rows=default)
        for rows in (2, 3, 4):
            assert bits_equal(results[rows][0], results[1][0]), (m, k, rows)
            assert bits_equal(results[rows][1], results[1][1]), (m, k, rows)
        ref = a0.astype(np.float64) @ x0.astype(np.float64)
        scale = np.abs(a0.astype(np.float64)) @ np.abs(x0.astype(np.float64))
        tol = 2e-5 if dtype == np.float32 else 1e-13
        assert np.all(np.abs(results[4][0] - ref) <= tol * scale)
        assert np.array_equal(results[4][1], (a0 * x0 * w0).max(axis=1))


def test_floor_division_and_remainder_follow_numpy():
    """`//` and `%`: floored quotient, remainder with the divisor's sign, to the bit; zero
    divisors, infinities, NaN, signed zeros, exact multiples, quotients just below an integer;
    integers with zero divisors and the most negative value divided by -1; mixed operands."""
    rs = np.random.RandomState(48)
    n = 6001
    for dt in (np.float32, np.float64):
        a0 = (rs.standard_normal(n) * 50).astype(dt)
        b0 = (rs.standard_normal(n) * 3).astype(dt)
        special = np.array([0.0, -0.0, 1.0, -1.0, 3.0, -3.0, 0.5, -0.5, np.inf, -np.inf, np.nan, 1e30, -1e-30,
                            7.0, -7.0, 0.1, 0.3], dt)
        a0[:special.size ** 2] = np.repeat(special, special.size)
        b0[:special.size ** 2] = np.tile(special, special.size)
        a0[400:800] = np.round(a0[400:800])                       # exact multiples
        b0[400:800] = np.round(b0[400:800]) + (np.round(b0[400:800]) == 0)
        a, b = dr.array(a0), dr.array(b0)
        with np.errstate(all="ignore"):
            assert bits_equal((a // b).get(), a0 // b0), dt
            assert bits_equal((a % b).get(), a0 % b0), dt
            assert bits_equal((a // 3).get(), a0 // dt(3)) and bits_equal((a % -0.7).get(), a0 % dt(-0.7)), dt
            assert bits_equal(np.remainder(a, b).get(), np.remainder(a0, b0)), dt
            assert bits_equal(((a // b) * b + a % b).get(), (a0 // b0) * b0 + a0 % b0), dt
    for dt in (np.int32, np.int64, np.uint32, np.uint8):
        info = np.iinfo(dt)
        x0 = rs.randint(max(info.min, -10 ** 9), min(info.max, 10 ** 9), n).astype(dt)
        y0 = rs.randint(max(info.min, -40), min(info.max, 40) if dt != np.uint8 else 40, n).astype(dt)
        x0[:6] = [info.min, info.min, info.max, 0, info.min, 7]
        y0[:6] = [info.max if info.min == 0 else -1, 1, 1 if info.min == 0 else -1, 0, 0, 0]
        x, y = dr.array(x0), dr.array(y0)
        with np.errstate(all="ignore"):
            for got, want in [(x // y, x0 // y0), (x % y, x0 % y0), (x // 7, x0 // 7), (x % 7, x0 % 7),
                              ((x % 2 == 0), (x0 % 2 == 0))]:
                got = got.get()
                assert got.dtype == want.dtype and np.array_equal(got, want), dt
    i0 = rs.randint(-99, 99, n)
    f0 = rs.standard_normal(n)
    with np.errstate(all="ignore"):
        assert bits_equal((dr.array(i0) % dr.array(f0)).get(), i0 % f0)
        assert bits_equal((dr.array(f0) // dr.array(i0)).get(), f0 // i0)


def test_bitwise_operations_and_shifts_follow_numpy():
    """`&`, `|`, `^`, `~` on masks and integers, shifts with counts up to and beyond the
    type's width (NumPy shifts everything out), mixed bool / integer operands, float
    operands refused with NumPy's TypeError."""
    rs = np.random.RandomState(41)
    n = 5003
    a0, b0 = rs.standard_normal(n).astype(np.float32), rs.standard_normal(n).astype(np.float32)
    a, b = dr.array(a0), dr.array(b0)
    assert np.array_equal(((a > b) & (a < 1.0)).get(), (a0 > b0) & (a0 < 1.0))
    assert np.array_equal(((a > b) | ~(b < 0.5)).get(), (a0 > b0) | ~(b0 < 0.5))
    assert np.array_equal(((a > 0) ^ (b > 0)).get(), (a0 > 0) ^ (b0 > 0))
    assert bits_equal(np.where((a > b) & (b > 0), a, b).get(), np.where((a0 > b0) & (b0 > 0), a0, b0))
    assert int(dr.sum((a > 0) & (b > 0))) == int(np.sum((a0 > 0) & (b0 > 0)))
    for dt in (np.int32, np.int64, np.uint32, np.uint8):
        info = np.iinfo(dt)
        x0 = rs.randint(info.min, info.max, n, dtype=dt)
        y0 = rs.randint(info.min, info.max, n, dtype=dt)
        k0 = rs.randint(0, 8 * np.dtype(dt).itemsize + 3, n).astype(dt)
        x, y, k = dr.array(x0), dr.array(y0), dr.array(k0)
        for got, want in [((x & y), x0 & y0), ((x | y), x0 | y0), ((x ^ y), x0 ^ y0), (~x, ~x0),
                          ((x & 15), x0 & 15), ((x << 3), x0 << 3), ((x >> 2), x0 >> 2),
                          (np.left_shift(x, k), np.left_shift(x0, k0)),
                          (np.right_shift(x, k), np.right_shift(x0, k0)),
                          ((x & (a > 0)), x0 & (a0 > 0))]:
            got = got.get()
            assert got.dtype == want.dtype and np.array_equal(got, want), dt
    with pytest.raises(TypeError):
        (a & b).get()
    with pytest.raises(TypeError):
        (~a).get()


def test_transposed_operands_go_through_lds_and_match():
    rs = np.random.RandomState(15)
    for shape in [(64, 64), (100, 200), (257, 63), (1, 300), (1000, 3)]:
        a0 = rs.standard_normal(shape).astype(np.float32)
        b0 = rs.standard_normal(shape[::-1])
        a, b = dr.array(a0), dr.array(b0)
        assert bits_equal((a.T * 2.0).get(), a0.T * np.float32(2.0))
        assert bits_equal((a.T + b).get(), a0.T + b0)                   # mixed dtypes, one transposed
        assert bits_equal((a.T * b.T.T + 1.0).get(), a0.T * b0 + 1.0)
        assert bits_equal(a.T.copy().get(), np.ascontiguousarray(a0.T))
    c0 = rs.standard_normal((40, 50, 60))
    c = dr.array(c0)
    assert bits_equal((c.transpose(2, 0, 1) * 1.5).get(), c0.transpose(2, 0, 1) * 1.5)   # general nd
    assert bits_equal((c.transpose(1, 0, 2) + 1).get(), c0.transpose(1, 0, 2) + 1)


# ---- generated leaves: constant and index-valued arrays computed inside the kernel ------------

def _same(got, ref):
    return got.dtype == ref.dtype and got.shape == ref.shape and got.tobytes() == ref.tobytes()


@pytest.mark.parametrize("args", [(100000,), (3, 200001), (0.0, 1000.0, 0.01), (1.5, 90000.25, 0.7),
                                  (50000, 0, -1), (10.0, -7000.0, -0.07), (0.1, 1e5, 0.3)])
def test_arange_is_numpys_to_the_bit(args):
    for kw in ({}, {"dtype": np.float32}, {"dtype": np.float64}, {"dtype": np.int64},
               {"dtype": np.int32}):
        if kw.get("dtype") in (np.int64, np.int32) and any(isinstance(v, float) for v in args):
            continue
        lazy = dr.arange(*args, **kw)
        assert not isinstance(lazy, dr.NPArray)
        assert _same(lazy.get(), np.arange(*args, **kw)), (args, kw)


def test_linspace_is_numpys_to_the_bit():
    for lo, hi, n, ep in [(0, 1, 10000, True), (-2.0, 2.0, (1 << 20) + 1, True),
                          (0.1, 1e6, 5001, False), (3, -3, 4096, True)]:
        for dt in (None, np.float32, np.float64):
            lazy = dr.linspace(lo, hi, n, endpoint=ep, dtype=dt)
            assert not isinstance(lazy, dr.NPArray)
            assert _same(lazy.get(), np.linspace(lo, hi, n, endpoint=ep, dtype=dt)), (lo, hi, n, ep, dt)


def test_generated_leaves_inside_expressions_and_other_kernel_shapes():
    n = (1 << 18) + 3
    x = np.random.RandomState(5).uniform(-1, 1, n).astype(np.float32)
    before = hip.STATS["launches"]
    got = (dr.linspace(-2.0, 2.0, n, dtype=np.float32) * dr.array(x) + dr.ones(n, dtype=np.float32)).get()
    assert hip.STATS["launches"] - before == 1                    # one kernel, the grid is never stored
    assert _same(got, np.linspace(-2.0, 2.0, n, dtype=np.float32) * x + np.ones(n, np.float32))
    # fused with a reduction
    s = dr.sum(dr.arange(n) * dr.array(x.astype(np.float64)))
    ref = np.sum(np.arange(n) * x.astype(np.float64))
    assert abs(float(s) - ref) <= 1e-12 * np.sum(np.abs(np.arange(n) * x.astype(np.float64)))
    # index broadcast along rows of a matrix: the index array is materialised, result unchanged
    m = np.random.RandomState(6).uniform(-1, 1, (7, 8192))
    assert _same((dr.array(m) + dr.arange(8192)).get(), m + np.arange(8192))
    assert _same((dr.array(m) * dr.linspace(0, 1, 8192)).get(), m * np.linspace(0, 1, 8192))
    # written into a strided destination, and into a contiguous one
    dst = dr.array(np.zeros((8192, 2)))
    dst[:, 1] = dr.arange(0.0, 8192.0, 1.0) * 2
    ref = np.zeros((8192, 2)); ref[:, 1] = np.arange(0.0, 8192.0, 1.0) * 2
    assert _same(dst.get(), ref)
    row = dr.array(np.zeros(8192))
    row[:] = dr.arange(8192) + 0.5
    assert _same(row.get(), np.arange(8192) + 0.5)
    # axis reduction over an expression with a generated operand
    assert np.allclose(dr.sum(dr.array(m) * dr.arange(8192), axis=1).get(),
                       (m * np.arange(8192)).sum(axis=1), rtol=1e-13)


def test_constant_arrays_stay_lazy_until_written():
    z = dr.zeros((300, 400), dtype=np.float32)
    assert "array" not in z.__dict__
    a = np.random.RandomState(7).uniform(0, 1, (300, 400)).astype(np.float32)
    y = z + dr.array(a) * 2
    assert _same(y.get(), np.zeros((300, 400), np.float32) + a * 2) and "array" not in z.__dict__
    assert _same(z.get(), np.zeros((300, 400), np.float32))        # asked for: now an array
    z[1:-1, 1:-1] = 3.0
    ref = np.zeros((300, 400), np.float32); ref[1:-1, 1:-1] = 3.0
    w = z + dr.array(a) * 2                                        # same structure as y, new values
    assert _same(w.get(), ref + a * 2)
    # a plan made while the constant was lazy is not reused after the write
    c = dr.full((1 << 14,), 2.5)
    expr = c * 2.0
    assert _same(expr.get(), np.full(1 << 14, 5.0))
    c[0] = 1.0
    ref = np.full(1 << 14, 2.5); ref[0] = 1.0
    assert _same((c * 2.0).get(), ref * 2.0)
    for make, ref in [(lambda: dr.ones((5000,), dtype=np.int32), np.ones(5000, np.int32)),
                      (lambda: dr.full((70, 70), 7, dtype=np.int64), np.full((70, 70), 7, np.int64)),
                      (lambda: dr.zeros_like(dr.array(a)), np.zeros_like(a)),
                      (lambda: dr.full_like(dr.array(a), 1.5, dtype=np.float64), np.full_like(a, 1.5, dtype=np.float64)),
                      (lambda: dr.zeros(4096, dtype=bool), np.zeros(4096, bool))]:
        assert _same(make().get(), ref)
    with pytest.raises(ValueError):                                # shapes are still checked
        dr.array(np.zeros(6000))[:] = dr.zeros(5000) + 1.0
    # the Jacobi set-up of configuration C4 starts from zeros and writes the interior
    u = dr.zeros((64, 64), dtype=np.float32)
    u[1:-1, 1:-1] = dr.array(a[:62, :62])
    ref = np.zeros((64, 64), np.float32); ref[1:-1, 1:-1] = a[:62, :62]
    assert _same(u.get(), ref)


# ---- views of unevaluated expressions -----------------------------------------------------------

def test_slices_transposes_and_rolls_of_lazy_expressions():
    rs = np.random.RandomState(12)
    ha, hb = rs.uniform(-1, 1, (300, 520)).astype(np.float32), rs.uniform(-1, 1, 520).astype(np.float32)
    A, B = dr.array(ha), dr.array(hb)
    e, ref = A * 2 + B, ha * 2 + hb
    before = hip.STATS["launches"]
    assert _same(e[1:-1, ::2].get(), ref[1:-1, ::2])
    assert hip.STATS["launches"] - before == 1 and "array" not in e.__dict__
    assert _same(e[3].get(), ref[3]) and _same(e[:, None, 5].get(), ref[:, None, 5])
    assert _same(e[..., -1].get(), ref[..., -1]) and _same(e[10:20, 7].get(), ref[10:20, 7])
    assert _same(e.T.get(), ref.T) and _same(np.transpose(e, (1, 0))[2:40].get(), ref.T[2:40])
    assert _same(np.roll(e, 7, axis=1).get(), np.roll(ref, 7, axis=1))
    assert _same(np.roll(e, -3, axis=0).get(), np.roll(ref, -3, axis=0))
    assert _same(np.roll(e, 0, axis=0).get(), ref)
    assert _same(np.roll(A[0] + 1, 5).get(), np.roll(ha[0] + 1, 5)) and "array" not in e.__dict__
    # a stencil on an expression: one kernel, the expression is never stored
    s, r = A * A + 1, ha * ha + 1
    before = hip.STATS["launches"]
    lap = s[:-2, 1:-1] + s[2:, 1:-1] + s[1:-1, :-2] + s[1:-1, 2:]
    assert _same(lap.get(), r[:-2, 1:-1] + r[2:, 1:-1] + r[1:-1, :-2] + r[1:-1, 2:])
    assert hip.STATS["launches"] - before == 1 and "array" not in s.__dict__
    # three dimensions, a lazy constant, an index array, a comparison
    hc = rs.uniform(-1, 1, (6, 40, 130))
    C = dr.array(hc)
    assert _same((C * 3 - 1)[1:5, ::3, 2:-2].get(), (hc * 3 - 1)[1:5, ::3, 2:-2])
    assert _same(np.transpose(C + 1, (2, 0, 1)).get(), np.transpose(hc + 1, (2, 0, 1)))
    assert _same((dr.zeros((300, 520), dtype=np.float32) + A)[2:5].get(), ha[2:5])
    assert _same((dr.arange(8192) * 2.0)[100:200].get(), (np.arange(8192) * 2.0)[100:200])
    assert _same(dr.where(A > 0, A, 0.0)[::7, 1::5].get(), np.where(ha > 0, ha, np.float32(0))[::7, 1::5])
    # too large to rebuild: evaluated once, then viewed
    big, rbig = A, ha
    for _ in range(60):
        big, rbig = big + 1.0, rbig + np.float32(1.0)
    assert _same(big[1:3].get(), rbig[1:3]) and "array" in big.__dict__


def test_reductions_over_short_rows():
    """Many short rows: a lane per output, the row length compiled in."""
    rs = np.random.RandomState(21)
    for shape, dt in [((50000, 3), np.float32), ((4096, 16), np.float64), ((70001, 7), np.float32),
                      ((8192, 64), np.float32), ((5000, 33), np.int32)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (1,)))[0]
        if shape[1] <= 28:
            assert low.kind == "axis_short" and low.key[-1] == shape[1]
        else:
            assert low.kind == "axis_group" and low.key[-2:] == (shape[1], 8)
        tol = dict(rtol=1e-5, atol=1e-5) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=1).get(), (h * h).sum(axis=1), **tol)
        assert dr.sum(a * a, axis=1).get().dtype == (h * h).sum(axis=1).dtype
        assert np.array_equal(dr.max(a, axis=1).get(), h.max(axis=1))
        assert np.array_equal(dr.min(a, axis=-1).get(), h.min(axis=-1))
        if dt != np.int32:
            assert np.allclose(dr.mean(a, axis=1).get(), h.mean(axis=1), **tol)
    # operands constant along the row, one row for all, and rows with a pitch
    h = rs.uniform(-1, 1, (20000, 8)).astype(np.float32)
    w, v = rs.uniform(0, 1, (20000, 1)).astype(np.float32), rs.uniform(0, 1, 8).astype(np.float32)
    a, W, V = dr.array(h), dr.array(w), dr.array(v)
    assert np.allclose(dr.sum(a * W + V, axis=1).get(), (h * w + v).sum(axis=1), rtol=1e-5, atol=1e-5)
    assert np.allclose(dr.sum(a[:, 1:6] * 2.0, axis=1).get(), (h[:, 1:6] * 2.0).sum(axis=1), rtol=1e-5,
                       atol=1e-5)
    assert hip.lower_only(ReduceEx(np.add, a[:, 1:6] * 2.0, (1,)))[0].kind == "axis_short"
    assert np.allclose(dr.sum(a, axis=1, keepdims=True).get(), h.sum(axis=1, keepdims=True), rtol=1e-5,
                       atol=1e-5)
    hip.set_tune(ax_short=0)                      # the wave-per-row kernel gives the same numbers
    try:
        assert np.allclose(dr.sum(a * W + V, axis=1).get(), (h * w + v).sum(axis=1), rtol=1e-5, atol=1e-5)
    finally:
        hip.set_tune(ax_short=28)


def test_reductions_over_rows_of_a_few_hundred_elements():
    """Rows too long for a lane and too short for a wave: a group of lanes per row
    (8 lanes up to 32 16-byte units per row, 16 beyond, more when a lane would otherwise
    take more than 8 units), the row length compiled in."""
    rs = np.random.RandomState(23)
    cases = [((9000, 100), np.float32, 8), ((6001, 200), np.float32, 16), ((4100, 250), np.float32, 16),
             ((3000, 333), np.float64, 32), ((2500, 257), np.int32, 16), ((1500, 1000), np.float32, 32),
             ((1100, 2048), np.float32, 64), ((2000, 131), np.float64, 16), ((1024, 29), np.float32, 8)]
    for shape, dt, lanes in cases:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (1,)))[0]
        assert low.kind == "axis_group" and low.key[-2:] == (shape[1], lanes), (shape, low.key[-2:])
        tol = dict(rtol=2e-5, atol=1e-4) if dt == np.float32 else dict(rtol=1e-12, atol=1e-12)
        assert np.allclose(dr.sum(a * a, axis=1).get(), (h * h).sum(axis=1), **tol), shape
        assert dr.sum(a * a, axis=1).get().dtype == (h * h).sum(axis=1).dtype
        assert np.array_equal(dr.max(a, axis=1).get(), h.max(axis=1))
        assert np.array_equal(dr.min(a, axis=-1).get(), h.min(axis=-1))
    # operands constant along the row, one row for all, rows with a pitch, a misaligned start
    h = rs.uniform(-1, 1, (5000, 210)).astype(np.float32)
    w, v = rs.uniform(0, 1, (5000, 1)).astype(np.float32), rs.uniform(0, 1, 210).astype(np.float32)
    a, W, V = dr.array(h), dr.array(w), dr.array(v)
    assert np.allclose(dr.sum(a * W + V, axis=1).get(), (h * w + v).sum(axis=1), rtol=2e-5, atol=1e-4)
    part = ReduceEx(np.add, a[:, 3:204] * 2.0, (1,))
    assert hip.lower_only(part)[0].kind == "axis_group"
    assert np.allclose(dr.sum(a[:, 3:204] * 2.0, axis=1).get(), (h[:, 3:204] * 2.0).sum(axis=1), rtol=2e-5,
                       atol=1e-4)
    assert np.array_equal(dr.max(a[1:4999:3, 5:205], axis=1).get(), h[1:4999:3, 5:205].max(axis=1))
    hip.set_tune(ax_group=0)                      # the wave-per-row kernel gives the same numbers
    try:
        assert np.allclose(dr.sum(a * W + V, axis=1).get(), (h * w + v).sum(axis=1), rtol=2e-5, atol=1e-4)
    finally:
        hip.set_tune(ax_group=2048)


def test_reductions_over_the_rows_of_narrow_matrices():
    """Few columns, many rows: the matrix is read as one stream, lanes keep their columns."""
    rs = np.random.RandomState(22)
    for shape, dt in [((50000, 3), np.float32), ((8192, 16), np.float64), ((70001, 7), np.float32),
                      ((5000, 64), np.float32), ((20000, 33), np.int32), ((4096, 2), np.float64)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (0,)))[0]
        assert low.kind == "axis_narrow" and low.key[-1] == shape[1]
        ref = (h.astype(np.float64) ** 2).sum(axis=0)
        tol = dict(rtol=2e-5) if dt == np.float32 else dict(rtol=1e-13)
        got = dr.sum(a * a, axis=0).get()
        assert got.dtype == (h * h).sum(axis=0).dtype and np.allclose(got, ref, **tol)
        assert np.array_equal(dr.max(a, axis=0).get(), h.max(axis=0))
        assert np.array_equal(dr.min(a, axis=0).get(), h.min(axis=0))
        if dt != np.int32:
            assert np.allclose(dr.mean(a, axis=0).get(), h.astype(np.float64).mean(axis=0),
                               rtol=tol["rtol"], atol=1e-6)
            assert np.allclose(dr.var(a, axis=0).get(), h.astype(np.float64).var(axis=0), rtol=1e-4)
    # one row of weights for all rows, a scalar array, keepdims; fewer rows take the general kernel
    h = rs.uniform(0, 1, (30000, 12)).astype(np.float32)
    w, c = rs.uniform(0, 1, 12).astype(np.float32), np.float32(0.5)
    a, W = dr.array(h), dr.array(w)
    ex = a * W + dr.array(np.array([c]))
    assert hip.lower_only(ReduceEx(np.add, ex, (0,)))[0].kind == "axis_narrow"
    assert np.allclose(dr.sum(ex, axis=0).get(), (h.astype(np.float64) * w + c).sum(axis=0), rtol=2e-5)
    assert np.allclose(dr.sum(a, axis=0, keepdims=True).get(), h.sum(axis=0, keepdims=True), rtol=2e-5)
    assert hip.lower_only(ReduceEx(np.add, dr.array(h[:100]) * 1.0, (0,)))[0].kind == "axis_col"
    assert hip.lower_only(ReduceEx(np.add, a[:, :5] * 1.0, (0,)))[0].kind == "axis_col"   # not dense
    assert np.allclose(dr.sum(a[:, :5] * 1.0, axis=0).get(), h[:, :5].sum(axis=0), rtol=2e-5)
    # three dimensions: the leading two merge into the rows
    h3 = rs.uniform(-1, 1, (300, 200, 6))
    assert np.allclose(dr.sum(dr.array(h3), axis=(0, 1)).get(), h3.sum(axis=(0, 1)), rtol=1e-12, atol=1e-10)


def test_own_float64_functions_stay_within_two_ulp_of_numpy_on_the_device():
    """The device build differs from the host build checked in test_mathlib.py in two
    places (reciprocal seed + Newton steps, multiply-add with a scalar-register
    constant); libm and SciPy are within 1 resp. 2.6 ulp of the true value themselves."""
    from scipy.special import erf
    rs = np.random.RandomState(31)
    n = 1 << 20
    cases = {
        "log": (np.log, np.concatenate([rs.uniform(1e-6, 1e6, n), np.exp(rs.uniform(-700, 700, n)),
                                        1 + rs.uniform(-1e-6, 1e-6, n // 4),
                                        [5e-324, 1e-310, 2.2250738585072014e-308, 1.7976931348623157e308]]), 2),
        "exp": (np.exp, np.concatenate([rs.uniform(-20, 20, n), rs.uniform(-708, 709, n),
                                        rs.uniform(-1e-3, 1e-3, n // 4)]), 2),
        "erf": (erf, np.concatenate([rs.uniform(-6.5, 6.5, n), rs.uniform(-1, 1, n),
                                     10.0 ** rs.uniform(-300, 0, n // 4)]), 4),
    }
    for name, (fn, x, bar) in cases.items():
        got, ref = fn(dr.array(x)).get(), fn(x)
        d = np.abs(got - ref) / np.spacing(np.abs(ref))
        print(name, "worst ulp distance from the host library:", d.max())
        assert d.max() <= bar, (name, x[d.argmax()], d.max())
    hip.set_tune(dmath=0)          # the device library's versions, for comparison
    try:
        x = rs.uniform(0.1, 10, 1 << 16)
        assert np.max(np.abs(np.log(dr.array(x)).get() - np.log(x)) / np.spacing(np.abs(np.log(x)))) <= 2
    finally:
        hip.set_tune(dmath=1)


def test_generated_leaves_behave_like_arrays_everywhere():
    assert float(dr.sum(dr.ones(10000))) == 10000.0
    assert float(dr.max(dr.arange(10000))) == 9999
    assert np.array_equal(dr.ones((300, 400)).T.get(), np.ones((400, 300)))
    assert np.array_equal(dr.zeros(5000)[10:20].get(), np.zeros(10))
    assert dr.ones(5000).astype(np.float32).get().dtype == np.float32
    assert np.array_equal(dr.arange(5000).reshape(50, 100).get(), np.arange(5000).reshape(50, 100))
    assert np.array_equal(dr.where(dr.arange(5000) > 10, 1.0, 0.0).get(), np.where(np.arange(5000) > 10, 1.0, 0.0))
    assert abs(float(dr.mean(dr.linspace(0, 1, 5000))) - 0.5) < 1e-12
    assert np.array_equal(dr.sum(dr.ones((300, 400)), axis=0).get(), np.full(400, 300.0))
    assert np.array_equal(dr.sum(dr.ones((5000, 4)), axis=1).get(), np.full(5000, 4.0))
    assert np.array_equal(dr.sum(dr.ones((5000, 4)) * dr.array(np.arange(4.0)), axis=0).get(), np.arange(4.0) * 5000)
    a = dr.arange(6000); b = a.copy(); assert np.array_equal(b.get(), np.arange(6000))
    assert len(dr.zeros((5000, 3))) == 5000 and dr.zeros((5000, 3)).ndim == 2
    z = dr.zeros(5000); z += 1; assert np.array_equal(z.get(), np.ones(5000))
    e, f = dr.evaluate(dr.ones(5000) * 2, dr.arange(5000) + 1)
    assert np.array_equal(e.get(), np.full(5000, 2.0)) and np.array_equal(f.get(), np.arange(5000) + 1)
    assert np.array_equal(np.roll(dr.arange(5000) * 1, 3).get(), np.roll(np.arange(5000), 3))
    assert repr(dr.arange(5000)).startswith("[   0    1    2")
    assert np.array_equal(np.asarray(dr.arange(5000)), np.arange(5000))


def test_slices_of_generated_grids_stay_generated():
    n = 1 << 20
    g = dr.linspace(-2.0, 2.0, n, dtype=np.float32)
    p = ((0.5 * g + 1.0) * g - 3.0) * g
    lap = (p[:-2] + p[2:]) - 2.0 * p[1:-1]
    hg = np.linspace(-2.0, 2.0, n, dtype=np.float32)
    hp = ((np.float32(0.5) * hg + 1) * hg - 3) * hg
    assert len(hip.lower_only(lap)[0].srcs) == 0                 # nothing is read
    before = hip.STATS["launches"]
    got = lap.get()
    assert hip.STATS["launches"] - before == 1
    assert _same(got, (hp[:-2] + hp[2:]) - np.float32(2.0) * hp[1:-1])
    a = dr.arange(100000)
    assert _same((a * 3)[5:90000:7].get(), (np.arange(100000) * 3)[5:90000:7])
    assert _same((a * 3)[::-1][:10].get(), (np.arange(100000) * 3)[::-1][:10])


@pytest.mark.parametrize("groups", [True, False])
def test_row_reductions_with_vector_loads_and_ragged_ends(groups):
    """A wave per row (fewer than 1024 rows, or rows beyond 2048 elements) or a group of lanes
    per row, 16-byte loads at element alignment; the row length need not be a multiple of
    the vector, nor the row start aligned."""
    rs = np.random.RandomState(23)
    hip.set_tune(ax_group=2048 if groups else 0)
    try:
        _row_reduction_cases(rs, groups)
    finally:
        hip.set_tune(ax_group=2048)


def _row_reduction_cases(rs, groups):
    for shape, dt in [((3000, 200), np.float32), ((2000, 257), np.float64), ((1500, 515), np.float32),
                      ((700, 230), np.int32)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (1,)))[0]
        if groups and shape[0] >= 1024:
            assert low.kind == "axis_group"
        else:
            assert low.kind == "axis_row" and low.key[-1] == ("v",)
        tol = dict(rtol=2e-5, atol=1e-5) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=1).get(), (h.astype(np.float64) ** 2).sum(axis=1), **tol)
        assert np.array_equal(dr.max(a, axis=1).get(), h.max(axis=1))
        assert np.array_equal(dr.min(a[:, 3:-2], axis=1).get(), h[:, 3:-2].min(axis=1))
    h = rs.uniform(0, 1, (900, 300)).astype(np.float32)
    w = rs.uniform(0, 1, (900, 1)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(w) + 1.0, axis=1).get()
    assert np.allclose(got, (h.astype(np.float64) * w + 1.0).sum(axis=1), rtol=2e-5)


def test_reductions_over_long_rows_take_a_block_per_row_slice():
    """Rows from 4096 elements: a block streams a row (or a slice of it, when there are too
    few rows to fill the device) like a flat reduction; lengths that are not multiples of the
    vector, rows that start off 16 bytes, an operand constant along the row."""
    rs = np.random.RandomState(29)
    for shape, dt in [((300, 4096), np.float32), ((129, 5003), np.float64), ((3, 1 << 20), np.float32),
                      ((40, 4099), np.int32), ((1, 70001), np.float64)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (1,)))[0]
        assert low.kind == "axis_block", (shape, low.kind)
        tol = dict(rtol=2e-5, atol=1e-4) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=1).get(), (h.astype(np.float64) ** 2).sum(axis=1), **tol)
        assert np.array_equal(dr.max(a, axis=1).get(), h.max(axis=1))
        assert np.array_equal(dr.min(a[:, 3:-2], axis=1).get(), h[:, 3:-2].min(axis=1))
        if dt == np.int32:
            assert np.array_equal(dr.sum(a, axis=1).get(), h.sum(axis=1))
    h = rs.uniform(0, 1, (50, 6000)).astype(np.float32)
    w = rs.uniform(0, 1, (50, 1)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(w) + 1.0, axis=1).get()
    assert np.allclose(got, (h.astype(np.float64) * w + 1.0).sum(axis=1), rtol=2e-5)
    m = dr.mean(dr.array(h), axis=1).get()
    assert np.allclose(m, h.mean(axis=1, dtype=np.float64), rtol=2e-5)


def test_reductions_over_the_first_and_last_axis_of_a_three_dimensional_array():
    """Per-channel statistics: (N, C, L) reduced over N and L; rows of the last axis that
    are not multiples of the vector, an operand constant along the last axis."""
    rs = np.random.RandomState(33)
    for shape, dt in [((9, 5, 1024), np.float32), ((33, 7, 1500), np.float64), ((4, 3, 2049), np.int32)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (0, 2)))[0]
        assert low.kind == "axis_block" and low.key[-1] == "outer", (shape, low.kind)
        tol = dict(rtol=2e-5, atol=1e-4) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=(0, 2)).get(), (h.astype(np.float64) ** 2).sum(axis=(0, 2)), **tol)
        assert np.array_equal(dr.max(a, axis=(0, 2)).get(), h.max(axis=(0, 2)))
        assert np.array_equal(dr.min(a[1:, :, 3:-2], axis=(0, 2)).get(), h[1:, :, 3:-2].min(axis=(0, 2)))
    h = rs.uniform(0, 1, (40, 6, 1100)).astype(np.float32)
    w = rs.uniform(0, 1, (40, 6, 1)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(w), axis=(0, 2)).get()
    assert np.allclose(got, (h.astype(np.float64) * w).sum(axis=(0, 2)), rtol=2e-5)
    m = dr.mean(dr.array(h), axis=(0, 2)).get()
    assert np.allclose(m, h.mean(axis=(0, 2), dtype=np.float64), rtol=2e-5)


def test_reductions_over_the_middle_axis_of_a_three_dimensional_array():
    """(N, R, L) reduced over R with long rows L: the row-streaming kernel once per index of
    the first axis; ragged rows, views off 16 bytes, slices of R, an operand constant along L."""
    rs = np.random.RandomState(35)
    for shape, dt in [((3, 700, 1024), np.float32), ((5, 64, 1500), np.float64), ((2, 3000, 2049), np.int32)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (1,)))[0]
        assert low.kind == "axis_stream" and low.key[-1] == "outer", (shape, low.kind)
        tol = dict(rtol=2e-5, atol=1e-4) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=1).get(), (h.astype(np.float64) ** 2).sum(axis=1), **tol)
        assert np.array_equal(dr.max(a, axis=1).get(), h.max(axis=1))
        assert np.array_equal(dr.min(a[1:, 2:-1, 3:-2], axis=1).get(), h[1:, 2:-1, 3:-2].min(axis=1))
    h = rs.uniform(0, 1, (6, 90, 1100)).astype(np.float32)
    w = rs.uniform(0, 1, (6, 90, 1)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(w), axis=1).get()
    assert np.allclose(got, (h.astype(np.float64) * w).sum(axis=1), rtol=2e-5)
    v = rs.uniform(0, 1, (1, 90, 1100)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(v), axis=1).get()
    assert np.allclose(got, (h.astype(np.float64) * v).sum(axis=1), rtol=2e-5)


def test_reductions_over_the_rows_of_wide_matrices_stream_whole_rows():
    """Kept rows of 256 vectors or more: a block owns 256 lanes x one vector of columns and
    walks a slice of rows; widths that are not multiples of the vector, views that start off
    16 bytes, an operand constant along the kept dimension, integer sums, extrema."""
    rs = np.random.RandomState(31)
    for shape, dt in [((5000, 1024), np.float32), ((300, 3001), np.float64), ((64, 1030), np.float32),
                      ((2000, 2050), np.int32), ((70, 4096), np.float64)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int32 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        low = hip.lower_only(ReduceEx(np.add, a * a, (0,)))[0]
        assert low.kind == "axis_stream", (shape, low.kind)
        tol = dict(rtol=2e-5, atol=1e-4) if dt == np.float32 else dict(rtol=1e-13, atol=1e-13)
        assert np.allclose(dr.sum(a * a, axis=0).get(), (h.astype(np.float64) ** 2).sum(axis=0), **tol)
        assert np.array_equal(dr.max(a, axis=0).get(), h.max(axis=0))
        assert np.array_equal(dr.min(a[1:-1, 3:-2], axis=0).get(), h[1:-1, 3:-2].min(axis=0))
        if dt == np.int32:
            assert np.array_equal(dr.sum(a, axis=0).get(), h.sum(axis=0))
    h = rs.uniform(0, 1, (900, 1500)).astype(np.float32)
    w = rs.uniform(0, 1, (900, 1)).astype(np.float32)
    got = dr.sum(dr.array(h) * dr.array(w) + 1.0, axis=0).get()
    assert np.allclose(got, (h.astype(np.float64) * w + 1.0).sum(axis=0), rtol=2e-5)
    v = dr.var(dr.array(h), axis=0).get()
    assert np.allclose(v, h.astype(np.float64).var(axis=0), rtol=1e-4)


def test_transposes_of_arrays_with_more_than_two_dimensions_go_through_the_lds_tile():
    """Every permutation whose unit stride lands on another output dimension: the two
    dimensions the tiles span are transposed through LDS, the others are a batch."""
    import itertools
    rs = np.random.RandomState(37)
    for shape, dt in [((5, 70, 33), np.float32), ((3, 4, 130, 9), np.float64), ((40, 36, 64), np.float32),
                      ((6, 50, 20), np.int64)]:
        h = (rs.uniform(-3, 3, shape) if dt != np.int64 else rs.randint(-9, 9, shape)).astype(dt)
        a = dr.array(h)
        for perm in itertools.permutations(range(len(shape))):
            if perm[-1] == len(shape) - 1:
                continue
            ex = dr.transpose(a, perm) * 2
            low = hip.lower_only(ex)[0]
            assert low.kind in ("tile2dt", "thin_t"), (shape, perm, low.kind)
            assert np.array_equal(ex.get(), h.transpose(perm) * 2), (shape, perm)
    h = rs.uniform(-1, 1, (24, 40, 64)).astype(np.float32)
    d = rs.uniform(-1, 1, (64, 40, 24)).astype(np.float32)
    col = rs.uniform(-1, 1, (40, 1)).astype(np.float32)
    got = (dr.array(h).T + dr.array(d) * 3.0 + dr.array(col)).get()      # reversed axes, a dense
    assert np.array_equal(got, h.T + d * np.float32(3.0) + col)          # operand and a broadcast
    big = rs.uniform(-1, 1, (64, 96, 128))
    assert np.array_equal((dr.array(big).T * 2.0).get(), big.T * 2.0)


def test_masks_move_as_vectors_of_sixteen_bytes():
    """Bool and uint8 operands and results in flat kernels: sixteen per lane and access, the
    wider operands beside them four or eight vectors; lengths that are not multiples of
    sixteen, views that start at odd bytes."""
    rs = np.random.RandomState(47)
    for n in (1 << 20, (1 << 20) + 13, 100, 65):
        ha, hb = rs.uniform(-1, 1, n).astype(np.float32), rs.uniform(-1, 1, n)
        hm = rs.uniform(-1, 1, n) > 0
        hu = rs.randint(0, 200, n).astype(np.uint8)
        a, b, m, u = dr.array(ha), dr.array(hb), dr.array(hm), dr.array(hu)
        low, src = hip.lower_only(a > 0)
        assert low.kind == "flat" and (n < 64 or "u1x16" in src)
        assert np.array_equal((a > 0).get(), ha > 0)
        assert np.array_equal(dr.where(m, a, b).get(), np.where(hm, ha, hb))
        assert np.array_equal(np.logical_and(m, a > b).get(), np.logical_and(hm, ha > hb))
        assert np.array_equal((u + np.uint8(3)).get(), hu + np.uint8(3))
        assert np.array_equal(dr.where(m[1:], a[1:], 0.5).get(), np.where(hm[1:], ha[1:], np.float32(0.5)))
        assert np.array_equal((u[3:] * a[3:]).get(), hu[3:] * ha[3:])
        assert dr.sum(m) == hm.sum() and dr.sum(u) == hu.sum()


def test_reduction_strategy_follows_the_operands_that_carry_the_traffic():
    """A column of weights beside a matrix (unit stride along the reduced axis) must not
    switch a sum over rows to the kernel for sums along rows."""
    rs = np.random.RandomState(24)
    h, w = rs.uniform(0, 1, (3000, 500)), rs.uniform(0, 1, (3000, 1))
    a, W = dr.array(h), dr.array(w)
    assert hip.lower_only(ReduceEx(np.add, a * W, (0,)))[0].kind == "axis_col"
    assert np.allclose(dr.sum(a * W, axis=0).get(), (h * w).sum(axis=0), rtol=1e-13)
    r = rs.uniform(0, 1, (1, 500))
    assert hip.lower_only(ReduceEx(np.add, a * dr.array(r), (1,)))[0].kind in ("axis_row", "axis_group")
    assert np.allclose(dr.sum(a * dr.array(r), axis=1).get(), (h * r).sum(axis=1), rtol=1e-13)


def _laplace3d(u, f=None, c=1 / 6.0):
    s = (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1] + u[1:-1, 2:, 1:-1]
         + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:])
    return c * s if f is None else c * (s + f)


@pytest.mark.parametrize("shape,dtype", [((40, 36, 64), np.float32), ((33, 50, 132), np.float32),
                                         ((20, 24, 40), np.float64), ((9, 9, 260), np.float32)])
def test_stencils_in_three_dimensions_go_through_the_lds_window(shape, dtype):
    rs = np.random.RandomState(41)
    h = rs.uniform(0, 1, shape).astype(dtype)
    src_term = rs.uniform(0, 1, tuple(s - 2 for s in shape)).astype(dtype)
    u, ref = dr.array(h), h.copy()
    c = dtype(1 / 6.0) if dtype == np.float32 else 1 / 6.0
    kinds_before = {k[0] for k in hip._KERNELS}
    for _ in range(3):                                        # in place: ping-pong buffers
        u[1:-1, 1:-1, 1:-1] = _laplace3d(u)
        ref[1:-1, 1:-1, 1:-1] = _laplace3d(ref, c=c)
    assert u.get().tobytes() == ref.tobytes()
    assert "tile3d" in {k[0] for k in hip._KERNELS} | kinds_before
    # into another array, with a source term read directly and a row-constant operand
    F = dr.array(src_term)
    col = rs.uniform(0, 1, (shape[1] - 2, 1)).astype(dtype)
    v = dr.array(np.zeros(shape, dtype))
    v[1:-1, 1:-1, 1:-1] = _laplace3d(u, F) + dr.array(col)
    expect = np.zeros(shape, dtype)
    expect[1:-1, 1:-1, 1:-1] = _laplace3d(ref, src_term, c=c) + col
    assert v.get().tobytes() == expect.tobytes()
    # a fresh result, 27 points, wider reach along x
    w = (u[:-2, :-2, :-4] + u[1:-1, 1:-1, 2:-2] * 2 + u[2:, 2:, 4:] + u[2:, :-2, 1:-3]).get()
    r = ref[:-2, :-2, :-4] + ref[1:-1, 1:-1, 2:-2] * 2 + ref[2:, 2:, 4:] + ref[2:, :-2, 1:-3]
    assert w.tobytes() == r.tobytes()


@pytest.mark.parametrize("tune", [dict(), dict(s3_zc=8), dict(s3_zc=5, s3_depth=2), dict(s3_gpr=16, s3_rpt=1),
                                  dict(s3_gpr=32, s3_rpt=2, s3_depth=3)])
def test_ring_of_window_planes_at_the_ends_of_the_buffer(tune):
    """Views that begin at the first and end at the last element of the buffer (window
    vectors beyond either end are read from the nearest vector inside), stencils that reach
    one plane only, walks cut into stretches of planes that do not divide the extent, more
    than one plane in flight."""
    rs = np.random.RandomState(43)
    hip.set_tune(**tune)
    try:
        for shape, dt in (((37, 21, 72), np.float32), ((19, 11, 36), np.float64), ((3, 3, 12), np.float32)):
            h = rs.uniform(-1, 1, shape).astype(dt)
            u = dr.array(h)
            for expr in (lambda a: a[:-1, :-1, :-4] + a[1:, 1:, 4:] - a[:-1, 1:, :-4],   # both ends
                         lambda a: a[:-2, 1:-1, 4:-4] + a[2:, 1:-1, 4:-4] * 2,           # planes only
                         lambda a: a[:-1, 1:, 4:] - a[1:, :-1, :-4]):                     # one plane
                low = hip.lower_only(expr(u))[0]
                assert low.kind == "tile3d" or shape[0] == 3, (shape, low.kind)
                got = expr(u).get()
                assert got.tobytes() == expr(h).tobytes(), (tune, shape, dt)
        h = rs.uniform(-1, 1, (67, 20, 40)).astype(np.float32)
        u, ref = dr.array(h), h.copy()
        launched = set(hip._KERNELS)
        for _ in range(2):
            u[1:-1, 1:-1, 1:-1] = _laplace3d(u)
            ref[1:-1, 1:-1, 1:-1] = _laplace3d(ref, c=np.float32(1 / 6.0))
        assert u.get().tobytes() == ref.tobytes()
        assert {k[0] for k in set(hip._KERNELS) - launched} <= {"tile3d"}
    finally:
        hip.set_tune(s3_zc=0, s3_depth=1, s3_gpr=64, s3_rpt=2)


def test_three_dimensional_stencil_layouts_that_do_not_qualify_still_match():
    rs = np.random.RandomState(42)
    h = rs.uniform(0, 1, (20, 30, 63)).astype(np.float32)       # row pitch not a multiple of 16 bytes
    u, ref = dr.array(h), h.copy()
    u[1:-1, 1:-1, 1:-1] = _laplace3d(u)
    ref[1:-1, 1:-1, 1:-1] = _laplace3d(ref, c=np.float32(1 / 6.0))
    assert u.get().tobytes() == ref.tobytes()
    hip.set_tune(s3=0)
    try:
        h = rs.uniform(0, 1, (20, 30, 64)).astype(np.float32)
        u, ref = dr.array(h), h.copy()
        u[1:-1, 1:-1, 1:-1] = _laplace3d(u)
        ref[1:-1, 1:-1, 1:-1] = _laplace3d(ref, c=np.float32(1 / 6.0))
        assert u.get().tobytes() == ref.tobytes()
    finally:
        hip.set_tune(s3=1)


# ---- device random numbers (Philox-4x64-10) ----------------------------------------------

@pytest.mark.parametrize("seed,counter", [(0, 0), (20261125, 0), ((1 << 128) - 1, (1 << 256) - 3),
                                          (5, (1 << 64) - 1000)])
def test_device_random_stream_is_numpys_philox(seed, counter):
    """Integer work, so bit-exact: raw outputs equal `Philox(key, counter).random_raw`,
    doubles equal `Generator(Philox).random`, over successive draws of awkward lengths
    (the stream position stops inside a block, the counter carries into the next word,
    the last elements go through the kernel's leftover and tail paths)."""
    gen = dr.random.device(seed, counter)
    ref = np.random.Generator(np.random.Philox(key=seed, counter=counter))
    for n in (1, 3, 4097, (1 << 20) + 3, 70001):
        raw = gen.random_raw(n).get()
        assert raw.dtype == np.int64
        assert np.array_equal(raw.view(np.uint64), ref.bit_generator.random_raw(n)), n
    for n in (5, 1 << 16, (1 << 18) + 1):
        assert np.array_equal(gen.random(n).get(), ref.random(n)), n
    assert np.array_equal(gen.uniform(-2.5, 7.0, 100003).get(), ref.uniform(-2.5, 7.0, 100003))
    assert np.array_equal(gen.random((33, 65)).get(), ref.random((33, 65)))
    # float32 numbers take half an output each, low half first, and an odd draw leaves the
    # high half of its last output to the next float32 draw, whatever is drawn in between
    for n, dt in ((7, np.float32), (5, np.float64), (1 << 16, np.float32), (3, np.int64), (70001, np.float32),
                  ((1 << 18) + 5, np.float32), (2, np.float32), ((17, 33), np.float32)):
        if dt == np.int64:
            assert np.array_equal(gen.random_raw(n).get().view(np.uint64), ref.bit_generator.random_raw(n))
            continue
        got, want = gen.random(n, dtype=dt).get(), ref.random(n, dtype=dt)
        assert got.dtype == want.dtype and np.array_equal(got, want), (n, dt)
    f = gen.random(1 << 12, dtype=np.float32)
    assert np.array_equal((f * 2 + 1).get(), ref.random(1 << 12, dtype=np.float32) * np.float32(2) + np.float32(1))


def test_device_random_numbers_fuse_without_memory_traffic():
    gen = dr.random.device(11)
    ref = np.random.Generator(np.random.Philox(key=11))
    n = 1 << 22
    u, v = gen.random(n), gen.random(n)
    inside = (u * u + v * v) < 1.0                  # Monte-Carlo pi: no array is ever stored
    low, _ = hip.lower_only(ReduceEx(np.add, inside))
    assert low.srcs == []
    launches = hip.STATS["launches"]
    hits = int(dr.sum(inside))
    assert hip.STATS["launches"] == launches + 2     # fused body + finalize
    a, b = ref.random(n), ref.random(n)
    assert hits == int(np.sum((a * a + b * b) < 1.0))
    # asked for on its own, or used in another shape, the node becomes an ordinary array
    w = gen.random(6000)
    col = w.reshape(6000, 1) * dr.array(np.ones((1, 3)))
    assert np.array_equal(col.get(), ref.random(6000)[:, None] * np.ones((1, 3)))
    x = gen.random(5000)
    y = x[10:20] + 1.0
    want = ref.random(5000)
    assert np.array_equal(y.get(), want[10:20] + 1.0) and np.array_equal(x.get(), want)


# ---- the short division and square root, on the device itself ---------------------------------

def test_short_division_and_square_root_are_within_one_ulp_on_the_device():
    """`dr_div_f8` and `dr_sqrt_near_f8` start from the hardware's reciprocal and reciprocal
    square root estimates, which the host build of the same source only imitates: here the
    device's own results, 2^22 random operands each over the whole exponent range and the
    special values, against NumPy's correctly rounded ones."""
    import struct
    from delayrepay_amd import hiprt, mathlib
    from delayrepay_amd.devarray import ndarray
    src = mathlib.source(["sqrt"], soft_div=True) + """
extern "C" __global__ void dr_kernel(const double* a, const double* b, double* q, double* r, long long n)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) { q[i] = dr_div_f8_1(a[i], b[i]); r[i] = dr_sqrt_near_f8_1(b[i]); }
}
"""
    fn = hiprt.get_function(hip._load_or_compile(src), "dr_kernel")
    rs = np.random.RandomState(31)
    n = 1 << 21
    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 5e-324, 1e-310, 2.2250738585072014e-308,
                        1.7976931348623157e308, 1e-250, 3.0])
    a = np.concatenate([rs.uniform(-100, 100, n), np.exp(rs.uniform(-300, 300, n)) * rs.choice([-1, 1], n),
                        np.repeat(special, special.size)])
    b = np.concatenate([rs.uniform(0.01, 100, n), np.exp(rs.uniform(-300, 300, n)), np.tile(special, special.size)])
    da, db = dr.array(a)._force(), dr.array(b)._force()
    q, r = ndarray(a.shape, np.float64), ndarray(a.shape, np.float64)
    args = struct.pack("@PPPPq", da.ptr, db.ptr, q.ptr, r.ptr, a.size)
    hiprt.launch(fn, -(-a.size // 256), 256, 0, args, len(args))
    with np.errstate(all="ignore"):
        for got, want in ((q.get(), a / b), (r.get(), np.sqrt(b))):
            assert np.array_equal(np.isnan(got), np.isnan(want))
            fin = np.isfinite(want)
            assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
            assert np.array_equal(np.signbit(got[fin]), np.signbit(want[fin]))
            off = np.abs(got[fin] - want[fin]) / np.spacing(np.abs(want[fin]))
            assert off.max() <= 1.0, off.max()
            assert np.count_nonzero(off) <= a.size // 20000, np.count_nonzero(off)
    # the float32 forms (packs of four): the hardware's reciprocal with one correction, and
    # its square root as it is
    from delayrepay_amd import mathlib32
    src = mathlib32.source([], soft_div=True) + """
extern "C" __global__ void dr_kernel(const float* a, const float* b, float* q, float* r, long long n)
{
    const long long i = 4 * ((long long)blockIdx.x * 256 + threadIdx.x);
    if (i + 4 <= n) {
        const float x[4] = {a[i], a[i + 1], a[i + 2], a[i + 3]}, y[4] = {b[i], b[i + 1], b[i + 2], b[i + 3]};
        float u[4], v[4];
        dr_div_f4_pack<4>(x, y, u); dr_sqrt_near_f4_pack<4>(y, v);
        for (int e = 0; e < 4; ++e) { q[i + e] = u[e]; r[i + e] = v[e]; }
    }
}
"""
    fn = hiprt.get_function(hip._load_or_compile(src), "dr_kernel")
    sp = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, 1e-40, 1.1754944e-38, 3.4028235e38,
                   1e-30, 3.0], dtype=np.float32)
    a4 = np.concatenate([rs.uniform(-100, 100, n), np.exp(rs.uniform(-80, 80, n)) * rs.choice([-1, 1], n),
                         np.repeat(sp, sp.size), [1.0, 1.0, 1.0]]).astype(np.float32)
    b4 = np.concatenate([rs.uniform(0.01, 100, n), np.exp(rs.uniform(-80, 80, n)), np.tile(sp, sp.size),
                         [1.0, 1.0, 1.0]]).astype(np.float32)
    assert a4.size % 4 == 0
    da, db = dr.array(a4)._force(), dr.array(b4)._force()
    q, r = ndarray(a4.shape, np.float32), ndarray(a4.shape, np.float32)
    args = struct.pack("@PPPPq", da.ptr, db.ptr, q.ptr, r.ptr, a4.size)
    hiprt.launch(fn, -(-a4.size // 1024), 256, 0, args, len(args))
    with np.errstate(all="ignore"):
        for got, want in ((q.get(), a4 / b4), (r.get(), np.sqrt(b4))):
            assert np.array_equal(np.isnan(got), np.isnan(want))
            fin = np.isfinite(want)
            assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
            assert np.array_equal(np.signbit(got[fin]), np.signbit(want[fin]))
            off = np.abs(got[fin].astype(np.float64) - want[fin]) / np.spacing(np.abs(want[fin])).astype(np.float64)
            assert off.max() <= 1.0, off.max()


# ---- quotients that only inexact functions read ---------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_quotients_inside_functions_and_quotients_that_are_results(dtype):
    """`log(a / b)`: the quotient is computed the short way (within one ulp), the result
    stays within the bar for functions; special operands give what NumPy gives.  The same
    quotient asked for as a result as well is the correctly rounded one, to the bit."""
    rs = np.random.RandomState(21)
    n = 1 << 18
    wide = 30 if dtype == np.float32 else 250
    a = np.concatenate([rs.uniform(0.01, 100, n), np.exp(rs.uniform(-wide, wide, n))]).astype(dtype)
    b = np.concatenate([rs.uniform(0.01, 100, n), np.exp(rs.uniform(-wide, wide, n))]).astype(dtype)
    special = np.array([0.0, -0.0, 1.0, np.inf, np.nan, 5e-324 if dtype == np.float64 else 1e-45,
                        np.finfo(dtype).max, np.finfo(dtype).tiny], dtype=dtype)
    a = np.concatenate([a, np.repeat(special, special.size)])
    b = np.concatenate([b, np.tile(special, special.size)])
    da, db = dr.array(a), dr.array(b)
    low, _ = hip.lower_only([np.log(da / db)])
    assert low.key[1][-1] == (0,)                                      # the quotient is marked
    with np.errstate(all="ignore"):
        ref = np.log(a / b)
        got = np.log(da / db).get()
        assert np.array_equal(np.isnan(got), np.isnan(ref))
        fin = np.isfinite(ref)
        assert np.array_equal(got[~fin & ~np.isnan(ref)], ref[~fin & ~np.isnan(ref)])
        # near log(1) = 0 one ulp of the quotient is many ulps of the logarithm, for NumPy's
        # quotient as for this one: the bar is on the quotient's scale there
        err = np.abs(got[fin].astype(np.float64) - ref[fin].astype(np.float64))
        eps = float(np.finfo(dtype).eps)
        bound = (2 if dtype == np.float32 else 450) * eps * np.maximum(np.abs(ref[fin]).astype(np.float64), 1.0)
        assert np.all(err <= bound), float(np.max(err / bound))
        q = da / db
        lg = np.log(q)
        dr.evaluate(lg, q)
        assert bits_equal(q.get(), a / b)
        both = np.log(da / db) + da / db           # seen through an addition: exact as well
        want = ref + a / b
        g2 = both.get()
        ok = np.isfinite(want)
        assert np.array_equal(np.isnan(g2), np.isnan(want))
        tol = (4 if dtype == np.float32 else 900) * eps * np.maximum(np.abs(want[ok]).astype(np.float64), 1.0)
        assert np.all(np.abs(g2[ok].astype(np.float64) - want[ok].astype(np.float64)) <= tol)


def test_device_random_draws_of_more_than_2_to_31_numbers():
    """One draw of 2^31 + 2^20 + 3 doubles (17 GB): positions are 64-bit, so the numbers
    around element 2^31 and the last ones equal NumPy's stream advanced to that place, and
    the draw after it continues where NumPy's would."""
    n = (1 << 31) + (1 << 20) + 3
    gen = dr.random.device(21)
    big = gen.random(n)
    big.run()

    def numpy_at(start, count):
        bits = np.random.Philox(key=21)
        bits.advance(start // 4)                    # four outputs per block
        return np.random.Generator(bits).random(start % 4 + count)[start % 4:]
    for start, count in ((0, 9), ((1 << 31) - 5, 11), (n - 7, 7)):
        assert np.array_equal(big[start:start + count].get(), numpy_at(start, count)), start
    assert np.array_equal(gen.random(6).get(), numpy_at(n, 6))
    total = float(dr.sum(big))
    assert abs(total / n - 0.5) < 1e-4


def test_two_dimensional_kernels_on_more_than_2_to_31_elements():
    """A 46400 x 46400 float32 matrix (2.15e9 elements, 8.6 GB) built on the device as
    `col[:, None] + row[None, :]`, so that NumPy can compute any entry: the tiled kernels
    (transpose, broadcast, stencil), the axis reductions, strided columns and the row kernel
    address rows and tiles on both sides of element 2^31 correctly."""
    N = M = 46400
    rs = np.random.RandomState(0)
    col = rs.standard_normal(N).astype(np.float32)
    row = rs.standard_normal(M).astype(np.float32)
    a = dr.array(col)[:, None] + dr.array(row)[None, :]
    a.run()

    def entries(i, j):
        return (col[i][:, None] + row[j][None, :]).astype(np.float32)
    I = np.array([0, 1, 46339, 46340, 46341, N - 2, N - 1])       # 2^31 / 46400 = 46282.4
    I = np.concatenate([I, [46281, 46282, 46283]])
    J = np.array([0, 5, 4095, 4096, M - 3, M - 1])
    t = hip.run(a.T * 2.0)
    assert np.array_equal(np.stack([t[j].get()[I] for j in J]), (entries(I, J) * 2).T)
    del t
    b = hip.run(a + dr.array(row))
    assert np.array_equal(np.stack([b[i].get()[J] for i in I]), entries(I, J) + row[J])
    del b
    st = hip.run(0.25 * (a[:-2, 1:-1] + a[2:, 1:-1] + a[1:-1, :-2] + a[1:-1, 2:]))
    ii, jj = np.array([0, 46280, 46281, 46282, 46283, N - 3]), np.array([0, 4094, 4095, M - 3])
    ref = np.float32(0.25) * (((entries(ii, jj + 1) + entries(ii + 2, jj + 1)) + entries(ii + 1, jj))
                              + entries(ii + 1, jj + 2))
    assert np.array_equal(np.stack([st[i].get()[jj] for i in ii]), ref)
    del st
    s0, s1 = dr.sum(a, axis=0).get(), dr.sum(a, axis=1).get()
    np.testing.assert_allclose(s0[J], col.astype(np.float64).sum() + N * row[J].astype(np.float64), rtol=1e-5, atol=0.5)
    np.testing.assert_allclose(s1[I], M * col[I].astype(np.float64) + row.astype(np.float64).sum(), rtol=1e-5, atol=0.5)
    v = hip.run(a[:, ::2] * 2.0)
    assert np.array_equal(np.stack([v[i].get()[J[:4] // 2] for i in I]), entries(I, (J[:4] // 2) * 2) * 2)
    del v
    r = hip.run(a[:, :4096] - a[:, :4096].max(axis=1, keepdims=True))
    assert np.array_equal(np.stack([r[i].get()[:64] for i in I]),
                          entries(I, np.arange(64)) - (col[I] + row[:4096].max())[:, None])


def test_three_dimensional_kernels_on_more_than_2_to_31_elements():
    """1300^3 float32 (2.2e9 elements) built on the device as x[i] + y[j] + z[k]: the
    transpose over all axes, the 7-point stencil and a reduction along the middle axis,
    checked at entries on both sides of element 2^31 (plane 1270.7)."""
    N = 1300
    rs = np.random.RandomState(1)
    x, y, z = (rs.standard_normal(N).astype(np.float32) for _ in range(3))
    a = (dr.array(x)[:, None, None] + dr.array(y)[None, :, None]) + dr.array(z)[None, None, :]
    a.run()

    def entries(i, j, k):
        return ((x[i][:, None, None] + y[j][None, :, None]) + z[k][None, None, :]).astype(np.float32)

    def pick(arr, I, J, K):
        return np.stack([np.stack([arr[i, j].get()[K] for j in J]) for i in I])
    I, J = np.array([0, 1269, 1270, 1271, 1272, N - 3]), np.array([0, 700, 1000, N - 3])
    K = np.array([0, 3, 4, 1023, 1024, N - 3])
    t = hip.run(a.T * 2.0)
    assert np.array_equal(pick(t, K, J, I), np.transpose(entries(I, J, K) * 2, (2, 1, 0)))
    del t
    st = hip.run((1.0 / 6.0) * (a[:-2, 1:-1, 1:-1] + a[2:, 1:-1, 1:-1] + a[1:-1, :-2, 1:-1]
                                + a[1:-1, 2:, 1:-1] + a[1:-1, 1:-1, :-2] + a[1:-1, 1:-1, 2:]))
    ref = np.float32(1.0 / 6.0) * (((((entries(I, J + 1, K + 1) + entries(I + 2, J + 1, K + 1))
                                      + entries(I + 1, J, K + 1)) + entries(I + 1, J + 2, K + 1))
                                    + entries(I + 1, J + 1, K)) + entries(I + 1, J + 1, K + 2))
    assert np.array_equal(pick(st, I, J, K), ref)
    del st
    s = dr.sum(a, axis=1).get()
    np.testing.assert_allclose(s[I][:, K], N * (x[I][:, None] + z[K][None, :]).astype(np.float64)
                               + y.astype(np.float64).sum(), rtol=1e-5, atol=0.5)


def test_types_without_a_device_form_are_widened_aloud_or_refused():
    """float16, int8, int16, uint16 and uint64 arrays are held as float32 / int64: every
    value is kept, the results have the wide type, and the first upload of each type says
    so.  What cannot be kept is refused: uint64 values of 2^63 and more, long double,
    complex numbers."""
    import warnings
    from delayrepay_amd import devarray
    rs = np.random.RandomState(5)
    for dt, wide in ((np.float16, np.float32), (np.int8, np.int64), (np.int16, np.int64),
                     (np.uint16, np.int64), (np.uint64, np.int64)):
        h = rs.standard_normal(1000) * 10
        h = (np.abs(h) if np.dtype(dt).kind == "u" else h).astype(dt)
        devarray._WIDENED.discard(np.dtype(dt).name)
        with pytest.warns(RuntimeWarning, match=np.dtype(dt).name):
            a = dr.array(h)
        with warnings.catch_warnings():
            warnings.simplefilter("error")              # said once per type
            b = dr.array(h)
        assert a.dtype == wide and b.dtype == wide
        got = (a * 3 + b).get()
        assert got.dtype == wide and np.array_equal(got, h.astype(wide) * 3 + h.astype(wide))
    with pytest.raises(OverflowError):
        dr.array(np.array([1, 2 ** 63], dtype=np.uint64))
    for bad in (np.ones(3, np.longdouble), np.ones(3, np.complex64), np.ones(3, np.complex128)):
        with pytest.raises(TypeError):
            dr.array(bad)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_row_reductions_with_an_operand_shared_by_a_batch(dtype):
    """`sum(x + m, axis=-1)` with x of shape (batch, rows, columns) and m (rows, columns):
    the kept dimensions are two levels that m does not walk as one sequence.  The row-wise
    reduction kernels (a lane, a lane group or a block per row) split the row number
    instead of leaving the case to the general wave-per-row kernel."""
    rs = np.random.RandomState(16)
    for (B, N, R), kind in (((40, 300, 8), "axis_short"), ((6, 200, 64), "axis_group"),
                            ((5, 210, 1000), "axis_group"), ((3, 7, 16384), "axis_block"),
                            ((1, 1500, 200), "axis_group")):
        x = rs.standard_normal((B, N, R)).astype(dtype)
        m = rs.standard_normal((N, R)).astype(dtype)
        v = rs.standard_normal((B, 1, R)).astype(dtype)
        dx, dm, dv = dr.array(x), dr.array(m), dr.array(v)
        low, _ = hip.lower_only(ReduceEx(np.add, dx + dm, (2,)))
        assert low.kind == kind, (B, N, R, low.kind)
        tol = dict(rtol=2e-5, atol=1e-4) if dtype == np.float32 else dict(rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(dr.sum(dx + dm, axis=-1).get(), (x + m).sum(axis=-1), **tol)
        np.testing.assert_allclose(dr.sum(dx * dv + dm, axis=2).get(), (x * v + m).sum(axis=2), **tol)
        assert np.array_equal(dr.max(dx + dm, axis=-1).get(), (x + m).max(axis=-1))
        assert np.array_equal(dr.min(dx[::2] * dv[::2], axis=-1).get(), (x[::2] * v[::2]).min(axis=-1))
        kd = dr.sum(dx + dm, axis=-1, keepdims=True).get()
        assert kd.shape == (B, N, 1)
        np.testing.assert_allclose(kd, (x + m).sum(axis=-1, keepdims=True), **tol)


def test_element_wise_work_on_short_rows_takes_the_row_kernel():
    """`points * scale + shift` with points (n, 3), standardising a few dozen features, an
    operand per batch item: rows of at most 4 KB with operands that repeat go through the
    row kernel without reductions (a lane group per row); bit-equal to NumPy.  A result
    that is constant along the rows (a column repeated), a destination with its own pitch,
    shifted views of one buffer and longer rows keep the tiled kernels."""
    rs = np.random.RandomState(17)
    for dtype in (np.float32, np.float64, np.int32):
        for n, R in ((100003, 3), (5000, 8), (4099, 33), (1000, 64), (513, 200), (130, 500)):
            mk = (lambda *s: rs.standard_normal(s).astype(dtype)) if dtype != np.int32 else \
                 (lambda *s: rs.randint(-50, 50, s).astype(dtype))
            x, v, c = mk(n, R), mk(R), mk(n, 1)
            dx, dv, dc = dr.array(x), dr.array(v), dr.array(c)
            ex = dx * dv + dc
            assert hip.lower_only(ex)[0].kind == "rows", (dtype, n, R)
            assert bits_equal(ex.get(), x * v + c)
            p, q = dr.evaluate(dx - dv, (dx + dc) * dv)                   # two results, one kernel
            assert bits_equal(p.get(), x - v) and bits_equal(q.get(), (x + c) * v)
            assert bits_equal((dx[::2] * dv > dc[::2]).get(), x[::2] * v > c[::2])      # masks
            if dtype != np.int32:
                assert bits_equal((dx / dv).get(), x / v)
    # batches: an operand per item, one shared by all items
    x, m, w = rs.standard_normal((7, 50, 40)), rs.standard_normal((50, 40)), rs.standard_normal((7, 1, 40))
    dx, dm, dw = dr.array(x), dr.array(m), dr.array(w)
    assert hip.lower_only(dx * dw + dm)[0].kind == "rows"
    assert bits_equal((dx * dw + dm).get(), x * w + m)
    # images with few pixels per channel: a value per channel, rows of 7 x 7 merged
    img = rs.standard_normal((6, 20, 7, 7)).astype(np.float32)
    g, b = rs.standard_normal((1, 20, 1, 1)).astype(np.float32), rs.standard_normal((20, 1, 1)).astype(np.float32)
    di, dg, db = dr.array(img), dr.array(g), dr.array(b)
    low = hip.lower_only(np.maximum(di * dg + db, 0.0))[0]
    assert low.kind == "rows" and low.tail[0] == 120 and low.key[5] == 49
    assert bits_equal(np.maximum(di * dg + db, 0.0).get(), np.maximum(img * g + b, np.float32(0.0)))
    # what stays with the tiled kernels
    c = rs.standard_normal((300, 1))
    dc = dr.array(c)
    rep = dc * 2.0 + dr.zeros((300, 5))
    assert bits_equal(np.repeat(dr.array(c[:, 0]), 5).get(), np.repeat(c[:, 0], 5))
    a = rs.standard_normal((64, 100))
    da = dr.array(a)
    assert hip.lower_only(da[:, 1:] - da[:, :-1])[0].kind.startswith("tile2d")   # shifted views, 792 bytes
    assert bits_equal((da[:, 1:] - da[:, :-1]).get(), a[:, 1:] - a[:, :-1])
    wide = rs.standard_normal((40, 1300)).astype(np.float32)
    other = rs.standard_normal((40, 1300))
    col = rs.standard_normal((40, 1))
    mixed = dr.array(wide) * dr.array(other) + dr.array(col)
    assert hip.lower_only(mixed)[0].kind == "tile2d"                          # longer rows, mixed types
    assert bits_equal(mixed.get(), wide * other + col)
    dst = dr.zeros((64, 60))
    dst[:, 4:52] = da[:, :48] * dr.array(c[:64])                                 # its own pitch
    ref = np.zeros((64, 60)); ref[:, 4:52] = a[:, :48] * c[:64]
    assert bits_equal(dst.get(), ref)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_transposes_of_matrices_with_one_short_side(dtype):
    """Points as rows of a few coordinates and the coordinate vectors (`pts.T`): the
    transposing tiles are fitted to the short side (4 to 16 rows of the operand by 256, or
    256 by 4 to 32 columns); a short side of at most 16 that is no power of two takes a lane
    per index of the long side instead of a tile.  Bit-equal to NumPy for every short extent,
    with a second operand and with a batch in front."""
    rs = np.random.RandomState(18)
    for n, R in ((100003, 2), (100003, 3), (70001, 4), (30011, 7), (20000, 8), (9973, 12), (5000, 16),
                 (4099, 24), (3001, 32)):
        x = (rs.standard_normal((n, R)) * 50).astype(dtype)
        other = (rs.standard_normal((R, n)) * 50).astype(dtype)
        dx, do = dr.array(x), dr.array(other)
        low, _ = hip.lower_only(dx.T * 2)
        assert low.kind == ("tile2dt" if R & (R - 1) == 0 or R > 16 else "thin_t"), (n, R)
        assert bits_equal((dx.T * 2).get(), x.T * 2)
        assert bits_equal((dx.T + do).get(), x.T + other)            # with an operand read directly
        assert bits_equal((do.T * 2).get(), other.T * 2)             # the short side first
        assert bits_equal((do.T - dx).get(), other.T - x)
    b = (rs.standard_normal((5, 4001, 3)) * 50).astype(dtype)
    assert bits_equal((dr.transpose(dr.array(b), (0, 2, 1)) * 2).get(), b.transpose(0, 2, 1) * 2)


def test_element_wise_work_on_short_rows_written_into_existing_arrays():
    """`x[...] = x * v + c` over its own operand, a destination that is a view with a pitch
    (`y[:, :2] = ...`), a dense preallocated result: the row kernel writes them as it writes
    new arrays; a destination whose rows are on two levels keeps the tiled kernel.  Bit-equal
    to NumPy, repeated so that every sweep reads what the one before wrote."""
    rs = np.random.RandomState(21)
    for dtype in (np.float32, np.float64):
        for n, R in ((100003, 3), (4099, 33), (1000, 64), (513, 200)):
            x = rs.standard_normal((n, R)).astype(dtype)
            v = rs.uniform(0.5, 1.5, R).astype(dtype)
            c = rs.standard_normal((n, 1)).astype(dtype)
            dx, dv, dc = dr.array(x), dr.array(v), dr.array(c)
            for _ in range(3):
                before = hip.STATS["launches"]
                dx[...] = dx * dv + dc
                assert hip.STATS["launches"] == before + 1
                x[...] = x * v + c
            assert bits_equal(dx.get(), x)
            y, dy = np.zeros((n, R + 5), dtype), dr.zeros((n, R + 5), dtype=dtype)
            dy[:, 2:R + 2] = dx * dv
            y[:, 2:R + 2] = x * v
            assert bits_equal(dy.get(), y)
            k = max(1, R // 2)
            dy[:, :k] = dy[:, :k] * 2 + dc                      # a view over itself
            y[:, :k] = y[:, :k] * 2 + c
            assert bits_equal(dy.get(), y)
            dy[1:, 1:R + 1] = dx[:-1] - dv                     # rows shifted against the operand
            y[1:, 1:R + 1] = x[:-1] - v
            assert bits_equal(dy.get(), y)
    cube, dcube = np.zeros((4, 20, 40)), dr.zeros((4, 20, 40))
    src = rs.standard_normal((4, 16, 32))
    dcube[:, 2:18, 4:36] = dr.array(src) * 2.0                   # rows on two levels
    cube[:, 2:18, 4:36] = src * 2.0
    assert bits_equal(dcube.get(), cube)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_weighted_sums_of_the_rows_of_a_narrow_matrix(dtype):
    """`(points * w[:, None]).sum(axis=0)`: a centroid, a weighted mean of a few features.
    The matrix is read as one stream (`axis_narrow`) with the weight of each row beside
    it, instead of a lane per column walking rows a pitch apart."""
    rs = np.random.RandomState(22)
    for n, R in ((200003, 3), (100000, 2), (50001, 8), (30000, 16), (9000, 33), (5000, 64), (4100, 96),
                 (4100, 128)):
        x = rs.standard_normal((n, R)).astype(dtype)
        w = rs.uniform(0, 1, n).astype(dtype)
        v = rs.standard_normal(R).astype(dtype)
        dx, dw, dv = dr.array(x), dr.array(w), dr.array(v)
        low, _ = hip.lower_only(ReduceEx(np.add, dx * dw[:, None], (0,)))
        assert low.kind == "axis_narrow" and "c" in low.key[2], (n, R, low.kind)
        tol = dict(rtol=2e-4, atol=2e-2) if dtype == np.float32 else dict(rtol=1e-11, atol=1e-9)
        np.testing.assert_allclose(dr.sum(dx * dw[:, None], axis=0).get(), (x * w[:, None]).sum(axis=0), **tol)
        np.testing.assert_allclose(dr.sum((dx - dv) * dw.reshape(n, 1) + dv, axis=0).get(),
                                   ((x - v) * w.reshape(n, 1) + v).sum(axis=0), **tol)
        assert np.array_equal(dr.max(dx * dw[:, None], axis=0).get(), (x * w[:, None]).max(axis=0))
        mean = dr.sum(dx * dw[:, None], axis=0) / dr.sum(dw)
        np.testing.assert_allclose(np.asarray(mean.get()), (x * w[:, None]).sum(axis=0) / w.sum(),
                                   rtol=1e-3 if dtype == np.float32 else 1e-10, atol=1e-3 if dtype == np.float32 else 1e-10)


def test_shifted_views_of_a_matrix_with_short_rows():
    """`x[:, 1:] - x[:, :-1]` and a 5-point stencil on rows of at most 384 bytes: the tiled
    kernel's LDS window is 256 columns wide, so the row kernel reads the views one by one
    from the caches instead; wider rows and volumes keep their LDS windows.  Bit-equal."""
    rs = np.random.RandomState(23)
    for n, R, kind in ((100003, 3, "rows"), (20011, 16, "rows"), (5003, 64, "rows"), (3001, 96, "rows"),
                       (2000, 200, "tile2d")):
        x = rs.standard_normal((n, R)).astype(np.float32)
        dx = dr.array(x)
        d = dx[:, 1:] - dx[:, :-1]
        assert hip.lower_only(d)[0].kind == kind, (n, R)
        assert bits_equal(d.get(), x[:, 1:] - x[:, :-1])
        if R >= 3:
            lap = 0.25 * (dx[:-2, 1:-1] + dx[2:, 1:-1] + dx[1:-1, :-2] + dx[1:-1, 2:])
            ref = np.float32(0.25) * (((x[:-2, 1:-1] + x[2:, 1:-1]) + x[1:-1, :-2]) + x[1:-1, 2:])
            assert bits_equal(lap.get(), ref)
        for _ in range(2):                       # written back over the matrix: a hazard, not in place
            dx[:, 1:] = dx[:, 1:] - dx[:, :-1]
            x[:, 1:] = x[:, 1:] - x[:, :-1]
        assert bits_equal(dx.get(), x)


def test_vectors_stacked_as_the_columns_of_a_matrix_are_one_kernel():
    """`stack([x, y, z], axis=-1)` (coordinates into points) is one lazy expression over a
    column number, written row by row by the row kernel and fused with what reads it;
    bit-equal to NumPy's stack, also for arrays of more dimensions and mixed types."""
    rs = np.random.RandomState(24)
    n = 100003
    for dtype in (np.float32, np.float64, np.int32):
        cols = [(rs.standard_normal(n) * 100).astype(dtype) for _ in range(3)]
        dcols = [dr.array(c) for c in cols]
        st = dr.stack(dcols, axis=1)
        assert "array" not in st.__dict__ and st.shape == (n, 3) and st.dtype == dtype
        got, launched = hip.STATS["launches"], None
        out = st.get()
        assert hip.STATS["launches"] == got + 1 and bits_equal(out, np.stack(cols, axis=1))
        fused = (dr.stack(dcols, axis=-1) * 2).get()
        assert bits_equal(fused, np.stack(cols, axis=-1) * 2)
    a, b = rs.standard_normal((7, 50)), rs.randint(0, 9, (7, 50))
    got = np.stack([dr.array(a), dr.array(b)], axis=-1).get()
    ref = np.stack([a, b], axis=-1)
    assert got.dtype == ref.dtype and bits_equal(got, ref)
    eight = [rs.standard_normal(1000).astype(np.float32) for _ in range(8)]
    assert bits_equal(dr.stack([dr.array(e) for e in eight], axis=1).get(), np.stack(eight, axis=1))
    nine = eight + [eight[0]]
    assert bits_equal(dr.stack([dr.array(e) for e in nine], axis=1).get(), np.stack(nine, axis=1))
    assert bits_equal(dr.stack([dr.array(e) for e in eight[:3]], axis=0).get(), np.stack(eight[:3], axis=0))
