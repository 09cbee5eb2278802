"""NumPy oracle: what the reference's CPU backend computes.

TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg import this module; the delayrepay_amd package never
does.

The reference's CPU backend (delayrepay/cpu.py:12-31) evaluates a DAG by applying
each node's stored NumPy ufunc to its evaluated children (`node.func(*children)`,
cpu.py:19-26); leaves are the arrays and Python scalars themselves
(cpu.py:13-17).  Before that, the front end rewrites three things
(delayrepay/delayarray.py:316-336): `square(x)` becomes `multiply(x, x)`, and
`x ** k` for a Python-int k becomes k-1 left-associated multiplies (k <= 1 gives
x there; the restatement keeps that for k = 1 only and follows NumPy for k <= 0,
where returning x is plainly a slip: x**0 would be x).  Hence the reference's value of an expression is the value of the same Python
expression evaluated eagerly, node by node, on numpy.ndarrays with those rewrites
applied.  `OracleArray` is exactly that evaluator; the named functions below state
the five benchmark configurations directly in NumPy.

How each piece is pinned (see tests/test_oracle.py):
  OracleArray rewrites  the reference's own test expressions (tests/test.py:21-67,
                        79-85, 102-111, 122-124) against closed-form answers;
                        x**3 against the explicit left-associated product
  saxpy, horner, jacobi bit-exact against the independent C restatement in
                        dr_oracle.c (compiled with -ffp-contract=off); jacobi also
                        against a pure-Python loop on a small grid and the
                        fixed-point / zero-boundary invariants
  black_scholes         put-call parity C - P = S - K exp(-rT); mpmath at 50 digits
                        on sampled points; the C restatement (libm) within 1e-13
  sumsq                 math.fsum (exactly rounded sum) within 1e-13 relative
Parity unpinned by the reference itself: it ships no golden vectors; bit-level
results, erf, the stencil and the fused reduction are pinned only by the checks
above.
"""
import numpy as np
import numpy.lib.mixins

try:
    from scipy.special import erf as _erf
except ImportError:  # pragma: no cover
    _erf = None

INV_SQRT2 = 0.7071067811865476


class OracleArray(numpy.lib.mixins.NDArrayOperatorsMixin):
    """Eager node-by-node NumPy evaluation with the reference's rewrites."""

    def __init__(self, arr):
        self.a = arr.a if isinstance(arr, OracleArray) else np.asarray(arr)

    @property
    def shape(self):
        return self.a.shape

    @property
    def dtype(self):
        return self.a.dtype

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        if method != "__call__":
            return NotImplemented
        kwargs.pop("out", None)   # `x += y` rebinds, as in the reference (delayarray.py:46,60-61)
        args = [x.a if isinstance(x, OracleArray) else x for x in inputs]
        name = ufunc.__name__
        if name == "square":                                   # delayarray.py:330-331
            return OracleArray(np.multiply(args[0], args[0]))
        if name == "power" and isinstance(args[1], int) and not isinstance(args[1], bool):
            if args[1] < 1:
                # the reference returns x itself for k <= 1 (delayarray.py:316-324), which
                # is x**1; for k <= 0 the restatement follows NumPy's `**` instead
                return OracleArray(np.asarray(args[0]) ** args[1])
            acc = args[0]                                      # delayarray.py:316-324
            for _ in range(args[1] - 1):
                acc = np.multiply(acc, args[0])
            return OracleArray(acc)
        return OracleArray(ufunc(*args))                       # cpu.py:19-26

    def __array_function__(self, func, types, args, kwargs):
        args = [x.a if isinstance(x, OracleArray) else x for x in args]
        res = func(*args, **kwargs)
        return OracleArray(res) if isinstance(res, np.ndarray) and res.ndim else res

    def __getitem__(self, key):                                # delayarray.py:123-128 (views)
        return OracleArray(self.a[key])

    def __setitem__(self, key, item):                          # delayarray.py:114-121
        self.a[key] = item.a if isinstance(item, OracleArray) else item

    def astype(self, dtype):
        return OracleArray(self.a.astype(dtype))

    def sum(self):                                             # delayarray.py:516-518
        return np.sum(self.a)

    def get(self):
        return self.a

    def __array__(self, dtype=None, copy=None):
        return self.a if dtype is None else self.a.astype(dtype)


# ---- the five benchmark configurations, stated directly in NumPy -------------

def saxpy(a, x, y):
    """z = a*x + y with a Python-float `a` (weak scalar: stays in x's dtype)."""
    return np.add(np.multiply(a, x), y)


def horner(coeffs, x):
    """((c8*x + c7)*x + ...)*x + c0; coefficients are Python floats."""
    acc = np.add(np.multiply(coeffs[-1], x), coeffs[-2])
    for c in reversed(coeffs[:-2]):
        acc = np.add(np.multiply(acc, x), c)
    return acc


def black_scholes_expr(xp, S, K, T, r, sigma):
    """The fixed Black-Scholes source; `xp` supplies sqrt/log/exp/erf so the same
    text builds either NumPy values or a lazy DAG."""
    erf = getattr(xp, "erf", _erf)
    sqT = xp.sqrt(T)
    vs = sigma * sqT
    d1 = (xp.log(S / K) + (r + 0.5 * sigma * sigma) * T) / vs
    d2 = d1 - vs
    N1 = 0.5 * (1 + erf(d1 * INV_SQRT2))
    N2 = 0.5 * (1 + erf(d2 * INV_SQRT2))
    disc = K * xp.exp((-r) * T)
    call = S * N1 - disc * N2
    put = disc * (1 - N2) - S * (1 - N1)
    return call, put


class _NumpyWithErf:
    sqrt, log, exp = np.sqrt, np.log, np.exp
    erf = staticmethod(_erf)


def black_scholes(S, K, T, r, sigma):
    return black_scholes_expr(_NumpyWithErf, S, K, T, r, sigma)


def jacobi(u, sweeps):
    """5-point Jacobi on the interior, association ((up+down)+left)+right, then
    0.25*; the right-hand side is a temporary, so every sweep reads the old grid
    (delayarray.py:114-121)."""
    u = np.array(u, copy=True)
    for _ in range(sweeps):
        rhs = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        u[1:-1, 1:-1] = rhs
    return u


def sumsq(x, y, w):
    """sum((x - y)**2 * w) with **2 as d*d (delayarray.py:316-324) and NumPy's
    pairwise summation (delayarray.py:516-518 -> numpy.sum)."""
    d = np.subtract(x, y)
    return np.sum(np.multiply(np.multiply(d, d), w))


# ---- input generation shared by tests and bench (RNG convention of the configurations) ------

def make_inputs(config, n=None, seed=0):
    """Host inputs of a benchmark configuration: numpy.random.RandomState(seed),
    float64 draws in the listed order, cast to the configuration's dtype."""
    rs = np.random.RandomState(seed)
    if config == "saxpy":
        n = n or 1 << 24
        x = rs.uniform(-1, 1, n).astype(np.float32)
        y = rs.uniform(-1, 1, n).astype(np.float32)
        return {"a": 2.0, "x": x, "y": y}
    if config == "horner":
        n = n or 1 << 26
        c = rs.uniform(-1, 1, 9).astype(np.float32)
        x = rs.uniform(-2, 2, n).astype(np.float32)
        return {"c": [float(v) for v in c], "x": x}
    if config in ("bs32", "bs64"):
        n = n or 1 << 25
        dt = np.float32 if config == "bs32" else np.float64
        S = rs.uniform(5, 30, n).astype(dt)
        K = rs.uniform(1, 100, n).astype(dt)
        T = rs.uniform(0.25, 10, n).astype(dt)
        return {"S": S, "K": K, "T": T, "r": 0.02, "sigma": 0.30}
    if config == "jacobi":
        n = n or 8192
        u = np.zeros((n, n), np.float32)
        u[1:-1, 1:-1] = rs.uniform(0, 1, (n - 2, n - 2))
        return {"u": u, "sweeps": 10}
    if config == "sumsq":
        n = n or 1 << 27
        x = rs.standard_normal(n)
        y = rs.standard_normal(n)
        w = rs.uniform(0, 1, n)
        return {"x": x, "y": y, "w": w}
    raise KeyError(config)
