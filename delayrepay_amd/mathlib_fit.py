"""Prints the polynomial coefficients used in `mathlib.py` (needs mpmath).

    python -m delayrepay_amd.mathlib_fit [--tables]

Each fit is a weighted least-squares fit on Chebyshev nodes in 50-digit arithmetic;
the error printed beside it is measured with the coefficients rounded to double.
Coefficients are listed from the constant term up; `mathlib.py` uses them in Horner
order (highest first)."""
import math

import mpmath as mp

mp.mp.dps = 50


def fit(f, w, a, b, deg, var=lambda x: x):
    """Polynomial of degree `deg` in var(x) minimising sum (w(x) (p - f(x)))^2 over
    8 (deg + 1) Chebyshev nodes of [a, b]."""
    nodes = 8 * (deg + 1)
    xs = [(a + b) / 2 + (b - a) / 2 * mp.cos(mp.pi * (2 * k + 1) / (2 * nodes))
          for k in range(nodes)]
    A = mp.matrix(nodes, deg + 1)
    y = mp.matrix(nodes, 1)
    for i, x in enumerate(xs):
        wi, t, p = w(x), var(x), mp.mpf(1)
        for j in range(deg + 1):
            A[i, j] = wi * p
            p *= t
        y[i] = wi * f(x)
    c = mp.qr_solve(A, y)[0]
    return [c[j] for j in range(deg + 1)]


def worst(f, w, c, a, b, var=lambda x: x, n=4000):
    """max w(x) |p(x) - f(x)| on a grid, with the coefficients rounded to double."""
    c = [mp.mpf(float(x)) for x in c]
    m = mp.mpf(0)
    for k in range(n + 1):
        x = a + (b - a) * mp.mpf(k) / n
        p = mp.mpf(0)
        for cj in reversed(c):
            p = p * var(x) + cj
        m = max(m, abs(w(x) * (p - f(x))))
    return m


def show(name, c, err):
    print(f"{name}: error {mp.nstr(err, 3)}")
    for x in c:
        print("   ", float(x).hex())


def main():
    zero, one = mp.mpf(0), mp.mpf(1)
    # e^v - 1 = v + v^2 R(v) on |v| <= ln(2)/2; an error dR changes it by v^2 dR, relative
    # to e^v - 1 ~ v that is |v| dR (the small constant keeps the fit determined at 0)
    h = mp.log(2) / 2

    def fr(v):
        if v == 0:
            return one / 2
        return (mp.expm1(v) - v) / (v * v)
    c = fit(fr, lambda v: abs(v) + mp.mpf(10) ** -3, -h, h, 9)
    show("exp, R(v), |v| <= ln(2)/2 (relative error of e^v - 1)", c,
         worst(fr, lambda v: abs(v), c, -h, h))
    # log1p(r) = r + r^2 Q(r) for |r| < 2^-9 (the largest r the table of `log_table` leaves);
    # an error dQ changes the result by r^2 dQ, relative to log1p(r) ~ r that is |r| dQ
    rmax = mp.mpf(2) ** -9

    def fq(r):
        if r == 0:
            return -one / 2
        return (mp.log1p(r) - r) / (r * r)
    c = fit(fq, lambda r: abs(r) + mp.mpf(10) ** -6, -rmax, rmax, 4)
    show("log, Q(r), |r| <= 2^-9 (relative error of log1p(r))", c,
         worst(fq, lambda r: abs(r), c, -rmax, rmax))
    ln2_hi = mp.mpf(float.fromhex("0x1.62e42fee00000p-1"))
    print("ln 2 =", float(ln2_hi).hex(), "+", float(mp.log(2) - ln2_hi).hex(),
          "; 1 / ln 2 =", float(1 / mp.log(2)).hex())


LOG_INTERVALS, LOG_CENTRE = 256, 150
LOG_OFF = 0x3ff0000000000000 - (2 * LOG_CENTRE + 1) * (1 << 43)    # bits of 0.7060546875


def _double(bits):
    import struct
    return struct.unpack("<d", struct.pack("<Q", bits))[0]


def log_interval(i):
    """Ends of interval i of `dr_log_core`: the doubles whose bit pattern minus LOG_OFF has
    i in its bits 44..51.  Interval LOG_CENTRE is [1 - 2^-10, 1 + 2^-9): 1.0 is its centre
    in the bit pattern."""
    return _double(LOG_OFF + i * (1 << 44)), _double(LOG_OFF + (i + 1) * (1 << 44))


def log_table():
    """(1/c, log c) per interval.  c starts at the centre of the interval and is moved, by
    less than 2^-23 of itself, to a point where log(c) is a double to within 0.004 ulp, so
    that the table adds no rounding error of its own; the interval around 1 has c = 1."""
    import struct
    old = mp.mp.dps
    mp.mp.dps = 70
    table = []
    for i in range(LOG_INTERVALS):
        if i == LOG_CENTRE:
            table.append((1.0, 0.0))
            continue
        lo, hi = (mp.mpf(v) for v in log_interval(i))
        start = struct.unpack("<Q", struct.pack("<d", float(2 / (lo + hi))))[0]
        best = None
        for stride in (1, 1021, 65537, 1048583):
            for d in range(-400, 401):
                invc = _double(start + d * stride)
                exact = -mp.log(mp.mpf(invc))
                logc = float(exact)
                err = abs(exact - mp.mpf(logc)) / mp.mpf(math.ulp(logc))
                if best is None or err < best[0]:
                    best = (err, invc, logc)
            if best[0] < 0.004:
                break
        table.append(best[1:])
    mp.mp.dps = old
    return table


ERF_PER_UNIT, ERF_DEGREE, ERF_TOP = 16, 8, 6


def erf_table():
    """Rows (c, a0..a8) of `dr_erf_f8`: on [i/16, (i+1)/16) erf(x) ~ sum a_j (x - c)^j, a
    least-squares fit under the weight 1/erf (relative error); c is a point near the middle
    of the interval at which erf(c) is a double to within 0.25 ulp (found by stepping through
    nearby doubles), and a0 = erf(c).  Row 0 is centred on 0 and fits erf(x)/x, so its
    constant term is exactly 0 and tiny arguments keep their relative accuracy."""
    import struct
    old = mp.mp.dps
    mp.mp.dps = 60
    width = mp.mpf(1) / ERF_PER_UNIT
    rows = []
    for i in range(ERF_TOP * ERF_PER_UNIT):
        a, b = i * width, (i + 1) * width
        if i == 0:
            g = lambda x: mp.erf(x) / x if x != 0 else 2 / mp.sqrt(mp.pi)
            coef = [mp.mpf(0)] + fit(g, lambda x: 1 / g(x), a, b, ERF_DEGREE - 1)
            rows.append([0.0] + [float(v) for v in coef])
            continue
        start = struct.unpack("<Q", struct.pack("<d", float((a + b) / 2)))[0]
        best = None
        for stride in (4099, 1 << 24, 1 << 32, 1 << 38, 1 << 42):
            for d in range(-300, 301):
                cand = _double(start + d * stride)
                if not float(a) + 1 / 128 < cand < float(b) - 1 / 128:
                    continue
                exact = mp.erf(mp.mpf(cand))
                err = abs(exact - mp.mpf(float(exact))) / mp.mpf(math.ulp(float(exact)))
                if best is None or err < best[0]:
                    best = (err, cand)
            if best[0] < 0.01:
                break
        c = mp.mpf(best[1])
        coef = fit(mp.erf, lambda x: 1 / mp.erf(x), a, b, ERF_DEGREE, lambda x: x - c)
        coef[0] = mp.erf(c)
        rows.append([best[1]] + [float(v) for v in coef])
    mp.mp.dps = old
    return rows


if __name__ == "__main__":
    import sys
    main()
    if "--tables" in sys.argv:          # takes a few minutes
        print("log table, 1/c and log(c) per interval:")
        for invc, logc in log_table():
            print(f"    {invc.hex()}, {logc.hex()},")
        print("erf table, c and the coefficients of degree 0..8 per interval:")
        for row in erf_table():
            print("    " + ", ".join(v.hex() for v in row) + ",")
