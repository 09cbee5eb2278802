"""Prints the polynomial coefficients used in `mathlib.py` (needs mpmath).

    python -m delayrepay_amd.mathlib_fit

Each fit is a weighted least-squares fit on Chebyshev nodes in 50-digit arithmetic;
the error printed beside it is measured with the coefficients rounded to double.
Coefficients are listed from the constant term up; `mathlib.py` uses them in Horner
order (highest first)."""
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
    # erf(x) = -expm1(-w), w = -log(erfc(x)) = x (x + 1 + H(x)) on [0, 6].  An error dH
    # changes erf by erfc(x) x dH: the weight makes that relative to erf(x).
    def fh(x):
        if x == 0:
            return 2 / mp.sqrt(mp.pi) - 1
        return -mp.log(mp.erfc(x)) / x - x - 1

    def wh(x):
        if x == 0:
            return mp.sqrt(mp.pi) / 2
        return mp.erfc(x) * x / mp.erf(x)
    c = fit(fh, wh, zero, mp.mpf(6), 23)
    show("erf, 0 <= x <= 6, H(x) (relative error of erf)", c, worst(fh, wh, c, zero, mp.mpf(6)))
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
    # log((1+s)/(1-s)) = 2s + s z Q(z), z = s^2, s <= (sqrt(2)-1)/(sqrt(2)+1)
    smax = (mp.sqrt(2) - 1) / (mp.sqrt(2) + 1)

    def fl(z):
        if z == 0:
            return mp.mpf(2) / 3
        s = mp.sqrt(z)
        return (mp.log((1 + s) / (1 - s)) - 2 * s) / s / z
    c = fit(fl, lambda z: one, zero, smax ** 2, 6)
    show("log, Q(z) (absolute error of R = z Q)", c, worst(fl, lambda z: z, c, zero, smax ** 2))
    ln2_hi = mp.mpf(float.fromhex("0x1.62e42fee00000p-1"))
    print("ln 2 =", float(ln2_hi).hex(), "+", float(mp.log(2) - ln2_hi).hex(),
          "; 1 / ln 2 =", float(1 / mp.log(2)).hex())


if __name__ == "__main__":
    main()
