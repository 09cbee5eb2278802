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
    # erf(x) = x P(x^2) on [0, 1], relative error; the code adds x separately, so the
    # constant term is stored minus 1
    fa = lambda z: mp.erf(mp.sqrt(z)) / mp.sqrt(z) if z > 0 else 2 / mp.sqrt(mp.pi)
    wa = lambda z: 1 / fa(z)
    c = fit(fa, wa, zero, one, 12)
    show("erf, |x| < 1, P(z) - 1 with z = x^2 (relative)", [c[0] - 1] + c[1:], worst(fa, wa, c, zero, one))
    # erfc(x) = exp(-(x^2 + G(x - 3.5))) on [1, 6]; weight erfc(x): absolute error of erf
    gb = lambda x: -mp.log(mp.erfc(x)) - x * x
    tv = lambda x: x - mp.mpf(7) / 2
    c = fit(gb, mp.erfc, one, mp.mpf(6), 18, tv)
    show("erf, 1 <= x <= 6, G(t) with t = x - 3.5 (absolute error of erfc)", c,
         worst(gb, mp.erfc, c, one, mp.mpf(6), tv))
    # exp(v) on |v| <= ln(2)/2, relative
    h = mp.log(2) / 2
    c = fit(mp.exp, lambda v: mp.exp(-v), -h, h, 11)
    show("exp(v), |v| <= ln(2)/2 (relative)", c, worst(mp.exp, lambda v: mp.exp(-v), c, -h, h))
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
