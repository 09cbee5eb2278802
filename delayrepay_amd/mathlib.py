"""Double-precision `log`, `erf` and `exp` for the generated kernels.

The device library's versions cost 97, 105 and 41 vector instructions per element
(counted in gfx950 code), which makes a Black-Scholes kernel in float64 wait on the
fp64 pipes rather than on memory.  These cost 43, 64 and 25.  About half of the
difference is the polynomials themselves; the other half is how a Horner step is
issued, see `DR_FMA_K`.  Accuracy against 40-digit references
(`tests/test_mathlib.py` builds this same source for the host): log <= 0.8 ulp over
the whole range including denormals, erf and exp <= 1 ulp; special values (zeros,
infinities, NaN, negative arguments, overflow, gradual underflow) follow C99.
float32 keeps the device library's functions.

`log` is the classic reduction x = 2^k m, m in [sqrt(1/2), sqrt(2)), s = f/(2+f) with
f = m-1, log(1+f) = f - (f^2/2 - s (f^2/2 + R(s^2))).  `exp` is 2^k e^v with
k = rint(x / ln 2).  `erf` is x + x P(x^2) below 1 and 1 - exp(-(x^2 + G(x - 3.5)))
above, with G a polynomial for -log(erfc(x)) - x^2 on [1, 6] fitted under the weight
erfc(x) (the absolute error of the result is what matters there).  The coefficients
are least-squares fits on Chebyshev nodes in 50-digit arithmetic, printed by
`mathlib_fit.py` next to this file.
"""

DEVICE_MACROS = """\
#define DR_FN static __device__ __forceinline__
#define DR_RCP64(d) __builtin_amdgcn_rcp(d)
/* p * z + k with the constant k in a scalar register pair.  The compiler prefers the
   two-address v_fmac_f64 for a Horner step and then copies every 64-bit constant into
   the accumulator with two v_mov_b32, which doubles the cost of a polynomial. */
#define DR_FMA_K(p, z, k) ({ double dr_r_; \\
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(dr_r_) : "v"(p), "v"(z), "s"((double)(k))); dr_r_; })
"""

HOST_MACROS = """\
#define DR_FN static inline
#define DR_RCP64(d) (1.0 / (d))
#define DR_FMA_K(p, z, k) __builtin_fma(p, z, k)
"""

DIV_NEAR1 = r"""
/* n / d for d in [1, 4]: reciprocal seed, two Newton steps, one residual correction. */
DR_FN double dr_div_near1(double n, double d)
{
    double r = DR_RCP64(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    const double q = n * r;
    return __builtin_fma(__builtin_fma(-d, q, n), r, q);
}"""

LOG_F8 = r"""
DR_FN double dr_log_f8(double x)
{
    int k;
    double m = __builtin_frexp(x, &k);            /* x = m 2^k, m in [0.5, 1) */
    const int lo = m < 0x1.6a09e667f3bcdp-1;      /* below sqrt(1/2): use 2m, k-1 */
    m = __builtin_ldexp(m, lo);
    const double kd = (double)(k - lo);
    const double f = m - 1.0;
    const double s = dr_div_near1(f, 2.0 + f);
    const double z = s * s;
    double q = 0x1.2b5baa716e7eap-3;
    q = DR_FMA_K(q, z, 0x1.39fe142880193p-3);
    q = DR_FMA_K(q, z, 0x1.7462b73112de7p-3);
    q = DR_FMA_K(q, z, 0x1.c71c62dba6605p-3);
    q = DR_FMA_K(q, z, 0x1.2492492df9f94p-2);
    q = DR_FMA_K(q, z, 0x1.9999999995288p-2);
    q = DR_FMA_K(q, z, 0x1.5555555555558p-1);
    const double hfsq = 0.5 * f * f;
    double t = s * __builtin_fma(q, z, hfsq);      /* s (hfsq + R) */
    t = __builtin_fma(kd, 0x1.a39ef35793c76p-33, t);
    t = (hfsq - t) - f;
    const double r = __builtin_fma(kd, 0x1.62e42fee00000p-1, -t);
    if (x > 0.0 && x < __builtin_inf())
        return r;
    if (x == 0.0)
        return -__builtin_inf();
    return x < 0.0 ? __builtin_nan("") : x;        /* +inf and NaN pass through */
}"""

EXP_REDUCED = r"""
/* exp(u) = 2^k e^v with k = rint(u / ln 2) and |v| <= ln(2)/2; returns e^v (relative
   error of the polynomial 2.5e-17).  |u| must stay below 2^31 ln 2. */
DR_FN double dr_exp_reduced(double u, int* k)
{
    const double kd = __builtin_rint(u * 0x1.71547652b82fep+0);
    double v = __builtin_fma(kd, -0x1.62e42fee00000p-1, u);
    v = __builtin_fma(kd, -0x1.a39ef35793c76p-33, v);
    double e = 0x1.ad50f1fd5071ep-26;
    e = DR_FMA_K(e, v, 0x1.28b2fd7f7df2ap-22);
    e = DR_FMA_K(e, v, 0x1.71df5308de4f4p-19);
    e = DR_FMA_K(e, v, 0x1.a01992e94ed5ap-16);
    e = DR_FMA_K(e, v, 0x1.a01a0109b44eap-13);
    e = DR_FMA_K(e, v, 0x1.6c16c18776dfcp-10);
    e = DR_FMA_K(e, v, 0x1.11111111323f6p-7);
    e = DR_FMA_K(e, v, 0x1.555555554f3a8p-5);
    e = DR_FMA_K(e, v, 0x1.555555555549ap-3);
    e = DR_FMA_K(e, v, 0x1.0000000000010p-1);
    e = __builtin_fma(e, v, 1.0);
    e = __builtin_fma(e, v, 1.0);
    *k = (int)kd;
    return e;
}"""

EXP_F8 = r"""
DR_FN double dr_exp_f8(double x)
{
    /* beyond these bounds the result is 0 or infinity anyway; the clamp keeps k in
       range and turns NaN into a number, which the last line undoes */
    const double c = __builtin_fmin(__builtin_fmax(x, -746.0), 710.0);
    int k;
    const double e = dr_exp_reduced(c, &k);
    const double r = __builtin_ldexp(e, k);
    return x != x ? x : r;
}"""

ERF_F8 = r"""
DR_FN double dr_erf_f8(double x)
{
    const double a = __builtin_fabs(x);
    double r;
    if (a < 1.0) {
        const double z = a * a;
        double p = 0x1.0565f423b09cfp-34;
        p = DR_FMA_K(p, z, -0x1.386350e0c4e7ap-30);
        p = DR_FMA_K(p, z, 0x1.f7a19d528709cp-27);
        p = DR_FMA_K(p, z, -0x1.5f1cfb0eb6c5fp-23);
        p = DR_FMA_K(p, z, 0x1.b9deea6c3ea2cp-20);
        p = DR_FMA_K(p, z, -0x1.f4d1dea693fd5p-17);
        p = DR_FMA_K(p, z, 0x1.f9a321994fb79p-14);
        p = DR_FMA_K(p, z, -0x1.c02db3d8a714ep-11);
        p = DR_FMA_K(p, z, 0x1.565bcd0dae9f0p-8);
        p = DR_FMA_K(p, z, -0x1.b82ce312848f4p-6);
        p = DR_FMA_K(p, z, 0x1.ce2f21a042b1ep-4);
        p = DR_FMA_K(p, z, -0x1.812746b0379e6p-2);
        p = DR_FMA_K(p, z, 0x1.06eba8214db69p-3);
        r = __builtin_fma(a, p, a);                /* the constant term is 2/sqrt(pi) - 1 */
    } else {
        const double b = a > 6.0 ? 6.0 : a;        /* erfc(6) < 2^-54; NaN stays NaN */
        const double t = b - 3.5;
        double g = -0x1.221147b563ffbp-40;
        g = DR_FMA_K(g, t, -0x1.3885a5dbbe14ep-36);
        g = DR_FMA_K(g, t, -0x1.2a20218544ba9p-33);
        g = DR_FMA_K(g, t, -0x1.50aca32bd90fcp-31);
        g = DR_FMA_K(g, t, -0x1.d5301ca084a12p-30);
        g = DR_FMA_K(g, t, -0x1.94035ed7bbcc9p-29);
        g = DR_FMA_K(g, t, -0x1.19614d36f531bp-29);
        g = DR_FMA_K(g, t, 0x1.cff1d20d11d5bp-29);
        g = DR_FMA_K(g, t, -0x1.1e58cdc18bb96p-30);
        g = DR_FMA_K(g, t, 0x1.82398eb246889p-24);
        g = DR_FMA_K(g, t, -0x1.38cf9df71a6f9p-21);
        g = DR_FMA_K(g, t, 0x1.04c4438028a9ep-18);
        g = DR_FMA_K(g, t, -0x1.9937d18e49923p-16);
        g = DR_FMA_K(g, t, 0x1.34e6ce172f758p-13);
        g = DR_FMA_K(g, t, -0x1.ca104ff58326dp-11);
        g = DR_FMA_K(g, t, 0x1.567800c1697aep-8);
        g = DR_FMA_K(g, t, -0x1.105be5c3f99a5p-5);
        g = DR_FMA_K(g, t, 0x1.107c69161da5dp-2);
        g = DR_FMA_K(g, t, 0x1.dcc8b29511cd3p+0);
        int k;                                     /* erfc(b) = exp(-(b^2 + g)) */
        const double e = dr_exp_reduced(-__builtin_fma(b, b, g), &k);
        r = 1.0 - __builtin_ldexp(e, k);
    }
    return __builtin_copysign(r, x);
}"""

# ufunc name -> (device function, sources it needs in order), float64 only
FUNCTIONS = {
    "log": ("dr_log_f8", (DIV_NEAR1, LOG_F8)),
    "erf": ("dr_erf_f8", (EXP_REDUCED, ERF_F8)),
    "exp": ("dr_exp_f8", (EXP_REDUCED, EXP_F8)),
}


def source(names, macros=DEVICE_MACROS):
    """Definitions of the functions for the ufuncs in `names`, each piece once."""
    pieces = []
    for name in names:
        for piece in FUNCTIONS[name][1]:
            if piece not in pieces:
                pieces.append(piece)
    return macros + "".join(pieces) if pieces else ""
