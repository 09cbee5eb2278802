"""Double-precision `log`, `erf` and `exp` for the generated kernels.

The device library's versions cost 97, 105 and 41 vector instructions per element
(counted in gfx950 code), which makes a Black-Scholes kernel in float64 wait on the
fp64 pipes rather than on memory.  These cost about 43, 49 and 25, and are written so
that a thread evaluates them on a *pack* of P elements in lock step.

Why packs.  A 64-bit polynomial coefficient reaches `v_fma_f64` through a scalar
register pair (`DR_FMA_K`), which takes two scalar moves.  A SIMD issues at most one
scalar and one vector instruction per four cycles, so a Horner step that needs two
scalar moves for every multiply-add runs at half the rate of the vector unit: measured,
polynomial steps cost 8 cycles, not 4 (Black-Scholes float64, one element at a time:
254 vector instructions per option, 305 us where the vector unit alone would need
205).  With P elements per step the two moves are shared by P multiply-adds; P = 4
leaves the scalar unit at half load.  Every function is a template over P, and none of
them branches: a branch would split the pack's instruction stream (and the lanes of a
wave rarely agree on it anyway: on Black-Scholes arguments nearly every wave holds both
|x| < 1 and |x| >= 1, so a two-branch `erf` runs both branches).

Accuracy against 40-digit references (`tests/test_mathlib.py` builds this same source
for the host): log <= 0.8 ulp over the whole range including denormals, exp <= 1 ulp,
erf <= 2 ulp (SciPy's own is off by up to 2.6); special values (zeros, infinities, NaN,
negative arguments, overflow, gradual underflow) follow C99.  float32 keeps the device
library's functions.

`log` is the classic reduction x = 2^k m, m in [sqrt(1/2), sqrt(2)), s = f/(2+f) with
f = m-1, log(1+f) = f - (f^2/2 - s (f^2/2 + R(s^2))).  `exp` is 2^k (1 + m) with
k = rint(x / ln 2), m = e^v - 1 = v + v^2 R(v).  `erf` is -expm1(-w) with
w = -log(erfc|x|) = b (b + 1 + H(b)), b = min(|x|, 6), one polynomial H of degree 23
over the whole range, fitted under the weight x erfc(x)/erf(x) (the relative error of
the result is what matters).  The coefficients are least-squares fits on Chebyshev
nodes in 50-digit arithmetic, printed by `mathlib_fit.py` next to this file.
"""

DEVICE_MACROS = """\
#define DR_FN static __device__ __forceinline__
#define DR_RCP64(d) __builtin_amdgcn_rcp(d)
/* p * z + k with the constant k in a scalar register pair.  The compiler prefers the
   two-address v_fmac_f64 for a Horner step and then copies every 64-bit constant into
   the accumulator with two v_mov_b32, which triples the cost of a polynomial. */
#define DR_FMA_K(p, z, k) ({ double dr_r_; \\
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(dr_r_) : "v"(p), "v"(z), "s"((double)(k))); dr_r_; })
"""

HOST_MACROS = """\
#define DR_FN static inline
#define DR_RCP64(d) (1.0 / (d))
#define DR_FMA_K(p, z, k) __builtin_fma(p, z, k)
"""

STEP = r"""
/* One Horner step p = p * z + K on every element of a pack.  The elements advance in
   lock step so that the constant is fetched into its scalar register pair once per pack,
   not once per element. */
#define DR_STEP(p, z, K) _Pragma("unroll") for (int e_ = 0; e_ < P; ++e_) p[e_] = DR_FMA_K(p[e_], z[e_], K)"""

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
template <int P>
DR_FN void dr_log_f8(const double (&x)[P], double (&out)[P])
{
    double kd[P], f[P], s[P], z[P], q[P];
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        int k;
        double m = __builtin_frexp(x[e], &k);         /* x = m 2^k, m in [0.5, 1) */
        const int lo = m < 0x1.6a09e667f3bcdp-1;      /* below sqrt(1/2): use 2m, k-1 */
        m = __builtin_ldexp(m, lo);
        kd[e] = (double)(k - lo);
        f[e] = m - 1.0;
        s[e] = dr_div_near1(f[e], 2.0 + f[e]);
        z[e] = s[e] * s[e];
        q[e] = 0x1.2b5baa716e7eap-3;
    }
    DR_STEP(q, z, 0x1.39fe142880193p-3);
    DR_STEP(q, z, 0x1.7462b73112de7p-3);
    DR_STEP(q, z, 0x1.c71c62dba6605p-3);
    DR_STEP(q, z, 0x1.2492492df9f94p-2);
    DR_STEP(q, z, 0x1.9999999995288p-2);
    DR_STEP(q, z, 0x1.5555555555558p-1);
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double hfsq = 0.5 * f[e] * f[e];
        double t = s[e] * __builtin_fma(q[e], z[e], hfsq);      /* s (hfsq + R) */
        t = __builtin_fma(kd[e], 0x1.a39ef35793c76p-33, t);
        t = (hfsq - t) - f[e];
        const double r = __builtin_fma(kd[e], 0x1.62e42fee00000p-1, -t);
        const double bad = x[e] == 0.0 ? -__builtin_inf() : (x[e] < 0.0 ? __builtin_nan("") : x[e]);
        out[e] = (x[e] > 0.0 && x[e] < __builtin_inf()) ? r : bad;   /* +inf and NaN pass through */
    }
}"""

EXPM1_REDUCED = r"""
/* e^u - 1 = 2^k (1 + m) - 1 with k = rint(u / ln 2), v = u - k ln 2, |v| <= ln(2)/2 and
   m = e^v - 1 = v + v^2 R(v) (relative error of m: 2e-17 from the polynomial).  Returns
   m and k as a double; |u| must stay below 2^31 ln 2. */
template <int P>
DR_FN void dr_expm1_reduced(const double (&u)[P], double (&m)[P], double (&kd)[P])
{
    double v[P], r[P];
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        kd[e] = __builtin_rint(u[e] * 0x1.71547652b82fep+0);
        v[e] = __builtin_fma(kd[e], -0x1.62e42fee00000p-1, u[e]);
        v[e] = __builtin_fma(kd[e], -0x1.a39ef35793c76p-33, v[e]);
        r[e] = 0x1.af5f25602458cp-26;
    }
    DR_STEP(r, v, 0x1.28a29c8f1f3d8p-22);
    DR_STEP(r, v, 0x1.71ddf8126db6fp-19);
    DR_STEP(r, v, 0x1.a019a69461f34p-16);
    DR_STEP(r, v, 0x1.a01a01b0026afp-13);
    DR_STEP(r, v, 0x1.6c16c17f32eaep-10);
    DR_STEP(r, v, 0x1.111111110f659p-7);
    DR_STEP(r, v, 0x1.5555555552103p-5);
    DR_STEP(r, v, 0x1.5555555555559p-3);
    DR_STEP(r, v, 0x1.0000000000005p-1);
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        m[e] = __builtin_fma(v[e] * v[e], r[e], v[e]);
}"""

EXP_F8 = r"""
template <int P>
DR_FN void dr_exp_f8(const double (&x)[P], double (&out)[P])
{
    double c[P], m[P], kd[P];
    /* beyond these bounds the result is 0 or infinity anyway; the clamp keeps k in
       range and turns NaN into a number, which the last line undoes */
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        c[e] = __builtin_fmin(__builtin_fmax(x[e], -746.0), 710.0);
    dr_expm1_reduced<P>(c, m, kd);
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double r = __builtin_ldexp(1.0 + m[e], (int)kd[e]);
        out[e] = x[e] != x[e] ? x[e] : r;
    }
}"""

ERF_F8 = r"""
/* erf(x) = 1 - erfc(|x|) = -expm1(-w) with w = -log(erfc(|x|)) = b (b + 1 + H(b)),
   b = min(|x|, 6) (erfc(6) < 2^-54).  One formula over the whole range: there is no
   branch for the lanes of a wave to disagree on.  1 - 2^k (1 + m) is formed as
   (1 - 2^k) - 2^k m with one rounding; for k = 0 (|x| < 0.28) that is -m itself, which
   keeps full relative accuracy down to the smallest arguments. */
template <int P>
DR_FN void dr_erf_f8(const double (&x)[P], double (&out)[P])
{
    double b[P], h[P], w[P], m[P], kd[P];
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        b[e] = __builtin_fmin(__builtin_fabs(x[e]), 6.0);
        h[e] = -0x1.e6f307c4860f7p-49;
    }
    DR_STEP(h, b, 0x1.57729bb227674p-43);
    DR_STEP(h, b, -0x1.c0ed382958218p-39);
    DR_STEP(h, b, 0x1.680137d9754dbp-35);
    DR_STEP(h, b, -0x1.8a87ecbf415cap-32);
    DR_STEP(h, b, 0x1.361dab29e94e8p-29);
    DR_STEP(h, b, -0x1.61cbb40306505p-27);
    DR_STEP(h, b, 0x1.1a8f495cb20cfp-25);
    DR_STEP(h, b, -0x1.06135376c2286p-24);
    DR_STEP(h, b, -0x1.7c237a0b8c9e2p-26);
    DR_STEP(h, b, 0x1.3c30921a89064p-21);
    DR_STEP(h, b, -0x1.14dd76749ad98p-19);
    DR_STEP(h, b, 0x1.a84fb449f4921p-19);
    DR_STEP(h, b, 0x1.a6191f3df8156p-19);
    DR_STEP(h, b, -0x1.efea1cbd0a69cp-16);
    DR_STEP(h, b, 0x1.0e298369bd84ep-14);
    DR_STEP(h, b, 0x1.b2a9c5a5ac927p-16);
    DR_STEP(h, b, -0x1.35665db8187e2p-11);
    DR_STEP(h, b, 0x1.bca6954358943p-10);
    DR_STEP(h, b, -0x1.b6b6a561f0c7ep-13);
    DR_STEP(h, b, -0x1.3966858ff9ae2p-6);
    DR_STEP(h, b, 0x1.a4f4e2a1a827cp-4);
    DR_STEP(h, b, -0x1.7419f246c6e33p-2);
    DR_STEP(h, b, 0x1.06eba8214db68p-3);
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        w[e] = -__builtin_fma(b[e], b[e] + h[e], b[e]);
    dr_expm1_reduced<P>(w, m, kd);
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double s = __builtin_ldexp(1.0, (int)kd[e]);            /* 2^k, k <= 0 */
        const double r = __builtin_fma(-s, m[e], 1.0 - s);            /* 1 - 2^k (1 + m) */
        out[e] = x[e] != x[e] ? x[e] : __builtin_copysign(r, x[e]);
    }
}"""

# ufunc name -> (device function template, sources it needs in order), float64 only
FUNCTIONS = {
    "log": ("dr_log_f8", (STEP, DIV_NEAR1, LOG_F8)),
    "erf": ("dr_erf_f8", (STEP, EXPM1_REDUCED, ERF_F8)),
    "exp": ("dr_exp_f8", (STEP, EXPM1_REDUCED, EXP_F8)),
}

SCALAR_WRAPPER = """
DR_FN double {fn}_1(double x)
{{
    const double a[1] = {{x}};
    double r[1];
    {fn}<1>(a, r);
    return r[0];
}}
"""


def source(names, macros=DEVICE_MACROS):
    """Definitions of the function templates for the ufuncs in `names` (each piece
    once) and of their one-element forms `<function>_1(double)`."""
    pieces = []
    for name in names:
        for piece in FUNCTIONS[name][1]:
            if piece not in pieces:
                pieces.append(piece)
    if not pieces:
        return ""
    wrappers = "".join(SCALAR_WRAPPER.format(fn=FUNCTIONS[name][0]) for name in names)
    return macros + "".join(pieces) + wrappers
