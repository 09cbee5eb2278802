"""Single-precision `erf`, `exp` and `log` for the generated kernels.

The device library's versions cost 33, 14 and 13 vector instructions per element
(counted in gfx950 code); Black-Scholes in float32 spends 42 % of its 149 instructions
per option in two `erff` calls and is bound by the vector unit, not by memory.  These
cost 19, 8 and 6.  Nothing here branches on a per-element condition except for one
rarely taken path per function that handles arguments outside the ordinary range
(infinities, denormals, overflow): a wave skips it unless one of its lanes needs it.

The hardware evaluates 2^x, log2(x) (1 ulp each, no denormals) in one quarter-rate
instruction; everything is arranged around those:
  exp   k = rint(x log2 e), f = x log2 e - k in two fused steps (the product is never
        rounded on its own), 2^f by hardware, scaled by 2^k
  log   log2(x) by hardware, times ln 2 as a two-term product
  erf   |x| < 0.875: x + x P(x^2) (degree 5); above: 1 - 2^(-G(b)), b = min(|x|, 4),
        G(b) = -log2(erfc(b)) fitted directly (degree 6, under the weight erfc(x)/erf(x):
        the relative error of the result is what matters); erfc(4) < 2^-25.  Both are
        evaluated and one is selected: on Black-Scholes arguments nearly every wave
        holds both cases, so a branch would run both anyway, one after the other.
Accuracy: the polynomials contribute < 0.25 ulp; with 1 ulp hardware functions the
results stay within 2 ulp of the correctly rounded ones (measured on the device against
NumPy and SciPy on every float32 in the test suite).  Special values follow C99.
float64 functions are in `mathlib`.  Coefficients: `mathlib_fit.py`.
"""

DEVICE_MACROS = """\
#define DR_FN4 static __device__ __forceinline__
#define DR_EXP2F(x) __builtin_amdgcn_exp2f(x)
#define DR_LOG2F(x) __builtin_amdgcn_logf(x)
#define DR_RCPF(x) __builtin_amdgcn_rcpf(x)
#define DR_SQRTF(x) __builtin_amdgcn_sqrtf(x)
#define DR_ANY_LANE4(p) (__builtin_amdgcn_ballot_w64(p) != 0)
"""

HOST_MACROS = """\
#define DR_FN4 static inline
#define DR_EXP2F(x) exp2f(x)
#define DR_LOG2F(x) log2f(x)
#define DR_RCPF(x) (1.0f / (x))
#define DR_SQRTF(x) sqrtf(x)
#define DR_ANY_LANE4(p) (p)
"""

EXP_F4 = r"""
DR_FN4 float dr_exp_f4(float x)
{
    const float t = x * 0x1.715476p+0f;
    const float k = __builtin_rintf(t);
    float f = __builtin_fmaf(x, 0x1.715476p+0f, -k);      /* x log2(e) - k, rounded once */
    f = __builtin_fmaf(x, 0x1.4ae0cp-26f, f);              /* log2(e) - (float)log2(e) */
    float r = __builtin_ldexpf(DR_EXP2F(f), (int)k);
    if (!(__builtin_fabsf(x) <= 87.0f))                    /* overflow, underflow, inf, NaN */
        r = x != x ? x : (x > 0.0f ? (x > 88.8f ? __builtin_inff() : r)
                                   : (x < -104.0f ? 0.0f : r));
    return r;
}"""

LOG_F4 = r"""
DR_FN4 float dr_log_f4(float x)
{
    float y = DR_LOG2F(x);
    if (!(x >= 0x1p-126f && x < __builtin_inff())) {       /* denormal, zero, negative, inf, NaN */
        if (x > 0.0f && x < 0x1p-126f)
            y = DR_LOG2F(x * 0x1p+32f) - 32.0f;
        else
            return x == 0.0f ? -__builtin_inff() : (x < 0.0f ? __builtin_nanf("") : x);
    }
    const float h = y * 0x1.62e43p-1f;
    float l = __builtin_fmaf(y, 0x1.62e43p-1f, -h);
    l = __builtin_fmaf(y, -0x1.05c61p-29f, l);             /* ln 2 - (float)ln 2 */
    return h + l;
}"""

ERF_F4 = r"""
DR_FN4 float dr_erf_f4(float x)
{
    const float a = __builtin_fabsf(x);
    const float z = x * x;
    float p = -0x1.450632p-11f;
    p = __builtin_fmaf(p, z, 0x1.49bd4cp-8f);
    p = __builtin_fmaf(p, z, -0x1.b6f162p-6f);
    p = __builtin_fmaf(p, z, 0x1.ce20f8p-4f);
    p = __builtin_fmaf(p, z, -0x1.81270ap-2f);
    p = __builtin_fmaf(p, z, 0x1.06eba6p-3f);
    const float near = __builtin_fmaf(x, p, x);
    const float b = __builtin_fminf(a, 4.0f);
    float g = -0x1.3256eep-12f;
    g = __builtin_fmaf(g, b, 0x1.25a54cp-8f);
    g = __builtin_fmaf(g, b, -0x1.098dap-5f);
    g = __builtin_fmaf(g, b, 0x1.3485f6p-3f);
    g = __builtin_fmaf(g, b, 0x1.d642f2p-1f);
    g = __builtin_fmaf(g, b, 0x1.a09982p+0f);
    g = __builtin_fmaf(g, b, 0x1.71c77ap-13f);
    const float far = __builtin_copysignf(1.0f - DR_EXP2F(-g), x);
    return a >= 0.875f ? far : near;                        /* NaN takes `near` and stays NaN */
}"""

DIV_F4 = r"""
/* a / b for quotients that nothing reads but functions which round on their own: the
   hardware's reciprocal (1 ulp), the product and one correction by the exact residual,
   four operations where the correctly rounded division takes ten and two changes of the
   denormal mode.  Within one ulp of the exact quotient.  Whatever needs the long way
   (zero, infinite, NaN, denormal or overflowing operands and results) shows as a result
   that is not a normal number and takes the compiler's division, on a path that a wave
   skips when none of its lanes needs it.  One element at a time that test costs more than
   the six operations saved (Black-Scholes float32: 120 against 115 us), so kernels use
   the form for packs below, which tests once for all the elements of a thread (110 us). */
DR_FN4 float dr_div_f4(float a, float b)
{
    const float y = DR_RCPF(b);
    float q = a * y;
    const float r = __builtin_fmaf(-b, q, a);
    q = __builtin_fmaf(r, y, q);
    if (DR_ANY_LANE4(!__builtin_isnormal(q))) {
        if (!__builtin_isnormal(q))
            q = a / b;
    }
    return q;
}
/* the same on a pack of elements: one test per wave for all of them */
template <int P>
DR_FN4 void dr_div_f4_pack(const float (&a)[P], const float (&b)[P], float (&out)[P])
{
    bool rare = false;
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const float y = DR_RCPF(b[e]);
        float q = a[e] * y;
        const float r = __builtin_fmaf(-b[e], q, a[e]);
        q = __builtin_fmaf(r, y, q);
        out[e] = q;
        rare |= !__builtin_isnormal(q);
    }
    if (DR_ANY_LANE4(rare)) {
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            if (!__builtin_isnormal(out[e]))
                out[e] = a[e] / b[e];
    }
}
/* Square roots that nothing reads but functions which round on their own: the hardware's
   (1 ulp) as it is, where the correctly rounded one corrects it twice and rescales small
   arguments.  Denormal, zero, negative, infinite and NaN arguments take the compiler's
   square root, on a path a wave skips when none of its lanes needs it. */
template <int P>
DR_FN4 void dr_sqrt_near_f4_pack(const float (&x)[P], float (&out)[P])
{
    bool rare = false;
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        out[e] = DR_SQRTF(x[e]);
        rare |= !(x[e] >= 0x1p-126f && x[e] < __builtin_inff());
    }
    if (DR_ANY_LANE4(rare)) {
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            if (!(x[e] >= 0x1p-126f && x[e] < __builtin_inff()))
                out[e] = __builtin_sqrtf(x[e]);
    }
}"""

# ufunc name -> (device function, sources it needs in order), float32 only
FUNCTIONS = {
    "exp": ("dr_exp_f4", (EXP_F4,)),
    "log": ("dr_log_f4", (LOG_F4,)),
    "erf": ("dr_erf_f4", (ERF_F4,)),
}


def source(names, macros=DEVICE_MACROS, soft_div=False):
    """Definitions of the functions for the ufuncs in `names`, each piece once (and of the
    short division, when the program has quotients that qualify for it)."""
    pieces = []
    for name in names:
        for piece in FUNCTIONS[name][1]:
            if piece not in pieces:
                pieces.append(piece)
    if soft_div:
        pieces.append(DIV_F4)
    return macros + "".join(pieces) if pieces else ""
