"""Double-precision `log`, `erf`, `exp` and `sqrt` for the generated kernels.

The device library's versions cost 97, 105 and 41 vector instructions per element
(counted in gfx950 code), which makes a Black-Scholes kernel in float64 wait on the
fp64 pipes rather than on memory.  These cost about 25, 20 and 25.  Black-Scholes in
float64, n = 2^25, microseconds per launch on MI355X (vector instructions per option):
device library 398 (379); polynomial `log`/`erf`/`exp`, one element at a time 305 (254);
the same on packs of four 299 (245); `log` from a table 293 (227); `erf` from a table
read in memory 405, read in LDS 262, with workgroups that stay for eight chunks 241;
with the short `sqrt` 240 (138).  At that point the kernel moves its bytes at 85 % of a
plain copy's rate; the vector unit is busy 59 % of the time and LDS 43 %, more than half
of that in bank conflicts between the lanes' table rows (rocprofv3 `SQ_ACTIVE_INST_VALU`,
`SQ_LDS_IDX_ACTIVE`, `SQ_LDS_BANK_CONFLICT`).

`log` and `erf` are table driven.  `log`: x = 2^k z, z in [0.706, 1.412) falls into one of
256 intervals with centre c, log x = k ln 2 + log c + log1p(z/c - 1); 1/c and log c come
from a 4 KiB table (one 16-byte read per element), the last term is a polynomial of degree
6 in an argument below 2^-9; no division.  `erf`: |x| < 6 falls into one of 96 intervals of
width 1/16, on each of which erf is a polynomial of degree 8 around a point c; c and the
nine coefficients come from a 7.5 KiB table (five 16-byte reads per element); no
exponential, no branch for the lanes of a wave to disagree on (on Black-Scholes arguments
nearly every wave holds both |x| < 1 and |x| >= 1, and a two-branch `erf` runs both
branches, one after the other).  Both tables place c where the tabulated function value is
a double to within a small fraction of an ulp, so that the table adds almost no rounding
of its own.  Every lane reads its own row: through the vector memory path that is slow, so
flat kernels copy the tables into LDS first (`source(..., lds=True)`, `DR_STAGE_TABLES`);
other kernel shapes read them in memory.  `exp` is 2^k (1 + m) with k = rint(x / ln 2),
m = e^v - 1 = v + v^2 R(v), R of degree 9.  `sqrt` is the compiler's own correctly rounded
expansion without its rescaling and special-case selects (10 instructions instead of 21);
arguments that need those take the compiler's path, which a wave skips when none of its
lanes does (tested per wave: a per-lane condition is folded into selects and both
versions run).

Packs.  A 64-bit polynomial coefficient reaches `v_fma_f64` through a scalar register
pair (`DR_FMA_K`), which takes two scalar moves.  Every function is a template over P
and takes a pack of P elements through each polynomial step together, so the two moves
are shared: with all three functions polynomial, Black-Scholes issued 146 scalar
instructions per option one element at a time and 37 on packs of four (rocprofv3
`SQ_INSTS_SALU`).  The kernel is bound by the vector unit, so the gain in time is small;
the requirement is that nothing branches.

Accuracy against 40-digit references (`tests/test_mathlib.py` builds this same source
for the host): log <= 1 ulp over the whole range including denormals, exp <= 1 ulp,
erf <= 1.1 ulp (1.8 ulp below 1/16, where the result is a product with 2/sqrt(pi);
SciPy's own erf is off by up to 2.6); special values (zeros, infinities, NaN, negative
arguments, overflow, gradual underflow) follow C99.  float32 functions are in
`mathlib32`.  Coefficients and tables: `mathlib_fit.py` next to this file (least-squares
fits on Chebyshev nodes in 50-digit arithmetic).
"""

DEVICE_MACROS = """\
#define DR_FN static __device__ __forceinline__
#define DR_TABLE static __device__ const
#define DR_ALIGN16 __attribute__((aligned(16)))
#define DR_RSQ64(x) __builtin_amdgcn_rsq(x)
#define DR_RCP64(x) __builtin_amdgcn_rcp(x)
#define DR_ANY_LANE(p) (__builtin_amdgcn_ballot_w64(p) != 0)
/* p * z + k with the constant k in a scalar register pair.  The compiler prefers the
   two-address v_fmac_f64 for a Horner step and then copies every 64-bit constant into
   the accumulator with two v_mov_b32, which triples the cost of a polynomial. */
#define DR_FMA_K(p, z, k) ({ double dr_r_; \\
    asm("v_fma_f64 %0, %1, %2, %3" : "=v"(dr_r_) : "v"(p), "v"(z), "s"((double)(k))); dr_r_; })
"""

HOST_MACROS = """\
#define DR_FN static inline
#define DR_TABLE static const
#define DR_ALIGN16 __attribute__((aligned(16)))
/* a 24-bit estimate of 1/sqrt(x), like the hardware's */
static inline double dr_rsq64_host(double x)
{
    int ex;
    const double mant = frexp(1.0 / sqrt(x), &ex);
    return ldexp((double)(float)mant, ex);
}
#define DR_RSQ64(x) dr_rsq64_host(x)
/* a 24-bit estimate of 1/x, like the hardware's */
static inline double dr_rcp64_host(double x)
{
    int ex;
    const double mant = frexp(1.0 / x, &ex);
    return ldexp((double)(float)mant, ex);
}
#define DR_RCP64(x) dr_rcp64_host(x)
#define DR_ANY_LANE(p) (p)
#define DR_FMA_K(p, z, k) __builtin_fma(p, z, k)
"""

STEP = r"""
/* One Horner step p = p * z + K on every element of a pack.  The elements advance in
   lock step so that the constant is fetched into its scalar register pair once per pack,
   not once per element. */
#define DR_STEP(p, z, K) _Pragma("unroll") for (int e_ = 0; e_ < P; ++e_) p[e_] = DR_FMA_K(p[e_], z[e_], K)"""

LOG_TABLE = r"""
/* 1/c and log(c) for the 256 intervals of `dr_log_core`; c is the centre of its interval
   moved by less than 2^-23 of itself to a point whose logarithm is a double to within 0.004 ulp. */
DR_TABLE DR_ALIGN16 double dr_log_tab[512] = {
    0x1.6a13cd153728dp+0, -0x1.630030b3aac40p-2,
    0x1.691473a88d0e1p+0, -0x1.602d08af0924ap-2,
    0x1.68168155466eap+0, -0x1.5d5bddc0163d9p-2,
    0x1.6719f360166ebp+0, -0x1.5a8cadbbedf1bp-2,
    0x1.661ec6b2523cdp+0, -0x1.57bf756270459p-2,
    0x1.6524f853b4a9bp+0, -0x1.54f431b7be191p-2,
    0x1.642c8581d2076p+0, -0x1.522ae048c612bp-2,
    0x1.63356b88ac0dbp+0, -0x1.4f637ebba9807p-2,
    0x1.623fa78126351p+0, -0x1.4c9e0a12c5352p-2,
    0x1.614b36831affep+0, -0x1.49da7f3bcc839p-2,
    0x1.6058160f216a0p+0, -0x1.4718dc43155dcp-2,
    0x1.5f66434292df1p+0, -0x1.44591e0539f29p-2,
    0x1.5e75bb7ea1501p+0, -0x1.419b42135de26p-2,
    0x1.5d867c3ece430p+0, -0x1.3edf463c16cc3p-2,
    0x1.5c9882a760f3ap+0, -0x1.3c25273edfe3ep-2,
    0x1.5babcc647fa7ep+0, -0x1.396ce359bbf1bp-2,
    0x1.5ac056b015c29p+0, -0x1.36b6776be1540p-2,
    0x1.59d61f123cccap+0, -0x1.3401e12aecbffp-2,
    0x1.58ed230815a76p+0, -0x1.314f1e1d36172p-2,
    0x1.580560158052bp+0, -0x1.2e9e2bce121e8p-2,
    0x1.571ed3c506b28p+0, -0x1.2bef07cdc931fp-2,
    0x1.56397ba7c52e8p+0, -0x1.2941afb186b8ep-2,
    0x1.5555566655cccp+0, -0x1.269624464f1e2p-2,
    0x1.54725e6bb817dp+0, -0x1.23ec5991eb5c3p-2,
    0x1.5390949bc10b3p+0, -0x1.214456f69db30p-2,
    0x1.52aff56a803f2p+0, -0x1.1e9e1678895e2p-2,
    0x1.51d07eb72f8a5p+0, -0x1.1bf99650eed49p-2,
    0x1.50f22e111c35dp+0, -0x1.1956d3b9bbeb3p-2,
    0x1.5015014ba4fcep+0, -0x1.16b5ccad4a69bp-2,
    0x1.4f38f62dd4cc9p+0, -0x1.14167ef367811p-2,
    0x1.4e5e0a5ea03f4p+0, -0x1.1178e7e449097p-2,
    0x1.4d843bedc2c11p+0, -0x1.0edd060b77fcdp-2,
    0x1.4cab887ddb026p+0, -0x1.0c42d6997c518p-2,
    0x1.4bd3edda69144p+0, -0x1.09aa572e6cb1cp-2,
    0x1.4afd6a0bdbfc6p+0, -0x1.07138619861afp-2,
    0x1.4a27fad75ffe5p+0, -0x1.047e60cde7f64p-2,
    0x1.49539e3b2d06ep+0, -0x1.01eae5626c6a7p-2,
    0x1.4880520a0471fp+0, -0x1.feb222b514332p-3,
    0x1.47ae148ee15bbp+0, -0x1.f991c7483bb4ap-3,
    0x1.46dce34596079p+0, -0x1.f474b134df29fp-3,
    0x1.460cbc891d036p+0, -0x1.ef5ade8b0e3b9p-3,
    0x1.453d9e2c776cfp+0, -0x1.ea4449f04ab14p-3,
    0x1.446f86681db1ap+0, -0x1.e530f06fac726p-3,
    0x1.43a2730abee30p+0, -0x1.e020cc62359fdp-3,
    0x1.42d66271120c3p+0, -0x1.db13db8a93115p-3,
    0x1.420b5265e5944p+0, -0x1.d60a17f9034c1p-3,
    0x1.4141414da14dap+0, -0x1.d1037f753a369p-3,
    0x1.40782d10e63e3p+0, -0x1.cc000c9db32a9p-3,
    0x1.3fb01408514d0p+0, -0x1.c6ffbcc449cc5p-3,
    0x1.3ee8f42a5b073p+0, -0x1.c2028ab1802d7p-3,
    0x1.3e22cbc09a827p+0, -0x1.bd08732ba0328p-3,
    0x1.3d5d991a45661p+0, -0x1.b81173090a13cp-3,
    0x1.3c995a47babe5p+0, -0x1.b31d8575bce2ep-3,
    0x1.3bd60d7b327e5p+0, -0x1.ae2ca6614e285p-3,
    0x1.3b13b12113a5ep+0, -0x1.a93ed31fad546p-3,
    0x1.3a524387ac811p+0, -0x1.a454082e6aa94p-3,
    0x1.3991c2aea7e35p+0, -0x1.9f6c3ff541eaep-3,
    0x1.38d22d30e0836p+0, -0x1.9a8778bab87fap-3,
    0x1.3813814bf3952p+0, -0x1.95a5ae51de9a9p-3,
    0x1.3755bd0cd44f2p+0, -0x1.90c6db3830661p-3,
    0x1.3698df27d05e7p+0, -0x1.8beafe2215d77p-3,
    0x1.35dce5f112a6ap+0, -0x1.8712133a65de9p-3,
    0x1.3521cfa6177f7p+0, -0x1.823c160175e86p-3,
    0x1.34679ac5412bap+0, -0x1.7d690390da72bp-3,
    0x1.33ae45afabc55p+0, -0x1.7898d82d94209p-3,
    0x1.32f5ced6a1dffp+0, -0x1.73cb9074fd16ep-3,
    0x1.323e34ab11145p+0, -0x1.6f0128ef58e39p-3,
    0x1.318775819eae6p+0, -0x1.6a399d5498e11p-3,
    0x1.30d18ffa9d009p+0, -0x1.6574eb44900f6p-3,
    0x1.301c82ac403e5p+0, -0x1.60b3100b09eb0p-3,
    0x1.2f684bc7c2e43p+0, -0x1.5bf40639a75f6p-3,
    0x1.2eb4ea1fed15bp+0, -0x1.5737cc9018d49p-3,
    0x1.2e025c0c68112p+0, -0x1.527e5e7e3d0cfp-3,
    0x1.2d50a012d5083p+0, -0x1.4dc7b897bc102p-3,
    0x1.2c9fb4e102d2fp+0, -0x1.4913d8701e931p-3,
    0x1.2bef98e5a36ffp+0, -0x1.4462b9dc9b361p-3,
    0x1.2b404ac642aa3p+0, -0x1.3fb45a166ac97p-3,
    0x1.2a91c92f3c0ebp+0, -0x1.3b08b6757f1f5p-3,
    0x1.29e412a771331p+0, -0x1.365fcb4083407p-3,
    0x1.293725bb804bep+0, -0x1.31b994d3a5032p-3,
    0x1.288b013d0b15bp+0, -0x1.2d161155fca16p-3,
    0x1.27dfa38a1ce62p+0, -0x1.28753bc11ac33p-3,
    0x1.27350ba0f28c3p+0, -0x1.23d713512eccap-3,
    0x1.268b37dae01ffp+0, -0x1.1f3b92bd04322p-3,
    0x1.25e226f6491d5p+0, -0x1.1aa2b7668cf6ep-3,
    0x1.2539d7e91762dp+0, -0x1.160c8024b1d13p-3,
    0x1.2492484091e56p+0, -0x1.1178e1e67b8afp-3,
    0x1.23eb7986861acp+0, -0x1.0ce7ed7090fc7p-3,
    0x1.23456789abb4fp+0, -0x1.08598b59e2f0ap-3,
    0x1.22a0121b3113dp+0, -0x1.03cdc03cbc987p-3,
    0x1.21fb77fabfa02p+0, -0x1.fe891253900c1p-4,
    0x1.21579814756e5p+0, -0x1.f57bc8ba9ebf4p-4,
    0x1.20b470d10c182p+0, -0x1.ec7398c67ca84p-4,
    0x1.2012013352146p+0, -0x1.e3707ff4bb996p-4,
    0x1.1f7047ef220a1p+0, -0x1.da727747e9798p-4,
    0x1.1ecf43b97b764p+0, -0x1.d17977b304670p-4,
    0x1.1e2ef39b0b6e5p+0, -0x1.c8857eb6d84d0p-4,
    0x1.1d8f5682d4bbcp+0, -0x1.bf96884e98061p-4,
    0x1.1cf06ada2811bp+0, -0x1.b6ac88dad5b00p-4,
    0x1.1c522fca5e0e2p+0, -0x1.adc77f6109a44p-4,
    0x1.1bb4a3fa5ec88p+0, -0x1.a4e76379d4323p-4,
    0x1.1b17c67f2bae8p+0, -0x1.9c0c32d4d2595p-4,
    0x1.1a7b960717aedp+0, -0x1.9335e53c6bff5p-4,
    0x1.19e0119e01328p+0, -0x1.8a6477a91f286p-4,
    0x1.194538037a247p+0, -0x1.8197e2a6b0f1ap-4,
    0x1.18ab084e32d2ep+0, -0x1.78d023990de2ap-4,
    0x1.1811812ea197bp+0, -0x1.700d31f8a7587p-4,
    0x1.1778a17cbd534p+0, -0x1.674f075f9c73bp-4,
    0x1.16e0689c773fep+0, -0x1.5e95a5539096ep-4,
    0x1.1648d4f7a307fp+0, -0x1.55e0feedc7d50p-4,
    0x1.15b1e5e882620p+0, -0x1.4d3114f78b104p-4,
    0x1.151b9a296d462p+0, -0x1.4485def2152f5p-4,
    0x1.1485f0e0acd41p+0, -0x1.3bdf5a7d1eeb7p-4,
    0x1.13f0e8d594749p+0, -0x1.333d7fa3d796fp-4,
    0x1.135c81188c864p+0, -0x1.2aa04a919bc74p-4,
    0x1.12c8b889fbf5ep+0, -0x1.2207b4905912ep-4,
    0x1.12358e777304dp+0, -0x1.1973bd2cab6e5p-4,
    0x1.11a301aa64925p+0, -0x1.10e45c2b3ff12p-4,
    0x1.111110ff70ff7p+0, -0x1.08598a518297fp-4,
    0x1.107fbbc870f06p+0, -0x1.ffa68e547c6a3p-5,
    0x1.0fef010b8efcbp+0, -0x1.eea31b7c9f03fp-5,
    0x1.0f5edfc40272fp+0, -0x1.dda8b0b388d27p-5,
    0x1.0ecf56d4f9df9p+0, -0x1.ccb73f8861d76p-5,
    0x1.0e40654ee5f7dp+0, -0x1.bbcebeae2a29dp-5,
    0x1.0db20a92f4736p+0, -0x1.aaef2e3f72404p-5,
    0x1.0d24456159e1ap+0, -0x1.9a187b1a5dab3p-5,
    0x1.0c971514bdbcap+0, -0x1.894aa442962d2p-5,
    0x1.0c0a787a4428ap+0, -0x1.788597bc1a953p-5,
    0x1.0b7e6ec259f56p+0, -0x1.67c94f2d4eb02p-5,
    0x1.0af2f724fecd6p+0, -0x1.5715c4ff882d6p-5,
    0x1.0a6810aa310e2p+0, -0x1.466aedb442b0fp-5,
    0x1.09ddba659830ap+0, -0x1.35c8bf047460fp-5,
    0x1.0953f37a407f7p+0, -0x1.252f305758e27p-5,
    0x1.08cabb320658dp+0, -0x1.149e3d9baa047p-5,
    0x1.0842108f11133p+0, -0x1.0415d9f185971p-5,
    0x1.07b9f2b0eec38p+0, -0x1.e72bf7b12e165p-6,
    0x1.073260ad1f850p+0, -0x1.c63d30da34c65p-6,
    0x1.06ab59b2411a6p+0, -0x1.a55f4f5af910ep-6,
    0x1.0624dd318aa23p+0, -0x1.84925324e544ap-6,
    0x1.059ee9f9b74afp+0, -0x1.63d6143d07724p-6,
    0x1.05197f8153442p+0, -0x1.432a934ca9beep-6,
    0x1.04949cb3c63ebp+0, -0x1.228faea5f387ep-6,
    0x1.0410410a40473p+0, -0x1.0205670f07094p-6,
    0x1.038c6b84a48c4p+0, -0x1.c3173e769c1adp-7,
    0x1.03091b4f15decp+0, -0x1.824488ccd8bc8p-7,
    0x1.02864fdc22b34p+0, -0x1.4192a9d4b16e8p-7,
    0x1.020407fdd02e3p+0, -0x1.01014e42d4d09p-7,
    0x1.01824363c7a22p+0, -0x1.81211ff77d621p-8,
    0x1.010100fa10fa1p+0, -0x1.00804eac71c93p-8,
    0x1.00804034101c0p+0, -0x1.00403d49806c5p-9,
    0x1.0000000000000p+0, 0x0.0p+0,
    0x1.fe01fdf4ddf4ep-1, 0x1.ff00b7583de75p-9,
    0x1.fc07f02120806p-1, 0x1.fe02a5ffa5c83p-8,
    0x1.fa11caa9efaafp-1, 0x1.7dc4737cb22b4p-7,
    0x1.f81f81e0cf6abp-1, 0x1.fc0a90fb1627bp-7,
    0x1.f6310acfbdc10p-1, 0x1.3cea437adb9ebp-6,
    0x1.f44659de24209p-1, 0x1.7b91b1523be74p-6,
    0x1.f25f643f60a88p-1, 0x1.b9fc02d76f761p-6,
    0x1.f07c1ef561de2p-1, 0x1.f829b345e58dfp-6,
    0x1.ee9c7f7538d10p-1, 0x1.1b0d998cc0927p-5,
    0x1.ecc07b21cebdbp-1, 0x1.39e87c8ddec47p-5,
    0x1.eae807bec031dp-1, 0x1.58a5b9bd670e1p-5,
    0x1.e9131ab07b67ep-1, 0x1.774590571ac3ep-5,
    0x1.e741aa6f35240p-1, 0x1.95c82f7ee0d18p-5,
    0x1.e573ac9a6e619p-1, 0x1.b42dd663906d9p-5,
    0x1.e3a91793619cdp-1, 0x1.d276b95d6b652p-5,
    0x1.e1e1e1ca31ca3p-1, 0x1.f0a30d93c7bd4p-5,
    0x1.e01e01e01e026p-1, 0x1.075983598e42dp-4,
    0x1.de5d6e3858617p-1, 0x1.16536f27c2ebcp-4,
    0x1.dca01dca01dc5p-1, 0x1.253f62f0a1442p-4,
    0x1.dae6077d482f6p-1, 0x1.341d78c92e847p-4,
    0x1.d92f2219e7e0ap-1, 0x1.42edccba253eap-4,
    0x1.d77b654492bc5p-1, 0x1.51b0742ca6c00p-4,
    0x1.d5cac81597396p-1, 0x1.60658a1736900p-4,
    0x1.d41d41c49d325p-1, 0x1.6f0d2935f73c8p-4,
    0x1.d272ca5755c93p-1, 0x1.7da76608c7de2p-4,
    0x1.d0cb58eeabff0p-1, 0x1.8c345dabcdfaep-4,
    0x1.cf26e5b6bbeedp-1, 0x1.9ab424d9f532dp-4,
    0x1.cd8568a3b9c43p-1, 0x1.a926d2f79ca91p-4,
    0x1.cbe6d9601cbf5p-1, 0x1.b78c82bb0ed23p-4,
    0x1.ca4b304dbe10ep-1, 0x1.c5e5493ee9bd6p-4,
    0x1.c8b265b2d8a74p-1, 0x1.d4313d4ac419dp-4,
    0x1.c71c71bb4c65fp-1, 0x1.e270774cff98fp-4,
    0x1.c5894d17449edp-1, 0x1.f0a30bc6f2702p-4,
    0x1.c3f8f027ff9acp-1, 0x1.fec912b342414p-4,
    0x1.c26b53a4da13bp-1, 0x1.067150db16056p-3,
    0x1.c0e070430c18fp-1, 0x1.0d77e79b21b3dp-3,
    0x1.bf583ee868d92p-1, 0x1.147858467428cp-3,
    0x1.bdd2b89940707p-1, 0x1.1b72ad52f6758p-3,
    0x1.bc4fd652d3e20p-1, 0x1.2266f1aadd070p-3,
    0x1.bacf915b8bbc7p-1, 0x1.29552f3a990abp-3,
    0x1.b951e2a8efe99p-1, 0x1.303d71b64ea55p-3,
    0x1.b7d6c3ed13482p-1, 0x1.371fc1ba072f7p-3,
    0x1.b65e2e4e7ef2ep-1, 0x1.3dfc2ab8134bfp-3,
    0x1.b4e81b44e1ab5p-1, 0x1.44d2b6f9d5feep-3,
    0x1.b37484bd607ccp-1, 0x1.4ba36eeefb93ap-3,
    0x1.b203640e68153p-1, 0x1.526e5e16201f8p-3,
    0x1.b094b31d9211bp-1, 0x1.59338d99827cap-3,
    0x1.af286bb11ad98p-1, 0x1.5ff3078139b42p-3,
    0x1.adbe88072913cp-1, 0x1.66acd3e50b12fp-3,
    0x1.ac5701c427198p-1, 0x1.6d60fdffc22fep-3,
    0x1.aaf1d2ebceb32p-1, 0x1.740f8f90dff71p-3,
    0x1.a98ef60d6642ap-1, 0x1.7ab89000916ffp-3,
    0x1.a82e65175e19ep-1, 0x1.815c09ff6329cp-3,
    0x1.a6d01a6d01a76p-1, 0x1.87fa06520c8e5p-3,
    0x1.a574105e688c8p-1, 0x1.8e928e5dc2c95p-3,
    0x1.a41a41ae3a4bcp-1, 0x1.9525a99de93a0p-3,
    0x1.a2c2a88861d61p-1, 0x1.9bb362ace13d5p-3,
    0x1.a16d3f815499dp-1, 0x1.a23bc26ba4439p-3,
    0x1.a01a019439f5cp-1, 0x1.a8bed002f5ac0p-3,
    0x1.9ec8e95993462p-1, 0x1.af3c94bdc4d4fp-3,
    0x1.9d79f17df68a1p-1, 0x1.b5b519c512367p-3,
    0x1.9c2d14f5ca17ap-1, 0x1.bc28671d94a80p-3,
    0x1.9ae24ea550f57p-1, 0x1.c2968558c204bp-3,
    0x1.9999995e997fdp-1, 0x1.c8ff7da0aa232p-3,
    0x1.9852f0d8ec112p-1, 0x1.cf6354e09c57ep-3,
    0x1.970e4f728b78ep-1, 0x1.d5c216fcae00fp-3,
    0x1.95cbb0be377c8p-1, 0x1.dc1bca0abebf8p-3,
    0x1.948b0fd55ea5fp-1, 0x1.e27076ba80065p-3,
    0x1.934c67ff42d3fp-1, 0x1.e8c0250e6649cp-3,
    0x1.920fb4a8be2e4p-1, 0x1.ef0adc823cd7dp-3,
    0x1.90d4f12018f6ep-1, 0x1.f550a564b8261p-3,
    0x1.8f9c18e381796p-1, 0x1.fb918747ec54ap-3,
    0x1.8e6527af1374bp-1, 0x1.00e6c45ad4ffep-2,
    0x1.8d3018d88192bp-1, 0x1.0402593d1ef5ep-2,
    0x1.8bfce8062fdcdp-1, 0x1.071b85fcd5cbdp-2,
    0x1.8acb90f6bf224p-1, 0x1.0a324e27394d6p-2,
    0x1.899c0f60189d0p-1, 0x1.0d46b579ab6c4p-2,
    0x1.886e5f0abb04ap-1, 0x1.1058bf9ae4ad4p-2,
    0x1.87427bcc092a1p-1, 0x1.136870293a8efp-2,
    0x1.8618619ce8785p-1, 0x1.1675ca7ed8251p-2,
    0x1.84f00c2780774p-1, 0x1.1980d2dd41fd0p-2,
    0x1.83c977ab2c067p-1, 0x1.1c898c16995ebp-2,
    0x1.82a4a0182a33dp-1, 0x1.1f8ff9e48a69fp-2,
    0x1.8181816db16dbp-1, 0x1.22941ff1984b0p-2,
    0x1.8060180601698p-1, 0x1.2596010df7a09p-2,
    0x1.7f405fdcf800ep-1, 0x1.2895a11b81c7ep-2,
    0x1.7e225515a4dc9p-1, 0x1.2b9303ab8a0b4p-2,
    0x1.7d05f40f7056ep-1, 0x1.2e8e2bc493e99p-2,
    0x1.7beb3922e0145p-1, 0x1.31871c9544219p-2,
    0x1.7ad2209daedbdp-1, 0x1.347dd97f4b2b2p-2,
    0x1.79baa6bb639bbp-1, 0x1.3772662bfd7dap-2,
    0x1.78a4c8178a64fp-1, 0x1.3a64c556941c3p-2,
    0x1.77908119ac794p-1, 0x1.3d54fa5c1f2e6p-2,
    0x1.767dce4e2aa5fp-1, 0x1.4043084aade08p-2,
    0x1.756cac2017405p-1, 0x1.432ef2a04ebeep-2,
    0x1.745d174cd17b6p-1, 0x1.4618bc0e85d8ep-2,
    0x1.734f0c541fea6p-1, 0x1.490068040098bp-2,
    0x1.724287f46e027p-1, 0x1.4be5f957774b5p-2,
    0x1.713786d9c7ac8p-1, 0x1.4ec97326005e3p-2,
    0x1.702e05cad8212p-1, 0x1.51aad856b666bp-2,
    0x1.6f26016f25ec8p-1, 0x1.548a2c3add609p-2,
    0x1.6e1f76b4337d7p-1, 0x1.5767717455a3fp-2,
    0x1.6d1a62681c882p-1, 0x1.5a42ab0f4cf85p-2,
    0x1.6c16c16c16c19p-1, 0x1.5d1bdbf5809c4p-2,
    0x1.6b1490aa31a44p-1, 0x1.5ff3070a793c0p-2,
};"""

LOG_CORE = r"""
/* log(x) = k ln 2 + log(c) + log1p(r): x = 2^k z with z in [0.706, 1.412) cut into 256 intervals
   by the top bits of z - 0.706 (counted in the bit pattern, so 1.0 is the centre of its
   interval and that interval has c = 1, log(c) = 0 exactly: results near zero keep their
   relative accuracy); c is the centre of z's interval, r = z/c - 1 (one fused operation with
   the tabulated 1/c), |r| < 2^-9; log1p(r) = r + r^2 Q(r). */
DR_FN double dr_log_core(double x, int koff)
{
    const unsigned long long ix = __builtin_bit_cast(unsigned long long, x);
    const unsigned int top = (unsigned int)(ix >> 32);
    const unsigned int t = top - 0x3fe69800u;
    const int i = (int)((t >> 12) & 255u);
    const int k = ((int)t >> 20) + koff;
    const unsigned int ztop = top - (t & 0xfff00000u);
    const double z = __builtin_bit_cast(double, ((unsigned long long)ztop << 32) | (ix & 0xffffffffull));
    const double r = __builtin_fma(z, DR_LOG_TAB[2 * i], -1.0);
    const double kd = (double)k;
    const double w = __builtin_fma(kd, 0x1.62e42fee00000p-1, DR_LOG_TAB[2 * i + 1]);
    const double hi = w + r;
    const double lo = __builtin_fma(kd, 0x1.a39ef35793c76p-33, (w - hi) + r);
    double q = -0x1.5555c550b5bbdp-3;
    q = __builtin_fma(q, r, 0x1.9999fffe1dfcbp-3);
    q = __builtin_fma(q, r, -0x1.fffffffff201ap-3);
    q = __builtin_fma(q, r, 0x1.5555555551559p-2);
    q = __builtin_fma(q, r, -0x1.0000000000000p-1);
    return __builtin_fma(r * r, q, lo) + hi;
}

/* zero, negative, infinite, NaN and denormal arguments */
DR_FN double dr_log_special(double x)
{
    if (x > 0.0 && x < 0x1p-1022)
        return dr_log_core(x * 0x1p52, -52);
    return x == 0.0 ? -__builtin_inf() : (x < 0.0 ? __builtin_nan("") : x);
}"""

LOG_F8 = r"""
template <int P>
DR_FN void dr_log_f8(const double (&x)[P], double (&out)[P])
{
    double r[P], hi[P], lo[P], q[P];
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const unsigned long long ix = __builtin_bit_cast(unsigned long long, x[e]);
        const unsigned int top = (unsigned int)(ix >> 32);
        const unsigned int t = top - 0x3fe69800u;
        const int i = (int)((t >> 12) & 255u);
        const int k = (int)t >> 20;
        const unsigned int ztop = top - (t & 0xfff00000u);
        const double z = __builtin_bit_cast(double, ((unsigned long long)ztop << 32) | (ix & 0xffffffffull));
        r[e] = __builtin_fma(z, DR_LOG_TAB[2 * i], -1.0);
        const double kd = (double)k;
        const double w = __builtin_fma(kd, 0x1.62e42fee00000p-1, DR_LOG_TAB[2 * i + 1]);
        hi[e] = w + r[e];
        lo[e] = __builtin_fma(kd, 0x1.a39ef35793c76p-33, (w - hi[e]) + r[e]);
        q[e] = -0x1.5555c550b5bbdp-3;
    }
    DR_STEP(q, r, 0x1.9999fffe1dfcbp-3);
    DR_STEP(q, r, -0x1.fffffffff201ap-3);
    DR_STEP(q, r, 0x1.5555555551559p-2);
    DR_STEP(q, r, -0x1.0000000000000p-1);
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        out[e] = __builtin_fma(r[e] * r[e], q[e], lo[e]) + hi[e];
        if (!(x[e] >= 0x1p-1022 && x[e] < __builtin_inf()))
            out[e] = dr_log_special(x[e]);
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

ERF_TABLE = r"""
/* per interval of `dr_erf_f8`: the point c, then the coefficients of degree 0..8 */
DR_TABLE DR_ALIGN16 double dr_erf_tab[960] = {
    0x0.0p+0, 0x0.0p+0, 0x1.20dd750429b6dp+0, 0x1.543a16bb13eb4p-44, -0x1.812746b0a7461p-2, 0x1.beb969b974784p-29, 0x1.ce2eeac38586cp-4, 0x1.d4661442f6b38p-18, -0x1.ba56e52e23b2dp-6, 0x1.55662ef9e89e4p-10,
    0x1.7fffffff69e3ep-4, 0x1.b0081148008d9p-4, 0x1.1e565bca4204ep+0, -0x1.ad8189aebb061p-4, -0x1.7712743c4144fp-2, 0x1.aafd475beb8f1p-5, 0x1.ba14967ab8217p-4, -0x1.1afca37ae4aacp-6, -0x1.9d46b144eace0p-6, 0x1.17806b6b7b449p-8,
    0x1.3fffffffddf9ap-3, 0x1.662a0bdf55126p-3, 0x1.19e5e92b97c15p+0, -0x1.605f637658332p-3, -0x1.6582e9b69a7a6p-2, 0x1.5aa32b56ce3cap-4, 0x1.97594a5e93b1bp-4, -0x1.c69c44776f897p-6, -0x1.6f81fcdf786dap-6, 0x1.be0ec8845976ap-8,
    0x1.c000000103309p-3, 0x1.f190aa866adaap-3, 0x1.135e3075c1378p+0, -0x1.e1e4d4cf28e9bp-3, -0x1.4c04e66dcc3fdp-2, 0x1.d2855d59d512fp-4, 0x1.659a3494cdc89p-4, -0x1.2cf61d51b5073p-5, -0x1.2ed6f69981474p-6, 0x1.22bd60c04ebc8p-7,
    0x1.1ffffffee4cafp-2, 0x1.3c9aa8b724aadp-2, 0x1.0ae54fa4b9f79p+0, -0x1.2c41f99829f2ap-2, -0x1.2b900b64a3998p-2, 0x1.1c6c7eee938f2p-3, 0x1.277ad6a555598p-4, -0x1.66c9ac446caf1p-5, -0x1.bf5979f1a8f29p-7, 0x1.52bb5ebcf3f03p-7,
    0x1.5fffffff90eb3p-2, 0x1.7e15944d2ddeep-2, 0x1.00abcf3e2b9efp+0, -0x1.60ec3cf50c9acp-2, -0x1.05599bb02a02dp-2, 0x1.451ef627b8e23p-3, 0x1.c06c6d9d23dd3p-5, -0x1.8e2d6fe1cf0a2p-5, -0x1.0e96b702390ffp-7, 0x1.6c5bc0acbbefdp-7,
    0x1.9fffffff31d96p-2, 0x1.bccfec23c0219p-2, 0x1.e9d5a8e519546p-1, -0x1.8dfd99395f5aap-2, -0x1.b588d8dd7adaap-3, 0x1.623387885e862p-3, 0x1.26cf862bd8b20p-5, -0x1.a1bca90d7dfc5p-5, -0x1.5b6ef9cb99e39p-9, 0x1.6ebd587ce0711p-7,
    0x1.e0000000b2216p-2, 0x1.f86faa94ca534p-2, 0x1.cfc41e367c3dbp-1, -0x1.b2c7dc53b5d37p-2, -0x1.5a9de93ea02cbp-3, 0x1.7317958d47eafp-3, 0x1.133e05821d294p-6, -0x1.a155bb9dfa083p-5, 0x1.718aee4f6131fp-9, 0x1.5ac923728a69bp-7,
    0x1.1000000017045p-1, 0x1.1855a5fd516aep-1, 0x1.b3aafcc26033bp-1, -0x1.cee5ac8ead62fp-2, -0x1.fa02983c12453p-4, 0x1.77cd75ec7d14cp-3, -0x1.fa6f3a5bc9c28p-10, -0x1.8e0db5af06de7p-5, 0x1.008efe2c78a53p-7, 0x1.330b3e75a1559p-7,
    0x1.30000000c524fp-1, 0x1.32a54cb977c49p-1, 0x1.96164faf1f2ffp-1, -0x1.e23a7ea12dc32p-2, -0x1.3f5ee151f56a6p-4, 0x1.70e469ddc9d8fp-3, -0x1.3da681c06d2dfp-6, -0x1.6a0d087219839p-5, 0x1.8cb27717a6872p-7, 0x1.f6ce46c5a096ap-8,
    0x1.4ffffffeffd00p-1, 0x1.4b13713a17652p-1, 0x1.7791b887dde61p-1, -0x1.ecef4230db664p-2, -0x1.15c3c5d9a8704p-5, 0x1.5f6890b0bf418p-3, -0x1.1da63fa92970dp-5, -0x1.385992af51a0cp-5, 0x1.fa08b9effbd90p-7, 0x1.716212c5c18e9p-8,
    0x1.7000000011033p-1, 0x1.61955607e8897p-1, 0x1.58a445da6bfebp-1, -0x1.ef6c246a1225bp-2, 0x1.e83e0da3ab4f1p-8, 0x1.44cc65df8e294p-3, -0x1.87d3c56aed039p-5, -0x1.f9271e0e28cb0p-6, 0x1.222d6de9d5c56p-6, 0x1.c0e0a2cd8b268p-9,
    0x1.900000009f1ddp-1, 0x1.762870f7824c5p-1, 0x1.39ccc1b09e755p-1, -0x1.ea4feea4baa26p-2, 0x1.715e5958ada8fp-5, 0x1.22cdbdb427cd7p-3, -0x1.da50aafc8c277p-5, -0x1.7557937190659p-6, 0x1.350f6162355edp-6, 0x1.3a72e142c85d7p-10,
    0x1.b00000005f11dp-1, 0x1.88d1cd477ed1ep-1, 0x1.1b7e98fdcd4d0p-1, -0x1.de65a22cb3b9fp-2, 0x1.40686a4098226p-4, 0x1.f6b0cb685497ep-4, -0x1.09c7c9687060bp-4, -0x1.da66985051185p-7, 0x1.362e0f270415fp-6, -0x1.d270b3d54489ap-11,
    0x1.cfffffffbaf31p-1, 0x1.999d4192832bap-1, 0x1.fc3ee5d1ce87ap-2, -0x1.cc990045de9fdp-2, 0x1.b37338e5b4f2dp-4, 0x1.a0d11fea9b15dp-4, -0x1.19bb2b5c888e3p-4, -0x1.a0b7ebbd883c4p-8, 0x1.272f1bff67b26p-6, -0x1.642d432022eebp-9,
    0x1.f00000009e1dap-1, 0x1.a89c850bc3219p-1, 0x1.c40b0728dedb1p-2, -0x1.b5eaaef0237dfp-2, 0x1.0847c7db9a3c2p-3, 0x1.47de0a4dde07bp-4, -0x1.1d9de7bb1618ep-4, 0x1.3324ec62f2168p-10, 0x1.0a9f0a5c16071p-6, -0x1.129831ea07549p-8,
    0x1.08000000550ffp+0, 0x1.b5e62fce58502p-1, 0x1.8eed36b775754p-2, -0x1.9b64a06db5aeap-2, 0x1.2bb6e2c7e6adbp-3, 0x1.dee322bcf377ap-5, -0x1.1699602fa999ap-4, 0x1.feab3c8dc1b04p-8, 0x1.c753196e34392p-7, -0x1.580a7136da7e8p-8,
    0x1.18000000c424cp+0, 0x1.c194b1d51fe9ep-1, 0x1.5d4fd334df8c3p-2, -0x1.7e0f4f02e024bp-2, 0x1.444bc66d20039p-3, 0x1.356dbb4c77eb5p-5, -0x1.0643de1ce63bcp-4, 0x1.b2e1f2766293ap-7, 0x1.6b9967fe23643p-7, -0x1.810c6ffefda6bp-8,
    0x1.27ffffffc5f52p+0, 0x1.cbc54b473fe14p-1, 0x1.2f7cc3ff0e614p-2, -0x1.5ee8429ea3d17p-2, 0x1.52a8395f73829p-3, 0x1.313759f608b1cp-6, -0x1.dcf844d75f96ep-5, 0x1.1e45effbf956ep-6, 0x1.091c836a3e5bfp-7, -0x1.8e78b5a2ab1cap-8,
    0x1.38000000d3279p+0, 0x1.d4970f9d4bf2fp-1, 0x1.059f59ad6c921p-2, -0x1.3eda354c341cep-2, 0x1.57b85ad442a5fp-3, 0x1.8e90c1cc03d4cp-10, -0x1.a2893bad123a7p-5, 0x1.4d6af274608c2p-6, 0x1.4ce5772628cefp-8, -0x1.830cedab48757p-8,
    0x1.47fffffed5c82p+0, 0x1.dc29fb5fef03bp-1, 0x1.bf8e1b21da261p-3, -0x1.1eb70960ab11fp-2, 0x1.549ea6f82272cp-3, -0x1.b10f20b0d3880p-7, -0x1.61420c54f73c9p-5, 0x1.677b7de201b93p-6, 0x1.254b31de2faddp-9, -0x1.62f2fd9890a13p-8,
    0x1.57fffffef3cdcp+0, 0x1.e29e22a839fadp-1, 0x1.7bd5c7e36d5a4p-3, -0x1.fe6744980d031p-3, 0x1.4a9fead05da81p-3, -0x1.a0082c84ecebdp-6, -0x1.1cf0e8ac40cccp-5, 0x1.6e339636e84c3p-6, -0x1.36d17f8f18ffap-12, -0x1.333aa25bf127cp-8,
    0x1.68000000520f6p+0, 0x1.e812fc64f4d86p-1, 0x1.3fda6bbef63d0p-3, -0x1.c1cb2784f0cd1p-3, 0x1.3b105122b62aep-3, -0x1.1e645a2bc236bp-5, -0x1.b1f6468d0f080p-6, 0x1.64297d7e86449p-6, -0x1.3dbbf4031aa89p-9, -0x1.f2a47718ff65ep-9,
    0x1.77ffffffd8f8bp+0, 0x1.eca6ccd6ff24bp-1, 0x1.0b3f52cf03e71p-3, -0x1.8885019fe4fd3p-3, 0x1.274275fcc2fa2p-3, -0x1.57f7386b8d6bcp-5, -0x1.3076a2417db99p-6, 0x1.4c8231a4c06a8p-6, -0x1.0bed0c6feae66p-8, -0x1.7516df49fc3f8p-9,
    0x1.88000000cf26dp+0, 0x1.f0762fde72c05p-1, 0x1.bb1c972ad9cdfp-4, -0x1.5341e3bd82097p-3, 0x1.107929f5b8877p-3, -0x1.7e1b3630300dep-5, -0x1.73b6240017e8bp-7, 0x1.2aa764aae8967p-6, -0x1.596614835c117p-8, -0x1.eed5214e71f53p-10,
    0x1.9800000117345p+0, 0x1.f39bc24315ef6p-1, 0x1.6c7e64e234fa4p-4, -0x1.2274b86508fbap-3, 0x1.efb890e253700p-4, -0x1.92c7dbb968795p-5, -0x1.45477ae53180ap-8, 0x1.02047b7b1b09ep-6, -0x1.884b839f66921p-8, -0x1.034723d9a72a5p-10,
    0x1.a800000087195p+0, 0x1.f62fe80285e16p-1, 0x1.297db95edcea4p-4, -0x1.ecb83b05bae2cp-4, 0x1.bce1836216a97p-4, -0x1.985aaf9789f89p-5, 0x1.cd956453bf940p-12, 0x1.ab9d44d776cafp-7, -0x1.9b63967ae6b61p-8, -0x1.9d2a57c5536f1p-13,
    0x1.b7ffffff59e0ep+0, 0x1.f848acb5315eap-1, 0x1.e1d4cf22571abp-5, -0x1.9e12e200e685bp-4, 0x1.8a27806ff9150p-4, -0x1.91674e142ecc7p-5, 0x1.3bc75763c0d42p-8, 0x1.51b4d28e1660bp-7, -0x1.96b672fb22620p-8, 0x1.e05294589e11dp-12,
    0x1.c8000000490dbp+0, 0x1.f9f9ba8d435afp-1, 0x1.83298d6fe8789p-5, -0x1.58d101f7e2492p-4, 0x1.58f1456ea80acp-4, -0x1.808d17b2e891ep-5, 0x1.0c1bda4b3d181p-7, 0x1.f5ff2052896bfp-8, -0x1.7f0ad9b78d3d9p-8, 0x1.f7d68af7e3812p-11,
    0x1.d80000001a04ep+0, 0x1.fb54641aedb28p-1, 0x1.34ac36ad1a001p-5, -0x1.1c8ec267a3a7bp-4, 0x1.2a52c5d7f685cp-4, -0x1.68541b2be3c86p-5, 0x1.5afe4071f21dbp-7, 0x1.56303fa7692cfp-8, -0x1.596cafa6e0568p-8, 0x1.576f61190e6d3p-10,
    0x1.e7ffffff13d3cp+0, 0x1.fc67bcf2c9a4ap-1, 0x1.e85c44a4ed2b2p-6, -0x1.d177f16c50c83p-5, 0x1.fe23b75d0f47ep-5, -0x1.4b120f9fb22c3p-5, 0x1.8d9905f68256bp-7, 0x1.9201be5251cb2p-9, -0x1.2ac5a6f696c5bp-8, 0x1.8d146f1179a64p-10,
    0x1.f7ffffff6be44p+0, 0x1.fd40bd6d738a3p-1, 0x1.7f5188647712fp-6, -0x1.7954424276541p-5, 0x1.af5baae5ebd6ep-5, -0x1.2ad77b790c56dp-5, 0x1.a7b8c486d6de1p-7, 0x1.4593b97cd6d97p-10, -0x1.ef1a27d9ce9dap-9, 0x1.a16b6a62408e5p-10,
    0x1.03fffffefdcfap+1, 0x1.fdea6e061a3b4p-1, 0x1.2a875b6988febp-6, -0x1.2f3178d6020d9p-5, 0x1.68d1c463f24aep-5, -0x1.09648dd7728e9p-5, 0x1.ad8b14f0b4b13p-7, -0x1.f00f64620bce0p-13, -0x1.8721c97e955c7p-9, 0x1.9a594ccb16682p-10,
    0x1.0c00000056102p+1, 0x1.fe6e1742fca83p-1, 0x1.cd5ec936ff421p-7, -0x1.e2ff3aa62e538p-6, 0x1.2aa4e57fce332p-5, -0x1.d049824d0b864p-6, 0x1.a34edae8a8bb7p-7, -0x1.682d877a237a0p-10, -0x1.23ae175b2b1b0p-9, 0x1.7e5c197b87c40p-10,
    0x1.13ffffff47dd8p+1, 0x1.fed37386111c3p-1, 0x1.61beae5c49b81p-7, -0x1.7d6193fa81093p-6, 0x1.e94727a74030ep-6, -0x1.906030162ad37p-6, 0x1.8d14d5ddc9d66p-7, -0x1.1f7959521b750p-9, -0x1.92528b9706934p-10, 0x1.53ebff434256cp-10,
    0x1.1c00000077165p+1, 0x1.ff20e0a7be75ap-1, 0x1.0d1d695244781p-7, -0x1.2a8ca0d7c124dp-6, 0x1.8cc071b21b006p-6, -0x1.54a148851c291p-6, 0x1.6e91375c3c5e2p-7, -0x1.65c02d4b8e55bp-9, -0x1.e9b5c95b18b9dp-11, 0x1.210079d7c4fbfp-10,
    0x1.23ffffff15d42p+1, 0x1.ff5b8fb26990dp-1, 0x1.9646f367b58dcp-8, -0x1.cf68eda0d7724p-7, 0x1.3e8735bdd96b1p-6, -0x1.1e1611b0a66c2p-6, 0x1.4afd8e1c22689p-7, -0x1.8c7200672605fp-9, -0x1.c7810d53df082p-12, 0x1.d5784ffb31f28p-11,
    0x1.2c000000fc2f4p+1, 0x1.ff87b19143343p-1, 0x1.30499b453f2afp-8, -0x1.649641f651c62p-7, 0x1.fa73d7dc69453p-7, -0x1.daa30050e297ap-7, 0x1.250943f668f48p-7, -0x1.9975798e333aep-9, -0x1.3f843a0204f0ap-15, 0x1.6a7b81a3f3f9bp-11,
    0x1.33ffffffc3f4cp+1, 0x1.ffa89fe5b28e3p-1, 0x1.c4412bf8b5ea7p-9, -0x1.100f34736864dp-7, 0x1.8ebda07954f80p-7, -0x1.850c68eb3579ap-7, 0x1.fdac857c5cd66p-8, -0x1.929de81be1badp-9, 0x1.100b05bb37c95p-12, 0x1.0722dea420912p-11,
    0x1.3bffffff01d06p+1, 0x1.ffc10194fa201p-1, 0x1.4d78bbb59013ep-9, -0x1.9ba107b2d2bbap-8, 0x1.36f2740590113p-7, -0x1.3b387097e8466p-7, 0x1.b3fe010c7e0f2p-8, -0x1.7d55d6cbf0058p-9, 0x1.ea43f6e7eac3ep-12, 0x1.5eefc5da010b5p-12,
    0x1.43fffffee2ca9p+1, 0x1.ffd2eae36780dp-1, 0x1.e7f232ef6289dp-10, -0x1.34c7443a6c8b3p-8, 0x1.e066bee2133c2p-8, -0x1.f914f2d5f7a16p-8, 0x1.6f46648edd747p-8, -0x1.5e6646f8dc224p-9, 0x1.39d319fa319f1p-11, 0x1.96c0873ddfe09p-13,
    0x1.4bffffffb9f2ep+1, 0x1.ffdff92db50d6p-1, 0x1.6235fbdb91d00p-10, -0x1.cb5e02a0602bbp-9, 0x1.6fa4c7f29d89bp-8, -0x1.903a08339148ap-8, 0x1.30f12dbdda7fap-8, -0x1.39d76b0fb9674p-9, 0x1.5d454a0693d2fp-11, 0x1.53f34152ff5d9p-14,
    0x1.5400000028078p+1, 0x1.ffe96a78a0727p-1, 0x1.fe41cd9865373p-11, -0x1.52d7b2875b1a9p-9, 0x1.16c192d6e7c74p-8, -0x1.39bfce99b9c79p-8, 0x1.f376a71f5dfa9p-9, -0x1.12e67dfba8babp-9, 0x1.66b084b77af1dp-11, -0x1.4961aa2f85014p-18,
    0x1.5bffffff5be14p+1, 0x1.fff0312b00967p-1, 0x1.6caa0d3f71674p-11, -0x1.efb72a01545efp-10, 0x1.a2da7cf5abdcep-9, -0x1.e6c27adcb5771p-9, 0x1.93b1f48e2fefep-9, -0x1.d8179efc1d592p-10, 0x1.5cdac8abab58ap-11, -0x1.163c7818873dap-14,
    0x1.63ffffffddf9ap+1, 0x1.fff50456daa79p-1, 0x1.0295ef670fdf3p-11, -0x1.679880eb2fb3ep-10, 0x1.37d38e3bf033cp-9, -0x1.75b371a3fc74fp-9, 0x1.4231c4838bdcbp-9, -0x1.8e184f0f6d88cp-10, 0x1.45c5821e0cb15p-11, -0x1.bf0d55d0dbb87p-14,
    0x1.6c000000971c5p+1, 0x1.fff86cfd3e9b2p-1, 0x1.6be020f9281f9p-12, -0x1.02b157718deb7p-10, 0x1.cc1d885ded29ep-10, -0x1.1bff70605b2f6p-9, 0x1.fc0f778239564p-10, -0x1.4a2229c071dfap-10, 0x1.2680710cd803dp-11, -0x1.0f7039ddcf455p-13,
    0x1.74000000da28ep+1, 0x1.fffad0b901ab7p-1, 0x1.fc0d553363db8p-13, -0x1.7121afe82f08dp-11, 0x1.506d698797e85p-10, -0x1.ab596008b79f0p-10, 0x1.8bdd79c400a85p-10, -0x1.0d88db9983033p-10, 0x1.031af07e0b4bap-11, -0x1.22d769aca3383p-13,
    0x1.7bffffffdaf91p+1, 0x1.fffc7a378576cp-1, 0x1.5feada39f9fbcp-13, -0x1.05304df6ee171p-11, 0x1.e79c081e62ef3p-11, -0x1.3e5dc107d7069p-10, 0x1.30eb2092cf855p-10, -0x1.b1b06d82ab718p-11, 0x1.bd57ef68519d6p-12, -0x1.2131c8ccda832p-13,
    0x1.840000008c1a4p+1, 0x1.fffd9fdeabdd7p-1, 0x1.e3bcf42a17b3cp-14, -0x1.6e9531086a580p-12, 0x1.5e3edf5f576fep-11, -0x1.d5be6d0baa2efp-11, 0x1.d07da033e7aabp-11, -0x1.58106d9d1f3d2p-11, 0x1.76d2fcf196e53p-12, -0x1.110e1f3ac13b8p-13,
    0x1.8c00000103309p+1, 0x1.fffe68f4fa8c5p-1, 0x1.49e17714cfad3p-14, -0x1.fe48c4357f445p-13, 0x1.f2bd95c1a146bp-12, -0x1.5738917ac6169p-11, 0x1.5decc2a7063bfp-11, -0x1.0d559d5a5a194p-11, 0x1.3591a2f7f4ba3p-12, -0x1.efc74cfb2c57cp-14,
    0x1.93ffffff37da8p+1, 0x1.fffef1960d7aep-1, 0x1.be6abbc240af3p-15, -0x1.60403826988e5p-13, 0x1.5fff1deaa9f68p-12, -0x1.f0c93c83cfd09p-12, 0x1.04cbf50df8d7dp-11, -0x1.a048939fd49d0p-12, 0x1.f68a5eeb819fbp-13, -0x1.b40bfa6d60924p-14,
    0x1.9c000000d8288p+1, 0x1.ffff4db27f1c5p-1, 0x1.2bb5cc162b9b3p-15, -0x1.e2589474ab4aap-14, 0x1.ec8a8e4776672p-13, -0x1.6425721ef32cbp-12, 0x1.80a837772d059p-12, -0x1.3dbb933f65568p-12, 0x1.915a68363fa76p-13, -0x1.7566cabfc0a09p-14,
    0x1.a3fffffee8cbbp+1, 0x1.ffff8b500e70fp-1, 0x1.8f4cccbe505bbp-16, -0x1.478cfff34436ep-14, 0x1.559f04beee3b2p-13, -0x1.f9e163c95cf07p-13, 0x1.18bda6001e1c7p-12, -0x1.df381afc67a3bp-13, 0x1.3bb27eb1c8d4dp-13, -0x1.38678f37763d3p-14,
    0x1.abffffffa8efbp+1, 0x1.ffffb43555b49p-1, 0x1.07ebd2a782f92p-16, -0x1.b93e442fb5496p-15, 0x1.d5cf151cdaa44p-14, -0x1.63f5eb4c07032p-13, 0x1.95a03c211df8bp-13, -0x1.652e5df5294c1p-13, 0x1.e98652d57fa74p-14, -0x1.000101308d836p-14,
    0x1.b3ffffff9dedap+1, 0x1.ffffcf23ff5ebp-1, 0x1.5a2adfa7c3839p-17, -0x1.26c882749a3f7p-15, 0x1.404735786213dp-14, -0x1.f057dbfc528bbp-14, 0x1.22178e43a9135p-13, -0x1.07323ebc98125p-13, 0x1.76560deef7de9p-14, -0x1.9bbb3189972e1p-15,
    0x1.bc00000108318p+1, 0x1.ffffe0bd3e86fp-1, 0x1.c282cd2024dfcp-18, -0x1.86ad6de2c88bap-16, 0x1.b0f313d9a0c59p-15, -0x1.56e457640c00fp-14, 0x1.9ad1eed9191e8p-14, -0x1.7f92aabb6f3dfp-14, 0x1.1a7d1d100dffbp-14, -0x1.4561c5cd6104fp-15,
    0x1.c40000010430cp+1, 0x1.ffffec2641ab0p-1, 0x1.22df2971c4509p-18, -0x1.00c902970335dp-16, 0x1.22234ea9370c0p-15, -0x1.d57a2bc9b393ap-15, 0x1.200c29c68f518p-14, -0x1.14758338d1185p-14, 0x1.a4f21bff16086p-15, -0x1.f9ff5dfaa04a1p-16,
    0x1.cc00000002006p+1, 0x1.fffff37d63a36p-1, 0x1.74adc8f3dc35bp-19, -0x1.4ed4228b196fep-17, 0x1.81918baddc04fp-16, -0x1.3e81c09c72ac9p-15, 0x1.9004a5f638c34p-15, -0x1.8a40dcf098b34p-15, 0x1.35c7669e84bf8p-15, -0x1.83756940dad99p-16,
    0x1.d4000000a41ecp+1, 0x1.fffff82cdcf20p-1, 0x1.d9c73687a0a43p-20, -0x1.b11017d890eaep-18, 0x1.fc0dfacd357a6p-17, -0x1.ac4e1a9786884p-16, 0x1.131808ba345afp-15, -0x1.1629d552482bdp-15, 0x1.c27ecce107b4dp-16, -0x1.246858abb1a37p-16,
    0x1.dbfffffed7c88p+1, 0x1.fffffb248c398p-1, 0x1.2acee30a03a1ap-20, -0x1.15cc5712a2aa9p-18, 0x1.4be757cf8ee5cp-17, -0x1.1d6ab70a53347p-16, 0x1.76c596c494920p-16, -0x1.84732bd381ae4p-16, 0x1.43c0e3385a525p-16, -0x1.b342340effa51p-17,
    0x1.e400000028078p+1, 0x1.fffffd01f36afp-1, 0x1.75fa8db90fe33p-21, -0x1.6186d9f90e825p-19, 0x1.ae02322cf8f4ap-18, -0x1.79082bedb3d8ap-17, 0x1.f9c25b38ce26bp-17, -0x1.0c767cd43d1e8p-16, 0x1.cc0bd83d6f68ep-17, -0x1.3fa6e36ec5d24p-17,
    0x1.ec000000b6222p+1, 0x1.fffffe2ba0ea6p-1, 0x1.d06ad6d906e37p-22, -0x1.be46aa7532349p-20, 0x1.143860bb9dd5ap-18, -0x1.edabcbb2a300fp-18, 0x1.52138e3c56d4dp-17, -0x1.6f56743ce9a64p-17, 0x1.4337cec096dbfp-17, -0x1.cf7d5621ecd9fp-18,
    0x1.f3fffffee4cafp+1, 0x1.fffffee3cc32bp-1, 0x1.1e1e858e2da3cp-22, -0x1.1769ce6c3a966p-20, 0x1.5fe5d48e77b77p-19, -0x1.405da05d015bfp-18, 0x1.bfc955826a39cp-18, -0x1.f19fe8a11298ap-18, 0x1.c135b9e65d954p-18, -0x1.4bdb14109e2e6p-18,
    0x1.fbffffff22d69p+1, 0x1.ffffff54dab71p-1, 0x1.5dcd66b1e9969p-23, -0x1.5b11cbe3ef137p-21, 0x1.bc91a6cc510eap-20, -0x1.9c2c5d2888726p-19, 0x1.25d1d45480473p-18, -0x1.4dbe1c99a0819p-18, 0x1.34ce6311c524cp-18, -0x1.d57ad3155e248p-19,
    0x1.020000003409cp+2, 0x1.ffffff99b79d2p-1, 0x1.a854ea09317e4p-24, -0x1.aba593dd9abb3p-22, 0x1.167c2526b3c05p-20, -0x1.06d78c9b91931p-19, 0x1.7e0f4390d108cp-19, -0x1.bb4d38c27d485p-19, 0x1.a416a3f49fbf8p-19, -0x1.482eb849f2660p-19,
    0x1.05ffffffcef6dp+2, 0x1.ffffffc355dfdp-1, 0x1.febc1089e18ffp-25, -0x1.055a3c765def7p-22, 0x1.59ff3782d256bp-21, -0x1.4c53adc344c30p-20, 0x1.ec490449eb472p-20, -0x1.23926f70d7e61p-19, 0x1.1ac321899336ap-19, -0x1.c58c0b62bb2e7p-20,
    0x1.09fffed000000p+2, 0x1.ffffffdc4ad1fp-1, 0x1.30f96b404c834p-25, -0x1.3ce32806a7eb6p-23, 0x1.aa504e61b5983p-22, -0x1.a08f2c1dde786p-21, 0x1.3a4a7ec9c066ap-20, -0x1.7be208779a2a0p-20, 0x1.78bf677671786p-20, -0x1.35df2f88d26a2p-20,
    0x1.0dfff64000000p+2, 0x1.ffffffeb242afp-1, 0x1.6963895c8f53ep-26, -0x1.7d26ed1c158d5p-24, 0x1.0477ecdcaa587p-22, -0x1.02d4d2ac22f9dp-21, 0x1.8db4f764b4138p-21, -0x1.ea40eecfe68b6p-21, 0x1.f0e37a1fd2028p-21, -0x1.a2be4fcecdfa4p-21,
    0x1.11ffffff78e6bp+2, 0x1.fffffff3e8892p-1, 0x1.a8e406044fadbp-27, -0x1.c6c40e6fbe34dp-25, 0x1.3ba47a324e00ap-23, -0x1.3ee334d687c8dp-22, 0x1.f2bf73b102fd5p-22, -0x1.395bf7c43c288p-21, 0x1.4460916b92f31p-21, -0x1.17dcadf7e919ep-21,
    0x1.15fffba000000p+2, 0x1.fffffff90b29fp-1, 0x1.efad77e5d2fcbp-28, -0x1.0d232bdd7ee55p-25, 0x1.7b5c9eea0757fp-24, -0x1.8588f514b36c3p-23, 0x1.35f4b36428f47p-22, -0x1.8cda394f31e0fp-22, 0x1.a35431b632cfbp-22, -0x1.7216b7feec3a8p-22,
    0x1.1a000ef000000p+2, 0x1.fffffffc07515p-1, 0x1.1edd55bbde8c6p-28, -0x1.3bffe12dfe571p-26, 0x1.c42c07c98cd8ep-25, -0x1.d7c3482cc8759p-24, 0x1.7dd3ec704295bp-23, -0x1.f1e8a1b8b0bf1p-23, 0x1.0c5dd91bf17b8p-22, -0x1.e440ce4885c41p-23,
    0x1.1dffeee000000p+2, 0x1.fffffffdbfed2p-1, 0x1.497cc07db01adp-29, -0x1.70194901f3dd9p-27, 0x1.0b4ad5fa39ae6p-25, -0x1.1b47261d1d1e4p-24, 0x1.d243a1fd3b635p-24, -0x1.357fce182a245p-23, 0x1.5431ea26a184ep-23, -0x1.39872badea599p-23,
    0x1.22000ce000000p+2, 0x1.fffffffebc1cfp-1, 0x1.7772c24ab56dcp-30, -0x1.a95012fa88d0ep-28, 0x1.3960cdea56c7ap-26, -0x1.51470d8c10e16p-25, 0x1.1a2773afb93eep-24, -0x1.7d33559a0d196p-24, 0x1.ab0bc15b8db47p-24, -0x1.91d2b18377cb1p-24,
    0x1.26000d1000000p+2, 0x1.ffffffff4b469p-1, 0x1.a884a11bafff8p-31, -0x1.e78866af12e68p-29, 0x1.6c6c668f48a83p-27, -0x1.8e3436bdaaa8cp-26, 0x1.52848875a7b5fp-25, -0x1.d1431abbbcffdp-25, 0x1.097caead050d9p-24, -0x1.fdc3f3f3766b5p-25,
    0x1.2a00003000000p+2, 0x1.ffffffff9bec8p-1, 0x1.dc4790e26645bp-32, -0x1.1535a7806dcc4p-29, 0x1.a45473f4ef3c2p-28, -0x1.d230814bb4b3cp-27, 0x1.929d04532a057p-26, -0x1.195d9ed5e3a87p-25, 0x1.46f98da701288p-25, -0x1.401c91d73e07ep-25,
    0x1.2dfffde000000p+2, 0x1.ffffffffc901bp-1, 0x1.0917435c9ff17p-32, -0x1.38b96f43f5430p-30, 0x1.e0d806278f57ep-29, -0x1.0e97afa495a43p-27, 0x1.daadcfc94c28ep-27, -0x1.513c8c46a178ep-26, 0x1.8ee78301dd8d8p-26, -0x1.8e0b97da2fd7fp-26,
    0x1.31fffb1000000p+2, 0x1.ffffffffe202cp-1, 0x1.24cbcac41dcfdp-33, -0x1.5dfb92b8bffb4p-31, 0x1.10cae03e495d9p-29, -0x1.377d54a34319ap-28, 0x1.1566d646e4aedp-27, -0x1.9093cd50c0f23p-27, 0x1.e21b782958b61p-27, -0x1.ea16c43bfeea8p-27,
    0x1.36000d6000000p+2, 0x1.ffffffffefc59p-1, 0x1.40dd4ed7a6ec7p-34, -0x1.848c0e3cb722ap-32, 0x1.32fc821c9f79bp-30, -0x1.638d54f8539c0p-29, 0x1.416a9dd14a292p-28, -0x1.d78c2df96154ap-28, 0x1.209d1ef6896b0p-27, -0x1.2ac51cfec1826p-27,
    0x1.3a000a8000000p+2, 0x1.fffffffff748fp-1, 0x1.5ce77964794e7p-35, -0x1.abf3f934bf08ep-33, 0x1.56ac0e5bdaf94p-31, -0x1.927a429357eacp-30, 0x1.713ad887ea1fdp-29, -0x1.13174994ee887p-28, 0x1.56617d04061f0p-28, -0x1.68c1af3a72a16p-28,
    0x1.3dfff16000000p+2, 0x1.fffffffffb5afp-1, 0x1.787630dbd0dbap-36, -0x1.d3a2bb2f51f2bp-34, 0x1.7b6ae59bd21a3p-32, -0x1.c3d2965a74389p-31, 0x1.a48a71f6f8094p-30, -0x1.3e23969b0ad26p-29, 0x1.92742fc5d9a1fp-29, -0x1.af6e00cb040d2p-29,
    0x1.4200036000000p+2, 0x1.fffffffffd8b3p-1, 0x1.92fe5d29d1505p-37, -0x1.fae3f67eb9835p-35, 0x1.a0a73552093e8p-33, -0x1.f6f3818f6bf54p-32, 0x1.dad81cc61ce44p-31, -0x1.6ca5a7e674aeap-30, 0x1.d4b4d81cd1a13p-30, -0x1.ff0a5c4226a96p-30,
    0x1.46000c7000000p+2, 0x1.fffffffffeb60p-1, 0x1.ac0c0fbc76fc0p-38, -0x1.108bb86aee1dep-35, 0x1.c5d7b7eaf55a2p-34, -0x1.159d3d688a518p-32, 0x1.09ccb45bbf0eap-31, -0x1.9e4a8bbdeb8ecp-31, 0x1.0e75551f44ee0p-30, -0x1.2bcfe1447396bp-30,
    0x1.49fff08000000p+2, 0x1.ffffffffff542p-1, 0x1.c32928d57a5d4p-39, -0x1.22c979a91d472p-36, 0x1.ea6400ef0822ep-35, -0x1.2ff4ab4e40581p-33, 0x1.27103a5c2e0c3p-32, -0x1.d29cf57ecea39p-32, 0x1.355434c9584d8p-31, -0x1.5c7b04b118f5bp-31,
    0x1.4e07d00000000p+2, 0x1.ffffffffffa7ap-1, 0x1.d56df3afb136bp-40, -0x1.3241e3acff62ep-37, 0x1.0583baac47a78p-35, -0x1.48771a28932f1p-34, 0x1.434086d27d863p-33, -0x1.034995776ace7p-32, 0x1.5d0a285a7f300p-32, -0x1.9145bbba7a68cp-32,
    0x1.520c500000000p+2, 0x1.ffffffffffd2dp-1, 0x1.e5a22f16cc8a1p-41, -0x1.40a3bec446aabp-38, 0x1.15360e1c76a49p-36, -0x1.60b28c82a5966p-35, 0x1.5fcc2259013eep-34, -0x1.1e2e5911fd606p-33, 0x1.870335fb8eae7p-33, -0x1.c9c749faedb3ep-33,
    0x1.560c000000000p+2, 0x1.ffffffffffe90p-1, 0x1.f4053945a3efcp-42, -0x1.4e0b35609d592p-39, 0x1.245708bed3fd1p-37, -0x1.78aed84836fa1p-36, 0x1.7cb53ba14cafap-35, -0x1.39ff326444b2cp-34, 0x1.b34ddf917372bp-34, -0x1.02b6b58c9a1dap-33,
    0x1.5a02b00000000p+2, 0x1.fffffffffff45p-1, 0x1.00efb7dbef055p-42, -0x1.5b46b10375018p-40, 0x1.33912201cc437p-38, -0x1.913d1b4cc0236p-37, 0x1.9ac875d4fbc5fp-36, -0x1.5764ca24965d0p-35, 0x1.e2db6a991c92fp-35, -0x1.21be3249e6c0ep-34,
    0x1.5deea00000000p+2, 0x1.fffffffffffa1p-1, 0x1.07ec73bdaf155p-43, -0x1.68c35c9182758p-41, 0x1.434225efaa157p-39, -0x1.aad659cd86c05p-38, 0x1.ba842b8b12098p-37, -0x1.76d01328ae9cdp-36, 0x1.0b27bb0a038b5p-35, -0x1.41888441f2b8fp-35,
    0x1.61f6700000000p+2, 0x1.fffffffffffd1p-1, 0x1.080e9d93e719ep-44, -0x1.6d1a58db1b9d5p-42, 0x1.4b0ae49aaa790p-40, -0x1.ba82431ede0bep-39, 0x1.d0a4a52f2bc90p-38, -0x1.8ecdfe1adcb07p-37, 0x1.20434953bc460p-36, -0x1.6192636015999p-36,
    0x1.6602b00000000p+2, 0x1.fffffffffffe9p-1, 0x1.054f702a029c8p-45, -0x1.6d6fd5202f2b8p-43, 0x1.4f427f4a98d6bp-41, -0x1.c5a084fb06f16p-40, 0x1.e25ce9c18e231p-39, -0x1.a3791ad9c019fp-38, 0x1.336c26ecdb337p-37, -0x1.8149e599fc53bp-37,
    0x1.68cc000000000p+2, 0x1.ffffffffffff2p-1, 0x1.407f57e315ab6p-46, -0x1.c3b2790f84330p-44, 0x1.a1b9f6cb76374p-42, -0x1.1cf42c19c71e1p-40, 0x1.319deb2a305ccp-39, -0x1.0c075731bf7c2p-38, 0x1.8681734994393p-38, -0x1.a012834c18e23p-38,
    0x1.6d80000000000p+2, 0x1.ffffffffffffap-1, 0x1.166731200af63p-47, -0x1.8d7c54a5470a5p-45, 0x1.748930ba50597p-43, -0x1.01a8ff3ad5550p-41, 0x1.1853ad632d4b5p-40, -0x1.f35e3e801af5bp-40, 0x1.7604983c91240p-39, -0x1.bd49ee38ecf75p-39,
    0x1.7150000000000p+2, 0x1.ffffffffffffdp-1, 0x1.18f97925219c2p-48, -0x1.9557659464a84p-46, 0x1.7ffbe5aa2b92ep-44, -0x1.0c87370fbfd54p-42, 0x1.2782f8872b9d0p-41, -0x1.0a56cd2251979p-40, 0x1.92dde13772db4p-40, -0x1.d84d888340823p-40,
    0x1.7744000000000p+2, 0x1.fffffffffffffp-1, 0x1.7cd7f3f568286p-50, -0x1.1722bfddae5abp-47, 0x1.0cd1c8d5bbba5p-45, -0x1.7e6d31c2d3dabp-44, 0x1.ac4e48038ae79p-43, -0x1.89760edb1c4b1p-42, 0x1.2947771fe604cp-41, -0x1.f0803b4ca9cfcp-41,
    0x1.7884000000000p+2, 0x1.fffffffffffffp-1, 0x1.2ec454f68b001p-50, -0x1.bd4c7a0c0f73ep-48, 0x1.ae4fddf5d1840p-46, -0x1.332a9e85f6902p-44, 0x1.59434226a3768p-43, -0x1.3da34280fdeb9p-42, 0x1.e27ec59e69a45p-42, -0x1.02a83150acae8p-41,
    0x1.7f7c000000000p+2, 0x1.0000000000000p+0, 0x1.4c5cefd624816p-52, -0x1.f1e007c92827ep-50, 0x1.ea4849b878b3ap-48, -0x1.64d8928dabc28p-46, 0x1.9938ad62c3fc2p-45, -0x1.81c13e54d0560p-44, 0x1.26f0233894f3cp-43, -0x1.0b1ebf86004ddp-42,
};"""

ERF_F8 = r"""
/* erf(x) from a table of polynomials: |x| below 6 falls into one of 96 intervals of width
   1/16; on each, erf is a polynomial of degree 8 in the distance from a point c near the
   middle (chosen so that erf(c), the constant term, is a double to within 0.2 ulp).  The
   first interval is centred on 0 with a zero constant term, which keeps full relative
   accuracy down to the smallest arguments.  An entry is c and the nine coefficients
   (80 bytes, five 16-byte loads); no exponential, no division, no branch.
   erfc(6) < 2^-54: arguments from 6 up are moved to the last double below 6. */
template <int P>
DR_FN void dr_erf_f8(const double (&x)[P], double (&out)[P])
{
    double t[P], p[P];
    DR_TAB_PTR row[P];
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double a = __builtin_fabs(x[e]);
        const double b = a > 0x1.7ffffffffffffp+2 ? 0x1.7ffffffffffffp+2 : a;    /* NaN stays NaN */
        row[e] = DR_ERF_TAB + 10 * (int)(b * 16.0);
        t[e] = b - row[e][0];
        p[e] = row[e][9];
    }
    _Pragma("unroll") for (int j = 8; j >= 1; --j)
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            p[e] = __builtin_fma(p[e], t[e], row[e][j]);
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        out[e] = __builtin_copysign(p[e], x[e]);
}"""

SQRT_F8 = r"""
/* Correctly rounded square root: reciprocal square root estimate, one coupled step for
   g ~ sqrt(x) and h ~ 1/(2 sqrt(x)), two residual corrections d = x - g^2, g += d h; the
   last fused operation rounds once.  This is the compiler's own expansion of sqrt for
   arguments that need no rescaling; zero, negative, infinite, NaN and arguments below
   2^-767 (whose estimate would lose bits) go to that expansion, on a path a wave skips
   when none of its lanes needs it. */
template <int P>
DR_FN void dr_sqrt_f8(const double (&x)[P], double (&out)[P])
{
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double y = DR_RSQ64(x[e]);
        double g = x[e] * y;
        double h = 0.5 * y;
        const double r = __builtin_fma(-h, g, 0.5);
        g = __builtin_fma(g, r, g);
        h = __builtin_fma(h, r, h);
        double d = __builtin_fma(-g, g, x[e]);
        g = __builtin_fma(d, h, g);
        d = __builtin_fma(-g, g, x[e]);
        out[e] = __builtin_fma(d, h, g);
    }
    bool rare = false;
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        rare |= !(x[e] >= 0x1p-767 && x[e] < __builtin_inf());
    if (DR_ANY_LANE(rare)) {        /* one test per wave: the compiler must not fold this into selects */
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            if (!(x[e] >= 0x1p-767 && x[e] < __builtin_inf()))
                out[e] = __builtin_sqrt(x[e]);
    }
}
/* The same for square roots that nothing reads but functions which round on their own
   (erf(x / (s * sqrt(t)))): the estimate, the coupled step for g alone and one correction
   by the residual, seven operations instead of ten.  The result is the correctly
   rounded root except in about one case in 2^20, then the neighbouring double. */
template <int P>
DR_FN void dr_sqrt_near_f8(const double (&x)[P], double (&out)[P])
{
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        const double y = DR_RSQ64(x[e]);
        double g = x[e] * y;
        const double h = 0.5 * y;
        const double r = __builtin_fma(-h, g, 0.5);
        g = __builtin_fma(g, r, g);
        const double d = __builtin_fma(-g, g, x[e]);
        out[e] = __builtin_fma(d, h, g);
    }
    bool rare = false;
    _Pragma("unroll") for (int e = 0; e < P; ++e)
        rare |= !(x[e] >= 0x1p-767 && x[e] < __builtin_inf());
    if (DR_ANY_LANE(rare)) {
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            if (!(x[e] >= 0x1p-767 && x[e] < __builtin_inf()))
                out[e] = __builtin_sqrt(x[e]);
    }
}
DR_FN double dr_sqrt_near_f8_1(double x)
{
    const double a[1] = {x};
    double r[1];
    dr_sqrt_near_f8<1>(a, r);
    return r[0];
}"""

DIV_F8 = r"""
/* a / b for quotients that nothing reads but functions which round on their own
   (log(a / b), erf(x / s)): the reciprocal estimate, one refinement, the product and
   one correction by the exact residual, six operations where the correctly rounded
   division takes thirteen (it refines twice, scales both operands first, so that no
   intermediate result leaves the normal range, and fixes up the special cases
   afterwards).  An estimate good to e makes the refined reciprocal good to e^2, the
   product likewise, and the correction squares that again: from 14 bits on the quotient
   is right to 2^-56 before it is rounded.  The result is the correctly rounded
   quotient except in about one case in 2^20, then the neighbouring double (checked
   against exact quotients in tests/test_mathlib.py, and on the device).
   Operands that need the scaling or the special cases show in the result (not a normal
   number: a NaN from 0 or infinity times its reciprocal, an infinity, a denormal, a zero,
   whose sign the correction would lose) or in the numerator (below 2^-1000 its residual,
   2^-48 of it, falls among the denormals and corrects nothing) and take the compiler's
   division, on a path a wave skips when none of its lanes needs it. */
#define DR_DIV_RARE(q, a) (!(__builtin_isnormal(q) && __builtin_fabs(a) >= 0x1p-1000))
template <int P>
DR_FN void dr_div_f8(const double (&a)[P], const double (&b)[P], double (&out)[P])
{
    bool rare = false;
    _Pragma("unroll") for (int e = 0; e < P; ++e) {
        double y = DR_RCP64(b[e]);
        const double t = __builtin_fma(-b[e], y, 1.0);
        y = __builtin_fma(y, t, y);
        double q = a[e] * y;
        const double r = __builtin_fma(-b[e], q, a[e]);
        q = __builtin_fma(r, y, q);
        out[e] = q;
        rare |= DR_DIV_RARE(q, a[e]);
    }
    if (DR_ANY_LANE(rare)) {
        _Pragma("unroll") for (int e = 0; e < P; ++e)
            if (DR_DIV_RARE(out[e], a[e]))
                out[e] = a[e] / b[e];
    }
}
DR_FN double dr_div_f8_1(double a, double b)
{
    const double x[1] = {a}, y[1] = {b};
    double r[1];
    dr_div_f8<1>(x, y, r);
    return r[0];
}"""

# ufunc name -> (device function template, sources it needs in order), float64 only
FUNCTIONS = {
    "log": ("dr_log_f8", (STEP, LOG_TABLE, LOG_CORE, LOG_F8)),
    "erf": ("dr_erf_f8", (ERF_TABLE, ERF_F8)),
    "exp": ("dr_exp_f8", (STEP, EXPM1_REDUCED, EXP_F8)),
    "sqrt": ("dr_sqrt_f8", (SQRT_F8,)),
}

# Where the functions read their tables.  In memory (the default): every lane's 16-byte
# load goes to a different row, which the vector memory path serves slowly (Black-Scholes
# float64 with `erf` reading its table from memory: 405 us).  In LDS: the kernel copies the
# tables in once per workgroup (`DR_STAGE_TABLES`, before anything else, every thread) and
# the functions read the copy (262 us; 244 us when a workgroup stays for several chunks, so
# that the copy is shared by more elements).
TABLE_SIZES = {"log": ("dr_log_tab", 512, "DR_LOG_TAB"), "erf": ("dr_erf_tab", 960, "DR_ERF_TAB")}

TABLES_IN_MEMORY = """\
#define DR_TAB_PTR const double*
{defines}
"""

TABLES_IN_LDS = """\
typedef double dr_tab2 __attribute__((ext_vector_type(2)));     /* the copies move 16 bytes per lane */
#define DR_TAB_PTR const __attribute__((address_space(3))) double*
{arrays}
{defines}
#define DR_STAGE_TABLES() do {{ {copies} __syncthreads(); }} while (0)
"""


def tables(names):
    """The tabulated functions among `names`."""
    return [name for name in names if name in TABLE_SIZES]


SCALAR_WRAPPER = """
DR_FN double {fn}_1(double x)
{{
    const double a[1] = {{x}};
    double r[1];
    {fn}<1>(a, r);
    return r[0];
}}
"""


def source(names, macros=DEVICE_MACROS, lds=0, stage_loop=False, soft_div=False):
    """Definitions of the function templates for the ufuncs in `names` (each piece
    once) and of their one-element forms `<function>_1(double)`.  `lds`: the functions
    read their tables from LDS copies, which a kernel with blocks of `lds` threads makes
    with `DR_STAGE_TABLES()`."""
    pieces = []
    for name in names:
        for piece in FUNCTIONS[name][1]:
            if piece not in pieces:
                pieces.append(piece)
    if not pieces:
        return macros + DIV_F8 if soft_div else ""
    tabs = tables(names)
    if lds and tabs:
        # Every lane first asks for all its 16-byte pieces of all tables and then writes
        # them: one trip to memory per block, not one per piece (a loop waits for each
        # piece before it asks for the next).
        loads, stores = [], []
        for t in tabs:
            name, count, _ = TABLE_SIZES[t]
            for k, first in enumerate(range(0, count // 2, lds)):
                some = count // 2 - first < lds     # the last piece of a table: some lanes only
                cond = f"threadIdx.x < {count // 2 - first}" if some else ""
                var = f"dr_t_{name}_{k}"
                src = f"((const dr_tab2*){name})[{first} + threadIdx.x]"
                loads.append(f"dr_tab2 {var}; if ({cond}) {var} = {src};" if some else f"const dr_tab2 {var} = {src};")
                dst = f"((dr_tab2*){name}_lds)[{first} + threadIdx.x] = {var};"
                stores.append(f"if ({cond}) {dst}" if some else dst)
        if stage_loop:
            loads = [f"for (int i_ = threadIdx.x; i_ < {TABLE_SIZES[t][1] // 2}; i_ += {lds}) "
                     f"((dr_tab2*){TABLE_SIZES[t][0]}_lds)[i_] = ((const dr_tab2*){TABLE_SIZES[t][0]})[i_];"
                     for t in tabs]
            stores = []
        where = TABLES_IN_LDS.format(
            arrays="\n".join(f"__shared__ DR_ALIGN16 double {TABLE_SIZES[t][0]}_lds[{TABLE_SIZES[t][1]}];" for t in tabs),
            defines="\n".join(f"#define {TABLE_SIZES[t][2]} ((DR_TAB_PTR){TABLE_SIZES[t][0]}_lds)" for t in tabs),
            copies=" ".join(loads + stores))
    else:
        where = TABLES_IN_MEMORY.format(
            defines="\n".join(f"#define {TABLE_SIZES[t][2]} {TABLE_SIZES[t][0]}" for t in tabs))
    # the tables themselves come first, then where they are read from, then the functions
    table_text = [p for p in pieces if p in (LOG_TABLE, ERF_TABLE)]
    rest = [p for p in pieces if p not in (LOG_TABLE, ERF_TABLE)]
    wrappers = "".join(SCALAR_WRAPPER.format(fn=FUNCTIONS[name][0]) for name in names)
    return macros + "".join(table_text) + "\n" + where + "".join(rest) + wrappers + (DIV_F8 if soft_div else "")
