"""HIP C++ source generation for fused expression kernels (gfx950).

Takes the place of the reference's CUDA-C emitter (delayrepay/cuda.py:46-88,
`CupyEmitter`, and `make_kernel`, :35-43).  The expression arrives as a
`Program`: a flat SSA list produced by one memoised walk of the DAG
(`hip.Tracer`), so a shared sub-expression is emitted once by construction;
the reference re-walks shared nodes and removes duplicate statements
afterwards (`dedup`, cuda.py:29-32).

Differences in what is emitted:
  * every value has its own C type (NumPy promotion), not one generic `T`;
  * Python scalars are typed kernel parameters, not literals, so an f32
    expression never computes in double and the kernel is reusable for any
    scalar value (the reference inlines `str(val)`, cuda.py:84-85);
  * names are positional (`l0`, `s1`, `v7`), so structurally equal
    expressions produce identical source and hit the kernel cache (the
    reference embeds a global serial number, delayarray.py:150-152).

Kernel shapes (all 256-thread blocks = 4 wave64):
  flat      contiguous operands: one run of 256 16-byte vectors per block, optional
            non-temporal access, scalar tail; supplies the element index to
            index-valued leaves (`arange`, `linspace`)          emit_flat
  tile2d    N-d operands whose last dimension has unit or zero stride; shifted views
            of one buffer are staged once through an LDS halo tile, tiles go to XCDs
            in contiguous bands                     emit_stencil, emit_stencil_vec
  tile2dt   some operand is a transposed matrix: 64x64 LDS transpose, diagonal tile
            order                                               emit_tile_transpose
  nd        arbitrary strides / broadcasting, one element per thread-iteration
                                                                emit_nd
  axis_*    reductions along some axes: col / row (sliced, two passes), short rows
            (a lane per output), narrow matrices (streamed, per-lane columns)
                           emit_axis_reduce, emit_short_rows, emit_narrow_cols
  + an optional reduction tail on flat/nd: per-thread accumulators, wave64
    shuffle tree, LDS across the 4 waves, one partial per block, and a
    one-block finalize kernel (no atomics, deterministic).
Vector accesses use 16-byte types at element alignment where 16-byte alignment is
missing; `log`, `erf`, `exp` come from `mathlib` (float64) and `mathlib32` (float32).
"""
import numpy as np

from . import mathlib, mathlib32

BLOCK = 256          # threads per block: 4 wave64
WAVE = 64
N_XCD = 8            # accelerator dies with private L2 on MI355X

# storage / arithmetic C type per dtype code
CTYPE = {
    "f4": "float",
    "f8": "double",
    "i4": "int",
    "i8": "long long",
    "u4": "unsigned int",
    "u1": "unsigned char",
    "b1": "unsigned char",
}
ITEMSIZE = {"f4": 4, "f8": 8, "i4": 4, "i8": 8, "u4": 4, "u1": 1, "b1": 1}
# 16-byte vector type per dtype code (bytes only in flat kernels: masks and their users)
VEC16 = {"f4": ("f4x4", 4), "f8": ("f8x2", 2), "i4": ("i4x4", 4), "i8": ("i8x2", 2),
         "u4": ("u4x4", 4), "u1": ("u1x16", 16), "b1": ("u1x16", 16)}

PREAMBLE = """\
typedef float f4x4 __attribute__((ext_vector_type(4)));
typedef double f8x2 __attribute__((ext_vector_type(2)));
typedef int i4x4 __attribute__((ext_vector_type(4)));
typedef long long i8x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u4x4 __attribute__((ext_vector_type(4)));
typedef float f4x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef double f8x2u __attribute__((ext_vector_type(2), aligned(8)));
typedef int i4x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef long long i8x2u __attribute__((ext_vector_type(2), aligned(8)));
typedef unsigned int u4x4u __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned char u1x16 __attribute__((ext_vector_type(16)));
typedef unsigned char u1x16u __attribute__((ext_vector_type(16), aligned(1)));
typedef float f4x2 __attribute__((ext_vector_type(2)));
typedef int i4x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u4x2 __attribute__((ext_vector_type(2)));
typedef unsigned char u1x2 __attribute__((ext_vector_type(2)));
typedef unsigned char u1x4 __attribute__((ext_vector_type(4)));
typedef unsigned char u1x8 __attribute__((ext_vector_type(8)));
typedef float f4x2u __attribute__((ext_vector_type(2), aligned(4)));
typedef int i4x2u __attribute__((ext_vector_type(2), aligned(4)));
typedef unsigned int u4x2u __attribute__((ext_vector_type(2), aligned(4)));
typedef unsigned char u1x2u __attribute__((ext_vector_type(2), aligned(1)));
typedef unsigned char u1x4u __attribute__((ext_vector_type(4), aligned(1)));
typedef unsigned char u1x8u __attribute__((ext_vector_type(8), aligned(1)));
// between accesses of one wave's lanes to the wave's own LDS: the hardware keeps them in order
#define DR_WAVE_SYNC() do { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); \
    __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront"); } while (0)
"""


def flat_vec(dt, E):
    """(vector type, elements per vector, vectors per thread) a flat kernel uses for a
    stream of type `dt` when a thread handles E elements per step: the whole 16-byte
    vector, several of them (only when E exceeds it), or a shorter vector of E elements,
    so that the lanes of a wave always read one contiguous stretch."""
    vt, per = VEC16[dt]
    if E >= per:
        return vt, per, E // per
    return f"{vt.split('x')[0]}x{E}", E, 1
# The `...u` types are the same vectors at element alignment: global memory takes 16-byte
# accesses at any 4-byte address (measured on MI355X: 6.2-6.6 TB/s for a copy shifted by one
# to three floats against 6.7 TB/s aligned, and 3.5 TB/s with one element per lane), so
# views that do not start on a 16-byte boundary, or whose rows do not, still move vectors.


def dtype_code(dtype):
    dtype = np.dtype(dtype)
    if dtype.kind == "b":
        return "b1"
    code = dtype.kind + str(dtype.itemsize)
    if code not in CTYPE:
        raise NotImplementedError(f"dtype {dtype} has no device representation")
    return code


def code_dtype(code):
    return np.dtype({"b1": "bool"}.get(code, code))


# ---- per-operation C expressions -------------------------------------------

_FLOAT_FUNCS1 = {
    "sin": "sin", "cos": "cos", "tan": "tan", "arcsin": "asin", "arccos": "acos",
    "arctan": "atan", "sinh": "sinh", "cosh": "cosh", "tanh": "tanh", "exp": "exp",
    "exp2": "exp2", "expm1": "expm1", "log": "log", "log2": "log2", "log10": "log10",
    "log1p": "log1p", "sqrt": "sqrt", "cbrt": "cbrt", "erf": "erf", "erfc": "erfc",
    "floor": "floor", "ceil": "ceil", "trunc": "trunc", "rint": "rint",
}
_FLOAT_FUNCS2 = {
    "power": "pow", "arctan2": "atan2", "hypot": "hypot", "copysign": "copysign",
    "fmod": "fmod", "fmax": "fmax", "fmin": "fmin",
}
# functions whose results carry a rounding error of their own (about an ulp)
_INEXACT = frozenset(("sin", "cos", "tan", "arcsin", "arccos", "arctan", "sinh", "cosh", "tanh", "exp",
                      "exp2", "expm1", "log", "log2", "log10", "log1p", "cbrt", "erf", "erfc", "power",
                      "arctan2", "hypot"))
_INFIX = {"add": "+", "subtract": "-", "multiply": "*", "divide": "/", "true_divide": "/"}
_COMPARE = {"greater": ">", "less": "<", "greater_equal": ">=", "less_equal": "<=",
            "equal": "==", "not_equal": "!="}

# arithmetic ufuncs whose bool loop is a logical operation (None: NumPy raises TypeError)
_BOOL_ARITH = {"add": "|", "maximum": "|", "fmax": "|", "multiply": "&", "minimum": "&",
               "fmin": "&", "subtract": None, "negative": None}

# results are bool; arithmetic happens in the operands' common type
_PREDICATES = {"isnan", "isinf", "isfinite", "logical_not", "logical_and", "logical_or",
               "logical_xor"}

# integer and bool operands only (NumPy has no loop for floats: the type probe raises its
# TypeError); on bool they are the logical operations
_BITWISE = {"bitwise_and": "&", "bitwise_or": "|", "bitwise_xor": "^"}
_SHIFTS = {"left_shift": "<<", "right_shift": ">>"}

SUPPORTED_UFUNCS = (set(_FLOAT_FUNCS1) | set(_FLOAT_FUNCS2) | set(_INFIX) | set(_COMPARE)
                    | _PREDICATES | set(_BITWISE) | set(_SHIFTS) | {"invert"}
                    | {"floor_divide", "remainder"}
                    | {"negative", "positive", "absolute", "fabs", "reciprocal", "maximum",
                       "minimum", "square", "sign"})


def _fn(name, dt):
    """C math function for a float dtype: `sinf` for f4, `sin` for f8."""
    return name + ("f" if dt == "f4" else "")


def _divmod_expr(name, dt, args):
    """`//` and `%` as NumPy computes them (numpy/_core/src/npymath/npy_math_internal.h.src,
    `npy_divmod`; loops.c.src for the integer rules): the quotient is floored, the
    remainder takes the divisor's sign; floats go through an exact `fmod`, the quotient
    is snapped to the nearest integer, zeros keep the sign NumPy gives them, a zero
    divisor gives a / b (quotient) and NaN (remainder); integer division by zero gives 0,
    and the most negative integer divided by -1 stays itself (remainder 0)."""
    ct = CTYPE[dt]
    a, b = args
    want_div = name == "floor_divide"
    if dt in ("f4", "f8"):
        fmod, floor, copysign = _fn("fmod", dt), _fn("floor", dt), _fn("copysign", dt)
        body = (f"const {ct} a_ = {a}, b_ = {b}; {ct} m_ = {fmod}(a_, b_); {ct} d_; "
                f"if (b_ == 0) {{ d_ = a_ / b_; }} else {{ "
                f"d_ = (a_ - m_) / b_; "
                f"if (m_ != 0) {{ if ((b_ < 0) != (m_ < 0)) {{ m_ += b_; d_ -= ({ct})1; }} }} "
                f"else {{ m_ = {copysign}(({ct})0, b_); }} "
                f"if (d_ != 0) {{ {ct} f_ = {floor}(d_); if (d_ - f_ > ({ct})0.5) f_ += ({ct})1; d_ = f_; }} "
                f"else {{ d_ = {copysign}(({ct})0, a_ / b_); }} }} ")
        return "({ " + body + ("d_" if want_div else "m_") + "; })"
    if dt == "b1":
        raise TypeError(f"ufunc {name!r} is not fused for boolean operands")
    if dt[0] == "u":
        op = "/" if want_div else "%"
        return f"({b} == 0 ? ({ct})0 : ({ct})({a} {op} {b}))"
    lowest = {"i4": "(-2147483647 - 1)", "i8": "(-9223372036854775807LL - 1)"}[dt]
    if want_div:
        return ("({ " + f"const {ct} a_ = {a}, b_ = {b}; {ct} q_; "
                f"if (b_ == 0) q_ = 0; else if (a_ == {lowest} && b_ == -1) q_ = a_; "
                f"else {{ q_ = a_ / b_; if (((a_ > 0) != (b_ > 0)) && q_ * b_ != a_) --q_; }} q_; " + "})")
    return ("({ " + f"const {ct} a_ = {a}, b_ = {b}; {ct} r_; "
            f"if (b_ == 0 || (a_ == {lowest} && b_ == -1)) r_ = 0; "
            f"else {{ r_ = a_ % b_; if (r_ != 0 && ((a_ > 0) != (b_ > 0))) r_ += b_; }} r_; " + "})")


def op_expr(name, dt, args):
    """C expression computing ufunc `name` in arithmetic type `dt` on `args`
    (C expressions already converted to `dt`)."""
    is_float = dt in ("f4", "f8")
    if dt == "b1" and name in _BOOL_ARITH:
        # NumPy's bool arithmetic is logical: True + True is True (a byte value of 2
        # in a bool array would break later comparisons); subtraction does not exist
        op = _BOOL_ARITH[name]
        if op is None:
            raise TypeError(f"numpy boolean {name} is not supported, as in NumPy "
                            "(use bitwise or logical operations instead)")
        return f"(unsigned char)({args[0]} {op} {args[1]})"
    if name in _BITWISE:
        if is_float:
            raise TypeError(f"ufunc {name!r} not supported for float operands")
        return f"({CTYPE[dt]})({args[0]} {_BITWISE[name]} {args[1]})"
    if name == "invert":
        if is_float:
            raise TypeError("ufunc 'invert' not supported for float operands")
        return f"(unsigned char)({args[0]} == 0)" if dt == "b1" else f"({CTYPE[dt]})(~{args[0]})"
    if name in _SHIFTS:
        if is_float or dt == "b1":
            raise TypeError(f"ufunc {name!r} not supported for these operands")
        # counts of the type's width or more shift everything out, as in NumPy (the
        # hardware would use the count modulo the width)
        bits = 8 * ITEMSIZE[dt]
        a, b = args
        uns = "unsigned " + CTYPE[dt] if dt[0] == "i" else CTYPE[dt]
        if name == "left_shift":
            return f"(({uns}){b} >= {bits} ? ({CTYPE[dt]})0 : ({CTYPE[dt]})(({uns}){a} << {b}))"
        fill = f"({CTYPE[dt]})({a} < 0 ? -1 : 0)" if dt[0] == "i" else f"({CTYPE[dt]})0"
        return f"(({uns}){b} >= {bits} ? {fill} : ({CTYPE[dt]})({a} >> {b}))"
    if name in ("floor_divide", "remainder"):
        return _divmod_expr(name, dt, args)
    if name in _INFIX:
        if name in ("divide", "true_divide") and not is_float:
            raise NotImplementedError("integer division has no float result type here")
        return f"{args[0]} {_INFIX[name]} {args[1]}"
    if name in _COMPARE:
        return f"(unsigned char)({args[0]} {_COMPARE[name]} {args[1]})"
    if name == "isnan":
        return f"(unsigned char)({args[0]} != {args[0]})"
    if name == "isinf":
        return (f"(unsigned char)({_fn('fabs', dt)}({args[0]}) == __builtin_inf{'f' if dt == 'f4' else ''}())"
                if is_float else "(unsigned char)0")
    if name == "isfinite":
        return (f"(unsigned char)({_fn('fabs', dt)}({args[0]}) < __builtin_inf{'f' if dt == 'f4' else ''}())"
                if is_float else "(unsigned char)1")
    if name == "logical_not":
        return f"(unsigned char)({args[0]} == 0)"
    if name == "logical_and":
        return f"(unsigned char)(({args[0]} != 0) && ({args[1]} != 0))"
    if name == "logical_or":
        return f"(unsigned char)(({args[0]} != 0) || ({args[1]} != 0))"
    if name == "logical_xor":
        return f"(unsigned char)(({args[0]} != 0) != ({args[1]} != 0))"
    if name == "sign":      # NaN stays NaN, as in NumPy
        a = args[0]
        body = f"({CTYPE[dt]})(({a} > 0) - ({a} < 0))"
        return f"(({a} != {a}) ? {a} : {body})" if is_float else body
    if name == "negative":
        return f"-{args[0]}"
    if name == "positive":
        return f"{args[0]}"
    if name in ("absolute", "fabs"):
        if is_float:
            return f"{_fn('fabs', dt)}({args[0]})"
        return f"({args[0]} < 0 ? -{args[0]} : {args[0]})"
    if name == "reciprocal":
        return f"({CTYPE[dt]})1 / {args[0]}"
    if name == "maximum":   # NaN-propagating, like NumPy
        a, b = args
        return f"(({a} >= {b} || {a} != {a}) ? {a} : {b})"
    if name == "minimum":
        a, b = args
        return f"(({a} <= {b} || {a} != {a}) ? {a} : {b})"
    if name in _FLOAT_FUNCS1:
        if not is_float:
            raise NotImplementedError(f"{name} on a non-float type")
        return f"{_fn(_FLOAT_FUNCS1[name], dt)}({args[0]})"
    if name in _FLOAT_FUNCS2:
        if not is_float:
            raise NotImplementedError(f"{name} on a non-float type")
        return f"{_fn(_FLOAT_FUNCS2[name], dt)}({args[0]}, {args[1]})"
    raise NotImplementedError(f"ufunc {name!r} cannot be fused")


# operations computed from the element index instead of from operands
INDEX_OPS = ("iota", "philox_raw", "philox_f8", "philox_f4")

# Philox-4x64-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11),
# the counter-based generator behind numpy.random.Philox.  Output r of the stream that
# starts at the 256-bit counter (c0..c3) is word r % 4 of the block computed from
# counter + r / 4 with the 128-bit key (k0, k1): ten rounds of two 64x64->128-bit
# multiplications, the key bumped by the Weyl constants between rounds.
PHILOX = """\
typedef unsigned long long dr_u64;
static __device__ __forceinline__ dr_u64 dr_mulhi64(dr_u64 a, dr_u64 b)
{
    return (dr_u64)(((unsigned __int128)a * b) >> 64);
}
/* the four outputs of block `blk` of the stream */
static __device__ __forceinline__ void dr_philox_block(dr_u64 k0, dr_u64 k1, dr_u64 c0, dr_u64 c1,
                                                       dr_u64 c2, dr_u64 c3, dr_u64 blk,
                                                       dr_u64 (&x)[4])
{
    x[0] = c0 + blk;                      /* 256-bit counter + block number */
    dr_u64 carry = x[0] < blk;
    x[1] = c1 + carry;
    carry = x[1] < carry;
    x[2] = c2 + carry;
    carry = x[2] < carry;
    x[3] = c3 + carry;
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        /* one 128-bit product gives both halves (asked for separately, the low half is
           multiplied out a second time) */
        const unsigned __int128 p0 = (unsigned __int128)0xD2E7470EE14C6C93ULL * x[0];
        const unsigned __int128 p1 = (unsigned __int128)0xCA5A826395121157ULL * x[2];
        const dr_u64 hi0 = (dr_u64)(p0 >> 64), lo0 = (dr_u64)p0;
        const dr_u64 hi1 = (dr_u64)(p1 >> 64), lo1 = (dr_u64)p1;
        x[0] = hi1 ^ x[1] ^ k0;
        x[2] = hi0 ^ x[3] ^ k1;
        x[1] = lo1;
        x[3] = lo0;
        k0 += 0x9E3779B97F4A7C15ULL;
        k1 += 0xBB67AE8584CAA73BULL;
    }
}
/* output r of the stream */
static __device__ __forceinline__ dr_u64 dr_philox(dr_u64 k0, dr_u64 k1, dr_u64 c0, dr_u64 c1,
                                                  dr_u64 c2, dr_u64 c3, dr_u64 r)
{
    dr_u64 x[4];
    dr_philox_block(k0, k1, c0, c1, c2, c3, r >> 2, x);
    const int lane = (int)(r & 3);
    return lane == 0 ? x[0] : lane == 1 ? x[1] : lane == 2 ? x[2] : x[3];
}
"""


def _philox_value(name, raw):
    """int64 bits, or a double in [0, 1) from the top 53 bits (what
    numpy.random.Generator.random makes of a raw output)."""
    return f"(long long){raw}" if name == "philox_raw" else f"(double)({raw} >> 11) * 0x1p-53"


def _philox_float(raw, half):
    """A float in [0, 1) from the top 24 bits of one half of a raw output: what
    numpy.random.Generator.random(dtype=float32) makes of it (a 64-bit output serves two
    numbers, its low half first)."""
    return f"(float)((unsigned int)({raw} >> (32 * ({half}))) >> 8) * 0x1p-24f"


def flat_elements(prog, leaf_class, out_dtypes, reduce_op):
    """Elements one thread handles per vector step of the flat kernel: a 16-byte vector of
    the widest streamed type (narrower streams move shorter vectors, see `flat_vec`: with
    several vectors of the wider type per lane a wave's load would touch every cache line
    of its stretch once per vector: float32 x float64 68 % of the HBM peak, a mask beside
    two float32 operands 31 %); four when the program draws Philox numbers, whose blocks
    hold four outputs (a thread then makes each block once)."""
    widths = [ITEMSIZE[dt] for dt, c in zip(prog.leaves, leaf_class) if c != "b"]
    if not reduce_op:
        widths += [ITEMSIZE[dt] for dt in out_dtypes]
    draws = {name for name, _, _, _ in prog.ops if name.startswith("philox")}
    if draws:       # a block of four outputs: four 64-bit numbers or eight floats
        widths.append(2 if "philox_f4" in draws else 4)
        return 16 // min(widths)
    return 16 // max(widths) if widths else 4


class Program:
    """Straight-line SSA form of an expression DAG.

    leaves   list of dtype codes, one per distinct input array
    scalars  list of dtype codes, one per scalar kernel parameter
    ops      list of (name, compute dtype, result dtype, arg refs); a ref is
             ('l', i) | ('s', i) | ('v', i); name 'cast' converts
    roots    list of (ref, dtype code)
    """

    __slots__ = ("leaves", "scalars", "ops", "roots", "own_math", "own_math32", "uses_index",
                 "soft_div")

    def __init__(self, leaves, scalars, ops, roots, own_math=True, own_math32=True, soft_div=True):
        self.leaves = tuple(leaves)
        self.scalars = tuple(scalars)
        self.ops = tuple(ops)
        self.roots = tuple(roots)
        # float64 functions taken from `mathlib` instead of the device library
        self.own_math = tuple(sorted({name for name, cdt, _, _ in self.ops
                                      if cdt == "f8" and name in mathlib.FUNCTIONS})) \
            if own_math else ()
        # float32 functions taken from `mathlib32`
        self.own_math32 = tuple(sorted({name for name, cdt, _, _ in self.ops
                                        if cdt == "f4" and name in mathlib32.FUNCTIONS})) \
            if own_math32 else ()
        # these operations read the element index: only the flat kernel supplies it
        self.uses_index = any(name in INDEX_OPS for name, _, _, _ in self.ops)
        # soft_div: 1 float64 only, 2 float32 as well.  The float32 forms are used by bodies
        # that evaluate packs of elements (one test for the rare cases per pack: element by
        # element the test costs more than the short forms save)
        self.soft_div = self._quotients_nobody_sees(("f8",) * bool(own_math)
                                                    + ("f4",) * bool(own_math32 and soft_div == 2)) \
            if soft_div else ()

    def _quotients_nobody_sees(self, types):
        """Divisions (in the float types `types`) and float64 square roots whose result
        reaches a root only through functions that round on their own (`log(S / K)`,
        `erf(d / (s * sqrt(t)))`): their last bit cannot be seen in any
        result beyond what those functions' own error already hides, so they may be
        computed to within one ulp instead of correctly rounded (`mathlib.DIV_F8`,
        `dr_sqrt_near_f8`, `mathlib32.DIV_F4`).  A
        quotient that a root can see through exact operations alone (+ - * /, sqrt, the
        selections, the reductions) stays the correctly rounded one: expressions of those
        remain equal to NumPy's to the bit."""
        seen = [False] * len(self.ops)      # visible at a root through exact operations only
        for (kind, j), _ in self.roots:
            if kind == "v":
                seen[j] = True
        for i in range(len(self.ops) - 1, -1, -1):
            name = self.ops[i][0]
            if seen[i] and name not in _INEXACT:
                for kind, j in self.ops[i][3]:
                    if kind == "v":
                        seen[j] = True
        return tuple(i for i, (name, cdt, _, _) in enumerate(self.ops)
                     if not seen[i] and cdt in types
                     and (name in ("divide", "true_divide")
                          or (name == "sqrt" and (cdt == "f4" or "sqrt" in self.own_math))))

    def key(self):
        return (self.leaves, self.scalars, self.ops, self.roots, self.own_math, self.own_math32,
                self.soft_div)

    def ref_dtype(self, ref):
        kind, i = ref
        if kind == "l":
            return self.leaves[i]
        if kind == "s":
            return self.scalars[i]
        return self.ops[i][2]


def _conv(expr, src, dst):
    if src == dst:
        return expr
    if dst == "b1":
        return f"(unsigned char)({expr} != 0)"
    return f"({CTYPE[dst]}){expr}"


def _op_statement(prog, i):
    """`const T v<i> = ...;` for operation i of `prog`, one element at a time."""
    name, cdt, rdt, args = prog.ops[i]
    cargs = [_conv(f"{k}{j}", prog.ref_dtype((k, j)), cdt) for k, j in args]
    if name == "cast":
        expr = cargs[0]
    elif name == "iota":
        expr = f"({CTYPE[cdt]})dr_i"
    elif name in ("philox_raw", "philox_f8"):
        # operands: key (2 words), counter (4 words), position of element 0 in the stream
        # (a seventh operand, when the draw starts inside a block: that offset)
        words = ", ".join(f"(dr_u64){k}{j}" for k, j in args[:6])
        pos = f"(dr_u64){args[6][0]}{args[6][1]} + " if len(args) > 6 else ""
        expr = _philox_value(name, f"dr_philox({words}, {pos}(dr_u64)dr_i)")
    elif name == "philox_f4":
        # the same operands, the position counted in halves of outputs
        words = ", ".join(f"(dr_u64){k}{j}" for k, j in args[:6])
        pos = f"(dr_u64){args[6][0]}{args[6][1]} + " if len(args) > 6 else ""
        at = f"({pos}(dr_u64)dr_i)"
        expr = _philox_float(f"dr_philox({words}, {at} >> 1)", f"(int)({at} & 1)")
    elif cdt == "f8" and name == "sqrt" and i in prog.soft_div:
        expr = f"dr_sqrt_near_f8_1({cargs[0]})"
    elif cdt == "f8" and name in prog.own_math:
        expr = f"{mathlib.FUNCTIONS[name][0]}_1({cargs[0]})"
    elif cdt == "f4" and name in prog.own_math32:
        expr = f"{mathlib32.FUNCTIONS[name][0]}({cargs[0]})"
    elif i in prog.soft_div and cdt == "f8":
        expr = f"dr_div_f8_1({cargs[0]}, {cargs[1]})"
    elif name == "where":    # the condition keeps its own type
        k, j = args[0]
        expr = f"(({k}{j} != 0) ? {cargs[1]} : {cargs[2]})"
    else:
        expr = op_expr(name, cdt, cargs)
    return f"    const {CTYPE[rdt]} v{i} = {expr};"


def emit_body(prog, out_dtypes, fname="dr_body", with_math=True, lds_tables=0, stage_loop=False):
    """Inline device function evaluating the whole program for one element.

    Parameters: leaf values, scalar values, then one reference per root."""
    params = ["const long long dr_i"] if prog.uses_index else []
    params += [f"const {CTYPE[dt]} l{i}" for i, dt in enumerate(prog.leaves)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += [f"{CTYPE[dt]}& r{i}" for i, dt in enumerate(out_dtypes)]
    uses_philox = any(name.startswith("philox") for name, _, _, _ in prog.ops)
    soft8 = any(prog.ops[i][1] == "f8" and prog.ops[i][0] != "sqrt" for i in prog.soft_div)
    soft4 = any(prog.ops[i][1] == "f4" for i in prog.soft_div)
    lines = [mathlib.source(prog.own_math, lds=lds_tables, stage_loop=stage_loop,
                            soft_div=soft8) if with_math else "",
             mathlib32.source(prog.own_math32, soft_div=soft4) if with_math else "",
             PHILOX if uses_philox and with_math else "",
             f"__device__ __forceinline__ void {fname}({', '.join(params)})", "{"]
    for i in range(len(prog.ops)):
        lines.append(_op_statement(prog, i))
    for i, ((k, j), rdt) in enumerate(prog.roots):
        lines.append(f"    r{i} = {_conv(f'{k}{j}', rdt, out_dtypes[i])};")
    lines.append("}")
    return "\n".join(lines)


def emit_body_packed(prog, out_dtypes, leaf_is_array, pack, fname="dr_body_pack", group=1):
    """The same program on a pack of `pack` elements held by one thread: every value
    is a small array and every operation a fully unrolled loop over it, so that the
    elements pass through each float64 `log`/`erf`/`exp` in lock step (see `mathlib`).
    Leaves flagged False in `leaf_is_array` are one value for the whole pack (broadcast
    operands).  The pack is made of groups of `group` consecutive elements; programs
    that read the element index get the index of each group's first element in `dr_g`
    (a multiple of `group`).  The arithmetic per element is exactly that of
    `emit_body`."""
    P = pack
    loop = f'_Pragma("unroll") for (int e = 0; e < {P}; ++e)'
    index = f"(dr_g[e / {group}] + e % {group})"

    def ref(k, j):
        if k == "s" or (k == "l" and not leaf_is_array[j]):
            return f"{k}{j}"
        return f"{k}{j}[e]"

    params = [f"const long long (&dr_g)[{P // group}]"] if prog.uses_index else []
    params += [f"const {CTYPE[dt]} (&l{i})[{P}]" if leaf_is_array[i] else f"const {CTYPE[dt]} l{i}"
               for i, dt in enumerate(prog.leaves)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += [f"{CTYPE[dt]} (&r{i})[{P}]" for i, dt in enumerate(out_dtypes)]
    lines = [f"__device__ __forceinline__ void {fname}({', '.join(params)})", "{"]
    for i, (name, cdt, rdt, args) in enumerate(prog.ops):
        cargs = [_conv(ref(k, j), prog.ref_dtype((k, j)), cdt) for k, j in args]
        lines.append(f"    {CTYPE[rdt]} v{i}[{P}];")
        if name == "iota":
            lines.append(f"    {loop} v{i}[e] = ({CTYPE[cdt]}){index};")
            continue
        if name in ("philox_raw", "philox_f8", "philox_f4"):
            words = ", ".join(f"(dr_u64){k}{j}" for k, j in args[:6])
            per = 8 if name == "philox_f4" else 4       # numbers that one block serves
            if len(args) == 6 and group % per == 0:
                # the draw starts on a block and a group is consecutive elements from a
                # multiple of a block's numbers: every block is made once
                for g in range(P // group):
                    for b in range(group // per):
                        at = group * g + per * b
                        if name == "philox_f4":
                            vals = " ".join(f"v{i}[{at + 2 * w + h}] = {_philox_float(f'x_[{w}]', h)};"
                                            for w in range(4) for h in range(2))
                        else:
                            vals = " ".join(f"v{i}[{at + w}] = {_philox_value(name, f'x_[{w}]')};"
                                            for w in range(4))
                        blk = f"((dr_u64)dr_g[{g}] >> {per.bit_length() - 1}) + {b}"
                        lines.append(f"    {{ dr_u64 x_[4]; dr_philox_block({words}, {blk}, x_); {vals} }}")
            else:
                pos = f"(dr_u64){args[6][0]}{args[6][1]} + " if len(args) > 6 else ""
                at = f"({pos}(dr_u64){index})"
                if name == "philox_f4":
                    value = _philox_float(f"dr_philox({words}, {at} >> 1)", f"(int)({at} & 1)")
                else:
                    value = _philox_value(name, f"dr_philox({words}, {at})")
                lines.append(f"    {loop} v{i}[e] = {value};")
            continue
        if cdt == "f8" and name in prog.own_math:
            k, j = args[0]
            fn = "dr_sqrt_near_f8" if name == "sqrt" and i in prog.soft_div else mathlib.FUNCTIONS[name][0]
            if prog.ref_dtype((k, j)) == "f8" and ref(k, j).endswith("[e]"):
                lines.append(f"    {fn}<{P}>({k}{j}, v{i});")
            else:       # converted or broadcast argument: gather it first
                lines.append(f"    {{ double t_[{P}]; {loop} t_[e] = {cargs[0]}; "
                             f"{fn}<{P}>(t_, v{i}); }}")
            continue
        if i in prog.soft_div and name == "sqrt":       # float32 (float64 went above)
            k, j = args[0]
            if prog.ref_dtype((k, j)) == "f4" and ref(k, j).endswith("[e]"):
                lines.append(f"    dr_sqrt_near_f4_pack<{P}>({k}{j}, v{i});")
            else:
                lines.append(f"    {{ float t_[{P}]; {loop} t_[e] = {cargs[0]}; "
                             f"dr_sqrt_near_f4_pack<{P}>(t_, v{i}); }}")
            continue
        if i in prog.soft_div:
            gather = []
            names = []
            for pos, (k, j) in enumerate(args):
                if prog.ref_dtype((k, j)) == cdt and ref(k, j).endswith("[e]"):
                    names.append(f"{k}{j}")
                else:       # converted or broadcast operand: gather it first
                    gather.append(f"{CTYPE[cdt]} q{pos}_[{P}]; {loop} q{pos}_[e] = {cargs[pos]};")
                    names.append(f"q{pos}_")
            fn = "dr_div_f8" if cdt == "f8" else "dr_div_f4_pack"
            lines.append(f"    {{ {' '.join(gather)} {fn}<{P}>({names[0]}, {names[1]}, v{i}); }}")
            continue
        if name == "cast":
            expr = cargs[0]
        elif name == "where":    # the condition keeps its own type
            expr = f"(({ref(*args[0])} != 0) ? {cargs[1]} : {cargs[2]})"
        elif cdt == "f4" and name in prog.own_math32:
            expr = f"{mathlib32.FUNCTIONS[name][0]}({cargs[0]})"
        else:
            expr = op_expr(name, cdt, cargs)
        lines.append(f"    {loop} v{i}[e] = {expr};")
    for i, ((k, j), rdt) in enumerate(prog.roots):
        lines.append(f"    {loop} r{i}[e] = {_conv(ref(k, j), rdt, out_dtypes[i])};")
    lines.append("}")
    return "\n".join(lines)


# ---- reduction pieces ------------------------------------------------------

def _combine(op, a, b):
    if op == "add":
        return f"{a} + {b}"
    return op_expr(op, "f8", [a, b])  # maximum/minimum expression is type-agnostic


def _identity(op, dt):
    if op == "add":
        return f"({CTYPE[dt]})0"
    if dt in ("f4", "f8"):
        inf = "__builtin_inff()" if dt == "f4" else "__builtin_inf()"
        return f"-{inf}" if op == "maximum" else inf
    lim = {"i4": ("(-2147483647 - 1)", "2147483647"),
           "i8": ("(-9223372036854775807LL - 1)", "9223372036854775807LL"),
           "u4": ("0u", "4294967295u"), "u1": ("0", "255"), "b1": ("0", "1")}[dt]
    return lim[0] if op == "maximum" else lim[1]


def emit_block_reduce(op, dt):
    """Device function: combine `v` over the block; valid in thread 0.

    Wave64 shuffle-down tree, then the 4 wave leaders meet through LDS."""
    ct = CTYPE[dt]
    shfl = "__shfl_down(v, off, 64)"
    if dt in ("u1", "b1"):
        shfl = f"({ct})__shfl_down((int)v, off, 64)"
    return f"""\
__device__ __forceinline__ {ct} dr_block_reduce({ct} v)
{{
    __shared__ {ct} dr_wave_part[{BLOCK // WAVE}];
#pragma unroll
    for (int off = {WAVE // 2}; off > 0; off >>= 1) {{
        const {ct} o = {shfl};
        v = {_combine(op, 'v', 'o')};
    }}
    const int lane = threadIdx.x & {WAVE - 1};
    const int wave = threadIdx.x >> 6;
    if (lane == 0) dr_wave_part[wave] = v;
    __syncthreads();
    if (threadIdx.x == 0) {{
        v = dr_wave_part[0];
#pragma unroll
        for (int w = 1; w < {BLOCK // WAVE}; ++w) v = {_combine(op, 'v', 'dr_wave_part[w]')};
    }}
    return v;
}}
"""


def emit_finalize(op, dt):
    ct = CTYPE[dt]
    return f"""\
extern "C" __global__ __launch_bounds__({BLOCK})
void dr_finalize(const {ct}* __restrict__ partial, {ct}* __restrict__ out, int count)
{{
    {ct} acc = {_identity(op, dt)};
    for (int i = threadIdx.x; i < count; i += {BLOCK}) acc = {_combine(op, 'acc', 'partial[i]')};
    acc = dr_block_reduce(acc);
    if (threadIdx.x == 0) out[0] = acc;
}}
"""


# ---- flat kernel -----------------------------------------------------------

def _ld(nt, ptr):
    return f"__builtin_nontemporal_load({ptr})" if nt else f"*({ptr})"


def _st(nt, val, ptr):
    return f"__builtin_nontemporal_store({val}, {ptr});" if nt else f"*({ptr}) = {val};"


def packs(prog, vec):
    """Whether the flat kernel evaluates this program on packs of elements: programs
    that use the float64 functions of `mathlib` or draw Philox numbers, in vector
    kernels."""
    return bool(vec and (prog.own_math or any(name.startswith("philox") for name, _, _, _ in prog.ops)
                         or any(prog.ops[i][1] == "f4" for i in prog.soft_div)))


def emit_flat(prog, leaf_class, out_dtypes, vec, unroll, nt_load, nt_store, restrict=True,
              reduce_op=None, unaligned=False, one_run=False, stage_loop=False, exchange=True,
              guard=False, runs=1):
    """Contiguous 1-D kernel.

    leaf_class  per leaf 'c' (contiguous, same length as the output), 'b' (single
                element broadcast to every position) or 's2' .. 's8' (every k-th element
                of a contiguous stretch: a thread loads the k vectors that hold its
                elements and picks them out of the registers; the lines in between
                are fetched whichever way the elements are read)
    vec         True: 16-byte vector accesses (all element types 4 or 8 bytes wide);
                False: one element per access
    unaligned   some pointer is not 16-byte aligned: vectors at element alignment
    reduce_op   None, or 'add' | 'maximum' | 'minimum': the single root is
                reduced instead of stored; the output is one partial per block
    one_run     block c handles run c and nothing else (the grid must have at least
                n / elements per run blocks); without the loop over runs the compiler
                needs fewer registers, and the block asks for its operands before it
                copies the functions' tables into LDS, so one wait covers both
    runs        with `one_run`: a block handles this many adjacent runs one after the other
                (straight-line code, no loop) and copies the tables once for all of them
    guard       the last vector of a strided operand would reach past its buffer's end:
                the last few elements are left to the element-wise tail
    exchange    outputs of which a lane holds several adjacent vectors (random numbers:
                four doubles per lane) change lanes through LDS before they are stored
    """
    rs = "__restrict__ " if restrict else ""
    ua = "u" if unaligned else ""

    def step_of(c):
        return int(c[1:]) if c[0] == "s" else 1

    def element(i, dt, c, e, tag):
        """Element e of leaf i among the values a thread has loaded for one step."""
        per, K = flat_vec(dt, E)[1], step_of(c)
        if K > 1 and K >= per:
            return f"L{i}_{e}{tag}"
        return f"L{i}_{e * K // per}{tag}[{e * K % per}]"
    n_leaf, n_out = len(prog.leaves), len(out_dtypes)
    red_dt = out_dtypes[0] if reduce_op else None
    E = flat_elements(prog, leaf_class, out_dtypes, reduce_op) if vec else 1
    src = [PREAMBLE, emit_body(prog, out_dtypes, lds_tables=BLOCK, stage_loop=stage_loop)]
    packed = packs(prog, vec)
    if packed:
        src.append(emit_body_packed(prog, out_dtypes, [c != "b" for c in leaf_class], E * unroll,
                                    group=E))
    if reduce_op:
        src.append(emit_block_reduce(reduce_op, red_dt))
        src.append(emit_finalize(reduce_op, red_dt))

    params = [f"const {CTYPE[dt]}* {rs}a{i}" for i, dt in enumerate(prog.leaves)]
    if reduce_op:
        params.append(f"{CTYPE[red_dt]}* {rs}partial")
    else:
        params += [f"{CTYPE[dt]}* {rs}o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long n")

    L = []
    L.append(f'extern "C" __global__ __launch_bounds__({BLOCK})')
    L.append(f"void dr_kernel({', '.join(params)})")
    L.append("{")
    staged = bool(mathlib.tables(prog.own_math))
    xch = sorted({(ITEMSIZE[dt],) + flat_vec(dt, E)[::2] for dt in out_dtypes
                  if flat_vec(dt, E)[2] > 1}) if packed and exchange and not reduce_op else []
    for size, vt, chunks in xch:
        L.append(f"    __shared__ {vt} dr_xch{size}[{BLOCK * chunks}];")
    if xch:
        L.append(f"    const int dr_lane = threadIdx.x & {WAVE - 1};")
    exchange = bool(xch)
    if staged and not one_run:
        L.append("    DR_STAGE_TABLES();      // the functions' tables, from memory into LDS")
    for i, c in enumerate(leaf_class):
        if c == "b":
            L.append(f"    const {CTYPE[prog.leaves[i]]} b{i} = a{i}[0];")
    if reduce_op:
        for e in range(max(E, 1)):
            L.append(f"    {CTYPE[red_dt]} acc{e} = {_identity(reduce_op, red_dt)};")
    scal = [f"s{i}" for i in range(len(prog.scalars))]

    def step(tag, idx, indent):
        """Code handling one vector (or element) at index expression `idx`:
        (loads, compute+stores)."""
        pad = " " * indent
        loads, work = [], []
        for i, (dt, c) in enumerate(zip(prog.leaves, leaf_class)):
            if c == "b":
                continue
            K = step_of(c)
            if vec and K > 1 and K >= flat_vec(dt, E)[1]:
                # no vector would hold two of the thread's elements: element loads
                for e in range(E):
                    loads.append(f"{pad}const {CTYPE[dt]} L{i}_{e}{tag} = "
                                 f"{_ld(nt_load, f'a{i} + (({idx}) * {E} + {e}) * {K}')};")
            elif vec:
                vt, per, chunks = flat_vec(dt, E)
                vt += ua
                chunks *= K
                for ch in range(chunks):
                    if not any((e * K) // per == ch for e in range(E)):
                        continue        # a vector that holds none of the thread's elements
                    ptr = f"(const {vt}*)a{i} + ({idx}) * {chunks} + {ch}" if chunks > 1 \
                        else f"(const {vt}*)a{i} + ({idx})"
                    loads.append(f"{pad}const {vt} L{i}_{ch}{tag} = {_ld(nt_load, ptr)};")
            else:
                at = f"({idx}) * {K}" if K > 1 else f"({idx})"
                loads.append(f"{pad}const {CTYPE[dt]} L{i}{tag} = "
                             f"{_ld(nt_load, f'a{i} + {at}')};")
        if vec and not reduce_op:
            for o, dt in enumerate(out_dtypes):
                vt, per, chunks = flat_vec(dt, E)
                for ch in range(chunks):
                    work.append(f"{pad}{vt} R{o}_{ch}{tag};")
        for e in range(E):
            args = []
            for i, (dt, c) in enumerate(zip(prog.leaves, leaf_class)):
                if c == "b":
                    args.append(f"b{i}")
                elif vec:
                    args.append(element(i, dt, c, e, tag))
                else:
                    args.append(f"L{i}{tag}")
            outs = [f"t{o}" for o in range(n_out)]
            decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
            index = [f"({idx}) * {E} + {e}" if vec else f"({idx})"] if prog.uses_index else []
            call = f"dr_body({', '.join(index + args + scal + outs)});"
            if reduce_op:
                tail = f"acc{e} = {_combine(reduce_op, f'acc{e}', 't0')};"
            elif vec:
                tail = " ".join(f"R{o}_{e // flat_vec(dt, E)[1]}{tag}[{e % flat_vec(dt, E)[1]}] = t{o};"
                                for o, dt in enumerate(out_dtypes))
            else:
                tail = " ".join(_st(nt_store, f"t{o}", f"o{o} + ({idx})") for o in range(n_out))
            work.append(f"{pad}{{ {decl} {call} {tail} }}")
        if vec and not reduce_op:
            for o, dt in enumerate(out_dtypes):
                vt, per, chunks = flat_vec(dt, E)
                vt += ua
                for ch in range(chunks):
                    ptr = f"({vt}*)o{o} + ({idx}) * {chunks} + {ch}" if chunks > 1 \
                        else f"({vt}*)o{o} + ({idx})"
                    work.append(pad + _st(nt_store, f"R{o}_{ch}{tag}", ptr))
        return loads, work

    # Block-contiguous chunks: a block streams `unroll` runs of 256 consecutive
    # vectors, then moves on by gridDim.x chunks.  Launched with one chunk per
    # block where possible: on MI355X that keeps the DRAM access stream nearly
    # sequential and measures 8-10% faster on read+write streams than a few
    # persistent blocks striding through memory.
    count = "nvec" if vec else "n"
    if vec:
        L.append(f"    const long long nvec = (n - {E}) / {E};" if guard else f"    const long long nvec = n / {E};")
    if one_run and runs > 1:
        L.append(f"    const long long nchunk = {count} / {BLOCK * unroll * runs} * {runs};")
        L.append(f"    const long long nblk = nchunk / {runs};")
    else:
        L.append(f"    const long long nchunk = {count} / {BLOCK * unroll};")
        if one_run:
            L.append("    const long long nblk = nchunk;")
    if one_run:
        L.append("    if (blockIdx.x < nblk) {")
        L.append(f"        const long long c = blockIdx.x * {runs}LL;")
    else:
        L.append("    for (long long c = blockIdx.x; c < nchunk; c += gridDim.x) {")
    L.append(f"        const long long v = c * {BLOCK * unroll} + threadIdx.x;")
    all_loads, all_work = [], []
    for u in range(unroll):
        lo, wo = step(f"_u{u}", f"v + {u * BLOCK}" if u else "v", 8)
        all_loads += lo
        all_work += wo
    if packed:
        # all E * unroll elements of this thread go through the program together
        P, pad = E * unroll, " " * 8
        all_work = []
        args = []
        if prog.uses_index:
            bases = ", ".join(f"(v + {u * BLOCK}) * {E}" if u else f"v * {E}" for u in range(unroll))
            all_work.append(f"{pad}const long long G[{unroll}] = {{{bases}}};")
            args.append("G")
        for i, (dt, c) in enumerate(zip(prog.leaves, leaf_class)):
            if c == "b":
                args.append(f"b{i}")
                continue
            items = ", ".join(element(i, dt, c, e, f"_u{u}") for u in range(unroll) for e in range(E))
            all_work.append(f"{pad}const {CTYPE[dt]} P{i}[{P}] = {{{items}}};")
            args.append(f"P{i}")
        for o, dt in enumerate(out_dtypes):
            all_work.append(f"{pad}{CTYPE[dt]} T{o}[{P}];")
        outs = [f"T{o}" for o in range(n_out)]
        all_work.append(f"{pad}dr_body_pack({', '.join(args + scal + outs)});")
        for u in range(unroll):
            if reduce_op:
                for e in range(E):
                    all_work.append(f"{pad}acc{e} = {_combine(reduce_op, f'acc{e}', f'T0[{u * E + e}]')};")
                continue
            for o, dt in enumerate(out_dtypes):
                vt, per, chunks = flat_vec(dt, E)
                idx = f"v + {u * BLOCK}" if u else "v"
                if chunks > 1 and exchange:
                    # A lane holds `chunks` adjacent vectors.  Stored as they are, every store
                    # of the wave would write 16 bytes in every 16 * chunks; the lanes swap
                    # vectors through the wave's own stretch of LDS instead, so that each
                    # store covers 1 KB without gaps.  A wave's LDS accesses complete in
                    # order; the fences keep the compiler from reordering them.
                    xv = f"dr_xch{ITEMSIZE[dt]}"
                    for ch in range(chunks):
                        items = ", ".join(f"T{o}[{u * E + ch * per + k}]" for k in range(per))
                        all_work.append(f"{pad}{{ const {vt} R = {{{items}}}; "
                                        f"{xv}[threadIdx.x * {chunks} + {ch}] = R; }}")
                    all_work.append(f"{pad}DR_WAVE_SYNC();")
                    for ch in range(chunks):
                        ptr = f"({vt + ua}*)o{o} + (({idx}) - dr_lane) * {chunks} + {ch * WAVE} + dr_lane"
                        all_work.append(f"{pad}{{ const {vt} R = {xv}[(threadIdx.x - dr_lane) * {chunks} "
                                        f"+ {ch * WAVE} + dr_lane]; {_st(nt_store, 'R', ptr)} }}")
                    all_work.append(f"{pad}DR_WAVE_SYNC();")
                    continue
                for ch in range(chunks):
                    items = ", ".join(f"T{o}[{u * E + ch * per + k}]" for k in range(per))
                    ptr = f"({vt + ua}*)o{o} + ({idx}) * {chunks} + {ch}" if chunks > 1 \
                        else f"({vt + ua}*)o{o} + ({idx})"
                    all_work.append(f"{pad}{{ const {vt} R = {{{items}}}; "
                                    f"{_st(nt_store, 'R', ptr)} }}")
    L += all_loads
    if staged and one_run:
        L.append("        DR_STAGE_TABLES();      // after the loads: both are in flight together")
    L += all_work
    for r in range(1, runs if one_run else 1):
        L.append(f"        {{ const long long v = (c + {r}) * {BLOCK * unroll} + threadIdx.x;")
        L += all_loads + all_work
        L.append("        }")
    L.append("    }")
    # what is left over (less than one chunk) is spread over the first blocks; with one run
    # per block it belongs to the blocks behind the last run (code that follows the main
    # path would keep its constants in registers across it)
    if one_run:
        # one element per thread and pass: this path is short and must not need more
        # registers than the main one
        L.append("    else {")
        if staged:
            L.append("        DR_STAGE_TABLES();")
        L.append(f"        for (long long t = nchunk * {BLOCK * unroll * E} + (blockIdx.x - nblk) * {BLOCK} "
                 f"+ threadIdx.x; t < n; t += (gridDim.x - nblk) * {BLOCK}) {{")
        args = [f"b{i}" if c == "b" else f"a{i}[t * {step_of(c)}]" for i, c in enumerate(leaf_class)]
        args = (["t"] if prog.uses_index else []) + args
        decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
        outs = [f"t{o}" for o in range(n_out)]
        L.append(f"            {decl} dr_body({', '.join(args + scal + outs)});")
        for o in range(n_out):
            L.append(f"            o{o}[t] = t{o};")
        L.append("        }")
        L.append("    }")
    else:
        L.append(f"    for (long long v = nchunk * {BLOCK * unroll} + (long long)blockIdx.x * {BLOCK} "
                 f"+ threadIdx.x; v < {count}; v += (long long)gridDim.x * {BLOCK}) {{")
        lo, wo = step("", "v", 8)
        L += lo + wo
        L.append("    }")
        if vec and E > 1:
            # scalar tail: the last n % E elements, by the first threads of block 0
            L.append(f"    const long long t = nvec * {E} + (long long)blockIdx.x * {BLOCK} + threadIdx.x;")
            L.append("    if (t < n) {")
            args = [f"b{i}" if c == "b" else f"a{i}[t * {step_of(c)}]" for i, c in enumerate(leaf_class)]
            args = (["t"] if prog.uses_index else []) + args
            decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
            outs = [f"t{o}" for o in range(n_out)]
            L.append(f"        {decl} dr_body({', '.join(args + scal + outs)});")
            if reduce_op:
                L.append(f"        acc0 = {_combine(reduce_op, 'acc0', 't0')};")
            else:
                for o in range(n_out):
                    L.append(f"        o{o}[t] = t{o};")
            L.append("    }")
    if reduce_op:
        accs = [f"acc{e}" for e in range(max(E, 1))]
        while len(accs) > 1:   # pairwise: (acc0 + acc1) + (acc2 + acc3)
            accs = [f"({_combine(reduce_op, accs[i], accs[i + 1])})" if i + 1 < len(accs)
                    else accs[i] for i in range(0, len(accs), 2)]
        L.append(f"    {CTYPE[red_dt]} total = {accs[0]};")
        L.append("    total = dr_block_reduce(total);")
        L.append("    if (threadIdx.x == 0) partial[blockIdx.x] = total;")
    L.append("}")
    src.append("\n".join(L))
    return "\n".join(src) + "\n", E


# ---- general strided kernel ------------------------------------------------

def emit_nd(prog, ndim, out_dtypes, index32, reduce_op=None):
    """Arbitrary strides and broadcasting: each thread-iteration handles one
    output element, decomposing its linear index over the (merged) shape."""
    it = "unsigned int" if index32 else "long long"
    n_out = len(out_dtypes)
    red_dt = out_dtypes[0] if reduce_op else None
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    if reduce_op:
        src.append(emit_block_reduce(reduce_op, red_dt))
        src.append(emit_finalize(reduce_op, red_dt))
    params = [f"const {CTYPE[dt]}* a{i}" for i, dt in enumerate(prog.leaves)]
    if reduce_op:
        params.append(f"{CTYPE[red_dt]}* partial")
    else:
        params += [f"{CTYPE[dt]}* o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long n")
    params += [f"const {it} d{k}" for k in range(ndim)]
    for i in range(len(prog.leaves)):
        params += [f"const long long sa{i}_{k}" for k in range(ndim)]
    if not reduce_op:
        for o in range(n_out):
            params += [f"const long long so{o}_{k}" for k in range(ndim)]
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{"]
    if reduce_op:
        L.append(f"    {CTYPE[red_dt]} acc0 = {_identity(reduce_op, red_dt)};")
    L.append(f"    const long long stride = (long long)gridDim.x * {BLOCK};")
    L.append(f"    for (long long g = (long long)blockIdx.x * {BLOCK} + threadIdx.x; g < n; g += stride) {{")
    L.append(f"        {it} rem = ({it})g;")
    for k in reversed(range(ndim)):
        if k == 0:
            L.append(f"        const {it} c0 = rem;")
        else:
            L.append(f"        const {it} c{k} = rem % d{k}; rem /= d{k};")
    for i in range(len(prog.leaves)):
        off = " + ".join(f"(long long)c{k} * sa{i}_{k}" for k in range(ndim)) or "0"
        L.append(f"        const {CTYPE[prog.leaves[i]]} x{i} = a{i}[{off}];")
    decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
    call = ([f"x{i}" for i in range(len(prog.leaves))] + [f"s{i}" for i in range(len(prog.scalars))]
            + [f"t{o}" for o in range(n_out)])
    L.append(f"        {decl} dr_body({', '.join(call)});")
    if reduce_op:
        L.append(f"        acc0 = {_combine(reduce_op, 'acc0', 't0')};")
    else:
        for o in range(n_out):
            off = " + ".join(f"(long long)c{k} * so{o}_{k}" for k in range(ndim)) or "0"
            L.append(f"        o{o}[{off}] = t{o};")
    L.append("    }")
    if reduce_op:
        L.append("    acc0 = dr_block_reduce(acc0);")
        L.append("    if (threadIdx.x == 0) partial[blockIdx.x] = acc0;")
    L.append("}")
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


# ---- 2-D stencil kernel with an LDS halo tile ------------------------------

def _row_bases(nouter, names, indent):
    """Lines computing, for row index `i`, the element offset of that row in each
    operand: `names` is a list of (variable, stride parameter prefix).  With one
    outer dimension the offset is i * stride; with several, `i` is decomposed over
    the outer extents od1.. (od0 is implied) and dotted with the operand's strides,
    which is how N-d arrays and row/plane broadcasts are walked."""
    pad = " " * indent
    if nouter == 1:
        return [f"{pad}const long long {var} = (long long)i * {sp}_0;" for var, sp in names]
    # rows and extents are below 2^31 (the lowering checks): 32-bit unsigned division,
    # a quarter of the instructions of the 64-bit one, which would otherwise cost more
    # than the memory traffic of a row
    lines = [f"{pad}unsigned int rem_o = (unsigned int)i;"]
    lines += [f"{pad}long long {var} = 0;" for var, _ in names]
    for d in reversed(range(nouter)):
        if d == 0:
            lines.append(f"{pad}const long long q0 = rem_o;")
        else:
            lines.append(f"{pad}const unsigned int e{d} = (unsigned int)od{d};")
            lines.append(f"{pad}const unsigned int n{d} = rem_o / e{d};")
            lines.append(f"{pad}const long long q{d} = rem_o - n{d} * e{d}; rem_o = n{d};")
        lines += [f"{pad}{var} += q{d} * {sp}_{d};" for var, sp in names]
    return lines


def _outer_params(leaf_kind, n_out, nouter):
    """Kernel parameters describing the outer dimensions: extents od1.., then the
    outer strides of every directly read operand, then of every output."""
    params = [f"const long long od{d}" for d in range(1, nouter)]
    for i, k in enumerate(leaf_kind):
        if k[0] in ("d", "dv", "dr", "r"):
            params += [f"const long long os{i}_{d}" for d in range(nouter)]
    for o in range(n_out):
        params += [f"const long long oos{o}_{d}" for d in range(nouter)]
    return params


def _base_names(leaf_kind, n_out):
    names = [(f"base{i}", f"os{i}") for i, k in enumerate(leaf_kind)
             if k[0] in ("d", "dv", "dr", "r")]
    return names + [(f"obase{o}", f"oos{o}") for o in range(n_out)]


def emit_stencil(prog, leaf_kind, group, out_dtypes, tile_w, tile_h, restrict=True, nouter=1,
                 xcd_bands=True):
    """2-D tiled kernel; operands that are shifted views of one buffer are staged
    through an LDS halo tile.

    leaf_kind  per leaf: ('g', dy, dx) member of the halo group, shifted by
               (dy, dx) elements from the group's reference view;
               ('d',) operand with unit stride along the last dimension, read directly;
               ('r',) operand constant along the last dimension (column broadcast);
               ('b',) single element broadcast
    group      None, or (dtype code, dy_max, dx_min, dx_max): extent of the shifts
               (dy in [0, dy_max], dx in [dx_min, dx_max]); only with nouter == 1
    nouter     number of merged dimensions in front of the last one: the kernel's
               "rows" are their product (see `_row_bases`)

    The block stages the (tile_h + dy_max) x (tile_w + dx_max - dx_min) window of
    the buffer in LDS with coalesced loads, then every thread computes
    tile_h * tile_w / 256 outputs reading its shifted operands from LDS.
    Consecutive tile numbers go to one XCD, so tiles that share halo rows meet
    in the same L2."""
    rs = "__restrict__ " if restrict else ""
    n_out = len(out_dtypes)
    per_thread = tile_w * tile_h // BLOCK
    assert tile_w * tile_h % BLOCK == 0
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    params = []
    for i, dt in enumerate(prog.leaves):
        if leaf_kind[i][0] != "g":
            params.append(f"const {CTYPE[dt]}* {rs}a{i}")
    if group is not None:
        gdt, dy_max, dx_min, dx_max = group
        LW = tile_w + dx_max - dx_min
        LH = tile_h + dy_max
        params.append(f"const {CTYPE[gdt]}* {rs}gp")
    params += [f"{CTYPE[dt]}* {rs}o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const int H", "const int W"]
    if group is not None:
        params += ["const long long grs", "const long long glo", "const long long ghi"]
    params.append("const int tiles_x")
    params += _outer_params(leaf_kind, n_out, nouter)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{"]
    if group is not None:
        L.append(f"    __shared__ {CTYPE[gdt]} tile[{LH * LW}];")
    if xcd_bands:   # contiguous band of tiles per XCD (blocks are dealt round-robin to XCDs)
        L += ["    const int nb = gridDim.x;",
              f"    const int xcd = blockIdx.x % {N_XCD};",
              f"    const int slot = blockIdx.x / {N_XCD};",
              f"    const int t = xcd * (nb / {N_XCD}) + min(xcd, nb % {N_XCD}) + slot;"]
    else:
        L.append("    const int t = blockIdx.x;")
    L += ["    const int ty = t / tiles_x;",
         "    const int tx = t - ty * tiles_x;",
         f"    const int r0 = ty * {tile_h};",
         f"    const int c0 = tx * {tile_w};"]
    if group is not None:
        L += [f"    for (int idx = threadIdx.x; idx < {LH * LW}; idx += {BLOCK}) {{",
              f"        const int lr = idx / {LW};",
              f"        const int lc = idx - lr * {LW};",
              f"        const long long lin = (long long)(r0 + lr) * grs + (c0 + lc + ({dx_min}));",
              "        if (lin >= glo && lin < ghi) tile[idx] = gp[lin];",
              "    }",
              "    __syncthreads();"]
    L += ["#pragma unroll",
          f"    for (int k = 0; k < {per_thread}; ++k) {{",
          f"        const int e = threadIdx.x + k * {BLOCK};",
          f"        const int lr = e / {tile_w};",
          f"        const int lc = e - lr * {tile_w};",
          "        const int i = r0 + lr;",
          "        const int j = c0 + lc;",
          "        if (i < H && j < W) {"]
    L += _row_bases(nouter, _base_names(leaf_kind, n_out), 12)
    args = []
    for i, k in enumerate(leaf_kind):
        if k[0] == "g":
            _, dy, dx = k
            args.append(f"tile[(lr + {dy}) * {LW} + lc + ({dx - dx_min})]")
        elif k[0] == "d":
            args.append(f"a{i}[base{i} + j]")
        elif k[0] == "r":
            args.append(f"a{i}[base{i}]")
        else:
            args.append(f"a{i}[0]")
    decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
    call = args + [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]
    L.append(f"            {decl} dr_body({', '.join(call)});")
    for o in range(n_out):
        L.append(f"            o{o}[obase{o} + j] = t{o};")
    L += ["        }", "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_stencil_vec(prog, leaf_kind, group, out_dtypes, groups_per_row, rows_per_thread,
                     phase_group, phase_out, restrict=True, nt_load=False, nt_store=False,
                     xcd_bands=True, nouter=1, unaligned=False):
    """Vectorised 2-D tiled kernel for the aligned case: every output's row stride
    is a multiple of the 16-byte vector width VW and all outputs start at the same
    address phase (`phase_out` = address of output [0, 0] / itemsize, mod VW).

    leaf_kind  per leaf: ('g', dy, dx) member of the halo group (staged through LDS);
               ('dv',) 2-D operand whose rows have the outputs' phase and a stride
               that is a multiple of VW: read with 16-byte loads;
               ('d',) other operand with unit stride along the last dimension: element
               loads; ('dr',) operand walked backwards along the last dimension (stride
               -1, a flipped view): one 16-byte load at element alignment from the
               mirrored place, its elements reversed in registers;
               ('r',) operand constant along the last dimension;
               ('b',) single element broadcast
    group      None, or (dtype code, dy_max, dx_min, dx_max) with the group's row
               stride a multiple of VW and `phase_group` its reference element's phase

    Tiles start `phase_out` columns left of the view, so a thread's VW adjacent
    outputs are one aligned 16-byte store; the first/last column group of a row takes
    an element-wise path.  A block owns TW = groups_per_row * VW columns by
    TH = (256 / groups_per_row) * rows_per_thread rows; a thread computes VW outputs
    for `rows_per_thread` consecutive rows, so shifted LDS reads of neighbouring rows
    are shared in registers."""
    rs = "__restrict__ " if restrict else ""
    first = group[0] if group is not None else out_dtypes[0]
    vt, VW = VEC16[first]
    n_out = len(out_dtypes)
    GPR = groups_per_row
    slots = BLOCK // GPR
    TW = GPR * VW
    TH = slots * rows_per_thread
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    params = []
    for i, dt in enumerate(prog.leaves):
        if leaf_kind[i][0] != "g":
            params.append(f"const {CTYPE[dt]}* {rs}a{i}")
    if group is not None:
        gdt, dy_max, dx_min, dx_max = group
        ph = (phase_group - phase_out + dx_min) % VW
        LW = -(-(TW + dx_max - dx_min + ph) // VW) * VW
        LWV = LW // VW
        LH = TH + dy_max
        ct = CTYPE[gdt]
        params.append(f"const {ct}* {rs}gp")
    params += [f"{CTYPE[dt]}* {rs}o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const int H", "const int W"]
    if group is not None:
        params += ["const long long grs", "const long long glo", "const long long ghi"]
    params.append("const int tiles_x")
    params += _outer_params(leaf_kind, n_out, nouter)
    for i, k in enumerate(leaf_kind):
        if k[0] == "dv":       # elements of the operand's buffer before and from its pointer
            params += [f"const long long lo{i}", f"const long long hi{i}"]
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{"]
    if group is not None:
        L.append(f"    __shared__ {vt} tile[{LH * LWV}];")
    L += ["    const int nb = gridDim.x;",
          f"    const int xcd = blockIdx.x % {N_XCD};",
          f"    const int slot = blockIdx.x / {N_XCD};",
          (f"    const int t = xcd * (nb / {N_XCD}) + min(xcd, nb % {N_XCD}) + slot;" if xcd_bands
           else "    const int t = blockIdx.x;"),
          "    const int ty = t / tiles_x;",
          "    const int tx = t - ty * tiles_x;",
          f"    const int r0 = ty * {TH};",
          f"    const int j0 = tx * {TW} - {phase_out};      // first output column of the tile"]
    if group is not None:
        L += [f"    const int cs = j0 + ({dx_min}) - {ph};       // buffer column held in LDS column 0",
              f"    for (int idx = threadIdx.x; idx < {LH * LWV}; idx += {BLOCK}) {{",
              f"        const int lr = idx / {LWV};",
              f"        const int lv = idx - lr * {LWV};",
              f"        const long long lin = (long long)(r0 + lr) * grs + cs + lv * {VW};",
              f"        {vt} val;",
              f"        if (lin >= glo && lin + {VW} <= ghi) {{",
              f"            val = {_ld(nt_load, f'(const {vt}*)(gp + lin)')};",
              "        } else {",
              "#pragma unroll",
              f"            for (int e = 0; e < {VW}; ++e)",
              f"                val[e] = (lin + e >= glo && lin + e < ghi) ? gp[lin + e] : ({ct})0;",
              "        }",
              "        tile[idx] = val;",
              "    }",
              "    __syncthreads();",
              f"    const {ct}* ts = (const {ct}*)tile;"]
    L += [f"    const int g = threadIdx.x % {GPR};",
          f"    const int rw = threadIdx.x / {GPR};",
          f"    const int jf = j0 + g * {VW};                // first of this thread's {VW} columns",
          f"    const bool inner = jf >= 0 && jf + {VW} <= W;",
          "#pragma unroll",
          f"    for (int k = 0; k < {rows_per_thread}; ++k) {{",
          f"        const int lr = rw * {rows_per_thread} + k;",
          "        const int i = r0 + lr;",
          "        if (i >= H) break;"]
    L += _row_bases(nouter, _base_names(leaf_kind, n_out), 8)

    def operand(i, k, e):
        if k[0] == "g":
            _, dy, dx = k
            return f"ts[(lr + {dy}) * {LW} + g * {VW} + {e + dx - dx_min + ph}]"
        if k[0] in ("d", "dv", "dr"):
            return f"D{i}[{e}]"
        if k[0] == "r":
            return f"a{i}[base{i}]"
        return f"a{i}[0]"

    decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
    tail_args = [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]
    # Directly read operands.  The first and last column group of a row hold columns outside
    # the view: their vectors are loaded whole where the operand's buffer reaches that far
    # (an interior view: always), element by element otherwise; the body then runs once per
    # output and only the stores are masked.  Evaluating such groups element by element,
    # loads included, cost every wave of a short row eight more memory instructions.
    for i, k in enumerate(leaf_kind):
        if k[0] == "dv":
            lvt = VEC16[prog.leaves[i]][0] + ("u" if unaligned else "")
            ptr = f"(const {lvt}*)(a{i} + base{i} + jf)"
            L += [f"        {VEC16[prog.leaves[i]][0]} D{i};",
                  f"        if (inner || (base{i} + jf >= lo{i} && base{i} + jf + {VW} <= hi{i})) {{",
                  f"            D{i} = {_ld(nt_load, ptr)};",
                  "        } else {"]
            L += [f"            D{i}[{e}] = (jf + {e} >= 0 && jf + {e} < W) ? a{i}[base{i} + jf + {e}] "
                  f": ({CTYPE[prog.leaves[i]]})0;" for e in range(VW)]
            L.append("        }")
        elif k[0] == "dr":
            lvt = VEC16[prog.leaves[i]][0]
            ptr = f"(const {lvt}u*)(a{i} + base{i} - jf - {VW - 1})"
            L += [f"        {lvt} D{i};",
                  "        if (inner) {",
                  f"            const {lvt}u T{i} = {_ld(nt_load, ptr)};",
                  "            " + " ".join(f"D{i}[{e}] = T{i}[{VW - 1 - e}];" for e in range(VW)),
                  "        } else {"]
            L += [f"            D{i}[{e}] = (jf + {e} >= 0 && jf + {e} < W) ? a{i}[base{i} - jf - {e}] "
                  f": ({CTYPE[prog.leaves[i]]})0;" for e in range(VW)]
            L.append("        }")
        elif k[0] == "d":
            ct_i = CTYPE[prog.leaves[i]]
            L.append(f"        {ct_i} D{i}[{VW}];")
            L.append("        if (inner) {")
            L.append("            " + " ".join(f"D{i}[{e}] = a{i}[base{i} + jf + {e}];" for e in range(VW)))
            L.append("        } else {")
            L += [f"            D{i}[{e}] = (jf + {e} >= 0 && jf + {e} < W) ? a{i}[base{i} + jf + {e}] "
                  f": ({ct_i})0;" for e in range(VW)]
            L.append("        }")
    for o, dt in enumerate(out_dtypes):
        L.append(f"        {VEC16[dt][0]} R{o};")
    for e in range(VW):
        args = [operand(i, k, e) for i, k in enumerate(leaf_kind)]
        sets = " ".join(f"R{o}[{e}] = t{o};" for o in range(n_out))
        L.append(f"        {{ {decl} dr_body({', '.join(args + tail_args)}); {sets} }}")
    L.append("        if (inner) {")
    for o, dt in enumerate(out_dtypes):
        ovt = VEC16[dt][0] + ("u" if unaligned else "")
        L.append("            " + _st(nt_store, f"R{o}", f"({ovt}*)(o{o} + obase{o} + jf)"))
    L.append("        } else {")
    for e in range(VW):
        stores = " ".join(f"o{o}[obase{o} + jf + {e}] = R{o}[{e}];" for o in range(n_out))
        L.append(f"            if (jf + {e} >= 0 && jf + {e} < W) {{ {stores} }}")
    L += ["        }", "    }", "}"]
    src.append("\n".join(L))
    lds_bytes = LH * LW * ITEMSIZE[first] if group is not None else 0
    return "\n".join(src) + "\n", TW, TH, lds_bytes


def emit_stencil3d(prog, leaf_kind, group, out_dtypes, groups_per_row, rows_per_thread,
                   phase_group, phase_out, restrict=True, nt_store=True, xcd_bands=True, depth=1):
    """Vectorised 3-D tiled kernel: operands that are shifted views of one buffer are
    staged through an LDS window of the buffer, like `emit_stencil_vec` does in two
    dimensions.  Without it a 7-point stencil fetches six vectors per four outputs
    through L2 and is bound by that cache (measured 40 % of HBM speed on 512^3).

    leaf_kind  per leaf: ('g', dz, dy, dx) member of the halo group; ('dv',) operand with
               the outputs' alignment, read with 16-byte loads; ('d',) other operand
               with unit stride along the last dimension; ('r',) operand constant along
               the last dimension; ('b',) single element broadcast
    group      (dtype code, dz_max, dy_min, dy_max, dx_min, dx_max): dz in [0, dz_max]

    A block owns TW = groups_per_row * VW columns and TY = rows_per_thread * 256 /
    groups_per_row rows, and walks ZC planes (a launch parameter) with a ring of window
    planes in LDS: every plane of the buffer is fetched once per block instead of once
    per plane that uses it (a window of 4 + 2 planes re-reads half the volume).  The
    ring holds dz_max + 2 planes rounded up to a power of two: a plane goes from registers
    to the ring slot of the plane that was retired one step earlier, so one barrier per
    plane is enough.  The next `depth` planes are in flight in registers meanwhile (the
    loop over planes is unrolled `depth` times, each copy with its own registers).
    A thread computes VW adjacent outputs in each of its rows; the body runs once per
    output, also in the first and last column group of a row, where only the loads of
    directly read operands and the stores are done element by element.
    Measured on 512^3 float32 (7-point, microseconds per sweep): 4 planes x 16 rows x 64
    columns without the ring 262; ring with tiles of 32 x 64: 235, 8 x 256: 211 (depth 1;
    2 and 3 planes in flight: 218, 223).  What bounds it is the number of cache lines a
    compute unit requests per line it stores, not the bytes from HBM (1.08 x algorithmic):
    a tile of 8 x 256 asks for 10 rows x 10 lines and stores 64, a copy asks for 64 and
    stores 64; 164 / 128 of the copy kernel's time is what the 8 x 256 tile takes, and
    the other shapes follow the same ratio.  Alignment works
    as in the 2-D kernel: tiles start `phase_out` columns left of the view, the first
    and last column group of a row take element stores.
    Parameters: directly read leaves, group pointer, outputs, scalars, Z, Y, W, group
    plane and row stride, first and last 16-byte aligned vector of the buffer (glo, ghi;
    in elements relative to the group pointer), tiles_x, tiles_y, ZC, then plane and row stride of every directly read leaf
    and of every output."""
    rs = "__restrict__ " if restrict else ""
    gdt, dz_max, dy_min, dy_max, dx_min, dx_max = group
    vt, VW = VEC16[gdt]
    ct = CTYPE[gdt]
    n_out = len(out_dtypes)
    GPR = groups_per_row
    RY = BLOCK // GPR
    RPT = rows_per_thread
    TY = RY * RPT
    TW = GPR * VW
    ph = (phase_group - phase_out + dx_min) % VW
    LW = -(-(TW + dx_max - dx_min + ph) // VW) * VW
    LWV = LW // VW
    WY = TY + dy_max - dy_min
    PV = WY * LWV                     # 16-byte vectors per window plane
    NV = -(-PV // BLOCK)              # of them per thread
    NS = 2
    while NS < dz_max + 2:
        NS *= 2
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    params = [f"const {CTYPE[dt]}* {rs}a{i}" for i, dt in enumerate(prog.leaves)
              if leaf_kind[i][0] != "g"]
    params.append(f"const {ct}* {rs}gp")
    params += [f"{CTYPE[dt]}* {rs}o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const int Z", "const int Y", "const int W", "const long long gps",
               "const long long grs", "const long long glo", "const long long ghi",
               "const int tiles_x", "const int tiles_y", "const int ZC"]
    for i, k in enumerate(leaf_kind):
        if k[0] in ("d", "dv", "r"):
            params += [f"const long long os{i}_0", f"const long long os{i}_1"]
    for o in range(n_out):
        params += [f"const long long oos{o}_0", f"const long long oos{o}_1"]

    def fetch(plane, ind, cur="cur0"):
        """`cur` <- this thread's vectors of buffer plane `plane`.  A vector that is not
        wholly inside the buffer is read from the nearest aligned place that is: only
        outputs outside the view would use its values, and those are not stored.  No branch
        surrounds the loads, so the compiler counts outstanding loads exactly instead of
        waiting for all of them at every join.  For the same reason the planes past the
        last one the block needs are fetched too (as that last plane again, from L2)."""
        return [ind + "#pragma unroll",
                ind + f"for (int q = 0; q < {NV}; ++q) {{",
                ind + f"    const long long lin = wlin[q] + (long long)min({plane}, zlast) * gps;",
                ind + f"    {cur}[q] = *(const {vt}*)(gp + min(max(lin, glo), ghi));",
                ind + "}"]

    def stash(slot, ind, cur="cur0"):
        return [ind + "#pragma unroll",
                ind + f"for (int q = 0; q < {NV}; ++q)",
                ind + f"    if (threadIdx.x + q * {BLOCK} < {PV}) "
                      f"tile[({slot}) * {PV} + threadIdx.x + q * {BLOCK}] = {cur}[q];"]

    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    __shared__ {vt} tile[{NS * PV}];",
         "    const int nb = gridDim.x;",
         f"    const int xcd = blockIdx.x % {N_XCD};",
         f"    const int slot = blockIdx.x / {N_XCD};",
         (f"    const int t = xcd * (nb / {N_XCD}) + min(xcd, nb % {N_XCD}) + slot;" if xcd_bands
          else "    const int t = blockIdx.x;"),
         "    const int tyz = t / tiles_x;",
         "    const int tx = t - tyz * tiles_x;",
         "    const int tz = tyz / tiles_y;",
         "    const int ty = tyz - tz * tiles_y;",
         "    const int z0 = tz * ZC;",
         "    const int nk = min(ZC, Z - z0);",
         f"    const int zlast = z0 + nk - 1 + {dz_max};      // last plane of the buffer the block needs",
         f"    const int y0 = ty * {TY};",
         f"    const int j0 = tx * {TW} - {phase_out};      // first output column of the tile",
         f"    const int cs = j0 + ({dx_min}) - {ph};       // buffer column held in LDS column 0",
         f"    long long wlin[{NV}];                         // this thread's window vectors in a plane",
         "#pragma unroll",
         f"    for (int q = 0; q < {NV}; ++q) {{",
         f"        const int idx = threadIdx.x + q * {BLOCK};",
         f"        const int wy = idx / {LWV};",
         f"        const int lv = idx - wy * {LWV};",
         f"        wlin[q] = (long long)(y0 + wy + ({dy_min})) * grs + cs + lv * {VW};",
         "    }",
         "    " + " ".join(f"{vt} cur{u}[{NV}];" for u in range(depth)),
         f"    for (int p = 0; p < {dz_max}; ++p) {{"]
    L += fetch("z0 + p", "        ") + stash("p", "        ") + ["    }"]
    for u in range(depth):
        L += fetch(f"z0 + {dz_max + u}", "    ", f"cur{u}")
    L += [f"    const {ct}* ts = (const {ct}*)tile;",
          f"    const int g = threadIdx.x % {GPR};",
          f"    const int ly = threadIdx.x / {GPR};",
          f"    const int jf = j0 + g * {VW};                // first of this thread's {VW} columns",
          f"    const bool inner = jf >= 0 && jf + {VW} <= W;",
          f"    for (int k0 = 0; k0 < nk; k0 += {depth}) {{"]
    decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
    tail_args = [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]

    def operand(i, kd, e):
        if kd[0] == "g":
            _, dz, dy, dx = kd
            return (f"ts[sl{dz} + (lyr + {dy - dy_min}) * {LW} + g * {VW} + "
                    f"{e + dx - dx_min + ph}]")
        if kd[0] in ("d", "dv"):
            return f"D{i}[{e}]"
        if kd[0] == "r":
            return f"a{i}[base{i}]"
        return f"a{i}[0]"

    for u in range(depth):
        L += ["        {",
              f"        const int k = k0 + {u};",
              "        if (k >= nk) break;"]
        L += stash(f"(k + {dz_max}) & {NS - 1}", "        ", f"cur{u}")
        L += ["        __syncthreads();"]
        L += fetch(f"z0 + k + {depth + dz_max}", "        ", f"cur{u}")
        L += ["        const int z = z0 + k;"]
        for dz in sorted({kd[1] for kd in leaf_kind if kd[0] == "g"}):
            L.append(f"        const int sl{dz} = ((k + {dz}) & {NS - 1}) * {PV * VW};")
        L += ["#pragma unroll",
              f"        for (int r = 0; r < {RPT}; ++r) {{",
              f"            const int lyr = ly + r * {RY};",
              "            const int y = y0 + lyr;",
              "            if (y >= Y) break;"]
        for i, kd in enumerate(leaf_kind):
            if kd[0] in ("d", "dv", "r"):
                L.append(f"            const long long base{i} = (long long)z * os{i}_0 + (long long)y * os{i}_1;")
        for o in range(n_out):
            L.append(f"            const long long obase{o} = (long long)z * oos{o}_0 + (long long)y * oos{o}_1;")
        # operands read directly: whole vectors where the thread's columns are all inside
        # the view, single elements (0 outside) in the first and last column group of a row
        for i, kd in enumerate(leaf_kind):
            if kd[0] in ("d", "dv"):
                lct = CTYPE[prog.leaves[i]]
                L.append(f"            {lct} D{i}[{VW}];")
        direct = [i for i, kd in enumerate(leaf_kind) if kd[0] in ("d", "dv")]
        if direct:
            L.append("            if (inner) {")
            for i in direct:
                if leaf_kind[i][0] == "dv":
                    lvt = VEC16[prog.leaves[i]][0]
                    L.append(f"                const {lvt} V{i} = *(const {lvt}*)(a{i} + base{i} + jf);")
                    L.append(f"                " + " ".join(f"D{i}[{e}] = V{i}[{e}];" for e in range(VW)))
                else:
                    L.append(f"                " + " ".join(f"D{i}[{e}] = a{i}[base{i} + jf + {e}];"
                                                             for e in range(VW)))
            L.append("            } else {")
            for i in direct:
                lct = CTYPE[prog.leaves[i]]
                for e in range(VW):
                    L.append(f"                D{i}[{e}] = (jf + {e} >= 0 && jf + {e} < W) "
                             f"? a{i}[base{i} + jf + {e}] : ({lct})0;")
            L.append("            }")
        for o, dt in enumerate(out_dtypes):
            L.append(f"            {VEC16[dt][0]} R{o};")
        for e in range(VW):
            args = [operand(i, kd, e) for i, kd in enumerate(leaf_kind)]
            sets = " ".join(f"R{o}[{e}] = t{o};" for o in range(n_out))
            L.append(f"            {{ {decl} dr_body({', '.join(args + tail_args)}); {sets} }}")
        L.append("            if (inner) {")
        for o, dt in enumerate(out_dtypes):
            L.append("                " + _st(nt_store, f"R{o}", f"({VEC16[dt][0]}*)(o{o} + obase{o} + jf)"))
        L.append("            } else {")
        for e in range(VW):
            stores = " ".join(f"o{o}[obase{o} + jf + {e}] = R{o}[{e}];" for o in range(n_out))
            L.append(f"                if (jf + {e} >= 0 && jf + {e} < W) {{ {stores} }}")
        L += ["            }", "        }", "        }"]
    L += ["    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n", TW, TY, NS, NS * PV * VW * ITEMSIZE[gdt]


# ---- reduction along some axes ------------------------------------------------

def emit_axis_reduce(prog, kdim, rdim, acc_dt, op, strategy, row_vec=None):
    """Reduce the (fused) expression over `rdim` merged dimensions, keeping `kdim`.

    The reduced extent R may be cut into S slices of RS elements; the kernel then
    writes S partial results per output and a second launch reduces those.

    strategy 'col'  a block owns 64 adjacent outputs (one per lane) and one slice;
                    its 4 waves walk different reduced indices and meet through LDS.
                    Coalesced when the fastest-varying memory dimension is kept
                    (sum over axis 0 of a row-major matrix).  Partials: [slice][output].
             'row'  a wave owns one (output, slice); its lanes stride over the
                    reduced extent and meet with a shuffle tree.  Coalesced when the
                    fastest-varying dimension is reduced (sum over the last axis).
                    Partials: [output][slice].
    row_vec         ('row' with one reduced dimension only) per leaf 'v' (unit stride
                    along the reduced dimension: 16-byte loads at element alignment)
                    or 'k' (constant along it)
    Parameters: leaf pointers, output pointer, scalars, K, R, S, RS, kept dims,
    reduced dims, then per leaf its kept strides and its reduced strides."""
    ct = CTYPE[acc_dt]
    src = [PREAMBLE, emit_body(prog, [acc_dt])]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const long long K", "const long long R", "const long long S", "const long long RS"]
    params += [f"const long long dk{d}" for d in range(kdim)]
    params += [f"const long long dr{d}" for d in range(rdim)]
    for i in range(len(prog.leaves)):
        params += [f"const long long sk{i}_{d}" for d in range(kdim)]
        params += [f"const long long sr{i}_{d}" for d in range(rdim)]
    nl = len(prog.leaves)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{"]

    def decompose(var, dims, prefix, n, out_prefix, indent):
        """Lines turning linear index `var` into per-leaf offsets `out_prefix{i}`."""
        pad = " " * indent
        lines = [f"{pad}long long rem_{prefix} = {var};"]
        for i in range(nl):
            lines.append(f"{pad}long long {out_prefix}{i} = 0;")
        for d in reversed(range(n)):
            if d == 0:
                lines.append(f"{pad}const long long c_{prefix}{d} = rem_{prefix};")
            else:
                lines.append(f"{pad}const long long c_{prefix}{d} = rem_{prefix} % {dims}{d}; "
                             f"rem_{prefix} /= {dims}{d};")
            for i in range(nl):
                lines.append(f"{pad}{out_prefix}{i} += c_{prefix}{d} * s{prefix}{i}_{d};")
        return lines

    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    args = [f"a{i}[bk{i} + br{i}]" for i in range(nl)]
    ident = _identity(op, acc_dt)
    if strategy == "col":
        waves = BLOCK // WAVE
        L += [f"    __shared__ {ct} red[{waves}][{WAVE}];",
              f"    const int tx = threadIdx.x & {WAVE - 1};",
              "    const int ty = threadIdx.x >> 6;",
              f"    const long long ktiles = (K + {WAVE - 1}) / {WAVE};",
              "    for (long long b = blockIdx.x; b < ktiles * S; b += gridDim.x) {",
              "        const long long sl = b / ktiles;",
              f"        const long long g = (b - sl * ktiles) * {WAVE} + tx;",
              f"        {ct} acc = {ident};",
              "        if (g < K) {"]
        L += decompose("g", "dk", "k", kdim, "bk", 12)
        L += ["            const long long r_end = (sl + 1) * RS < R ? (sl + 1) * RS : R;",
              "#pragma unroll 4",
              f"            for (long long r = sl * RS + ty; r < r_end; r += {waves}) {{"]
        L += decompose("r", "dr", "r", rdim, "br", 16)
        L += [f"                {ct} t0; dr_body({', '.join(args + call_tail)});",
              f"                acc = {_combine(op, 'acc', 't0')};",
              "            }",
              "        }",
              "        red[ty][tx] = acc;",
              "        __syncthreads();",
              "        if (ty == 0 && g < K) {",
              "#pragma unroll",
              f"            for (int w = 1; w < {waves}; ++w) acc = {_combine(op, 'acc', 'red[w][tx]')};",
              "            out[sl * K + g] = acc;",
              "        }",
              "        __syncthreads();",
              "    }"]
    else:
        shfl = "__shfl_down(acc, off, 64)"
        if acc_dt in ("u1", "b1"):
            shfl = f"({ct})__shfl_down((int)acc, off, 64)"
        L += [f"    const int lane = threadIdx.x & {WAVE - 1};",
              f"    const long long nwaves = (long long)gridDim.x * {BLOCK // WAVE};",
              "#pragma unroll 2",
              f"    for (long long o = (long long)blockIdx.x * {BLOCK // WAVE} + (threadIdx.x >> 6); "
              "o < K * S; o += nwaves) {",
              "        const long long g = o / S;",
              "        const long long sl = o - g * S;"]
        L += decompose("g", "dk", "k", kdim, "bk", 8)
        L += [f"        {ct} acc = {ident};",
              "        const long long r_end = (sl + 1) * RS < R ? (sl + 1) * RS : R;"]
        if row_vec:
            widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, row_vec) if k == "v"}
            V = 16 // widths.pop()
            for i, (dt, k) in enumerate(zip(prog.leaves, row_vec)):
                if k == "k":
                    L.append(f"        const {CTYPE[dt]} c{i} = a{i}[bk{i}];")
            L += ["        long long r = sl * RS + (long long)lane * " + str(V) + ";",
                  "#pragma unroll 2",
                  f"        for (; r + {V} <= r_end; r += {WAVE * V}) {{"]
            for i, (dt, k) in enumerate(zip(prog.leaves, row_vec)):
                if k == "v":
                    vt = VEC16[dt][0] + "u"
                    L.append(f"            const {vt} X{i} = *(const {vt}*)(a{i} + bk{i} + r);")
            for e in range(V):
                vargs = [f"X{i}[{e}]" if k == "v" else f"c{i}" for i, k in enumerate(row_vec)]
                L.append(f"            {{ {ct} t0; dr_body({', '.join(vargs + call_tail)}); "
                         f"acc = {_combine(op, 'acc', 't0')}; }}")
            L.append("        }")
            # exactly one lane is left with r < r_end: the one whose next vector would
            # straddle the end; it finishes the row element by element
            sargs = [f"a{i}[bk{i} + r]" if k == "v" else f"c{i}" for i, k in enumerate(row_vec)]
            L += ["        for (; r < r_end; ++r) {",
                  f"            {ct} t0; dr_body({', '.join(sargs + call_tail)});",
                  f"            acc = {_combine(op, 'acc', 't0')};",
                  "        }"]
        else:
            L += ["#pragma unroll 4",
                  f"        for (long long r = sl * RS + lane; r < r_end; r += {WAVE}) {{"]
            L += decompose("r", "dr", "r", rdim, "br", 12)
            L += [f"            {ct} t0; dr_body({', '.join(args + call_tail)});",
                  f"            acc = {_combine(op, 'acc', 't0')};",
                  "        }"]
        L += [
              "#pragma unroll",
              f"        for (int off = {WAVE // 2}; off > 0; off >>= 1) {{",
              f"            const {ct} other = {shfl};",
              f"            acc = {_combine(op, 'acc', 'other')};",
              "        }",
              "        if (lane == 0) out[o] = acc;",
              "    }"]
    L.append("}")
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_narrow_cols(prog, leaf_kind, acc_dt, op, K):
    """Reduction over the rows of a dense row-major matrix with few columns (K is a
    compile-time constant; at most 64 units of 16 bytes, or 64 elements when K is no
    multiple of a unit): the matrix is read as one contiguous stream, each
    lane keeps the columns it meets in its own accumulators, and lanes holding the
    same columns are combined once at the end.

    A wave uses LW = (64 / KC) * KC lanes, KC = K / V units per row, V elements per
    16-byte unit (V = 1 when K is not a multiple of that); chunk number w covers units
    [w LW, (w+1) LW), so lane l always sees columns (l mod KC) V ... + V - 1.  A wave
    takes four consecutive chunks at a time.

    leaf_kind  per leaf 'd' (dense R x K), 'w' (one row of K for all), 'c' (one value per
               row: the weights of a weighted sum of the rows), 'b' (one element)
    Parameters: leaf pointers, partials pointer, scalars, U (units in the matrix).
    Output: one partial per block and column, [block][K]."""
    ct = CTYPE[acc_dt]
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "d"}
    V = 16 // widths.pop() if len(widths) == 1 and widths <= {4, 8} else 1
    if K % V:
        V = 1
    KC = K // V
    LW = (WAVE // KC) * KC
    waves = BLOCK // WAVE
    src = [PREAMBLE, emit_body(prog, [acc_dt])]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long U")
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    ident = _identity(op, acc_dt)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    __shared__ {ct} red[{waves}][{WAVE * V}];",
         f"    const int lane = threadIdx.x & {WAVE - 1};",
         "    const int wave = threadIdx.x >> 6;",
         f"    const bool live = lane < {LW};",
         f"    const int cls = lane % {KC};"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        for e in range(V):
            if kind == "w":
                L.append(f"    const {CTYPE[dt]} w{i}_{e} = a{i}[cls * {V} + {e}];")
        if kind == "b":
            L.append(f"    const {CTYPE[dt]} b{i} = a{i}[0];")
    for e in range(V):
        L.append(f"    {ct} acc{e} = {ident};")
    UN = 4      # chunks in flight per wave: loads first, then arithmetic
    L += [f"    const long long nw = (long long)gridDim.x * {waves};",
          f"    for (long long g = (long long)blockIdx.x * {waves} + wave; g * {UN * LW} < U; g += nw) {{"]
    for j in range(UN):
        L.append(f"        const long long u{j} = (g * {UN} + {j}) * {LW} + lane;")
        L.append(f"        const bool ok{j} = live && u{j} < U;")
        for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
            if kind == "d":
                if V > 1:
                    vt = VEC16[dt][0] + "u"
                    L.append(f"        {VEC16[dt][0]} X{i}_{j} = {{}};")
                    L.append(f"        if (ok{j}) X{i}_{j} = *(const {vt}*)(a{i} + u{j} * {V});")
                else:
                    L.append(f"        {CTYPE[dt]} X{i}_{j} = 0;")
                    L.append(f"        if (ok{j}) X{i}_{j} = a{i}[u{j}];")
            elif kind == "c":       # the row of unit u: neighbouring lanes share it
                L.append(f"        {CTYPE[dt]} C{i}_{j} = 0;")
                L.append(f"        if (ok{j}) C{i}_{j} = a{i}[u{j} / {KC}];")
    for j in range(UN):
        L.append(f"        if (ok{j}) {{")
        for e in range(V):
            args = []
            for i, kind in enumerate(leaf_kind):
                if kind == "d":
                    args.append(f"X{i}_{j}[{e}]" if V > 1 else f"X{i}_{j}")
                elif kind == "w":
                    args.append(f"w{i}_{e}")
                elif kind == "c":
                    args.append(f"C{i}_{j}")
                else:
                    args.append(f"b{i}")
            L.append(f"            {{ {ct} t0; dr_body({', '.join(args + call_tail)}); "
                     f"acc{e} = {_combine(op, f'acc{e}', 't0')}; }}")
        L.append("        }")
    L.append("    }")
    for e in range(V):
        L.append(f"    red[wave][lane * {V} + {e}] = acc{e};")
    L += ["    __syncthreads();",
          f"    if (threadIdx.x < {K}) {{",
          f"        const int cc = threadIdx.x / {V};",
          f"        const int e = threadIdx.x - cc * {V};",
          f"        {ct} tot = {ident};",
          f"        for (int w = 0; w < {waves}; ++w)",
          f"            for (int l = cc; l < {LW}; l += {KC})",
          f"                tot = {_combine(op, 'tot', f'red[w][l * {V} + e]')};",
          f"        out[(long long)blockIdx.x * {K} + threadIdx.x] = tot;",
          "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n", V, LW


def emit_short_rows(prog, leaf_kind, acc_dt, op, R, outer2=False):
    """Reduction over a short unit-stride last dimension: a lane owns one output and
    walks its own row of R elements (R is a compile-time constant) with 16-byte loads
    at element alignment.  The lanes' loads are a row pitch apart, but a wave's R
    loads together consume whole cache lines, and there is no combining step at all;
    measured on MI355X this reads 4-7 TB/s for R <= 64 where a wave per row with a
    shuffle tree reaches 0.1-1.6.

    leaf_kind  per leaf 'v' (unit stride along the row) or 'k' (constant along it)
    Parameters: leaf pointers, output pointer, scalars, K, then per leaf the stride
    between rows (elements)."""
    ct = CTYPE[acc_dt]
    nl = len(prog.leaves)
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    V = 16 // widths.pop() if len(widths) == 1 and widths <= {4, 8} else 1
    src = [PREAMBLE, emit_body(prog, [acc_dt])]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long K")
    params += [f"const long long sk{i}" for i in range(nl)]
    if outer2:
        params.append("const unsigned int K1")
        params += [f"const long long sj{i}" for i in range(nl)]
        src.append(ROW_AT)
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    const long long k = (long long)blockIdx.x * {BLOCK} + threadIdx.x;",
         "    if (k >= K) return;"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            L.append(f"    const {CTYPE[dt]}* row{i} = a{i} + {_row_at(outer2, i, 'k')};")
        else:
            L.append(f"    const {CTYPE[dt]} c{i} = a{i}[{_row_at(outer2, i, 'k')}];")
    L.append(f"    {ct} acc = {_identity(op, acc_dt)};")

    def element(args):
        return [f"        {{ {ct} t0; dr_body({', '.join(args + call_tail)}); "
                f"acc = {_combine(op, 'acc', 't0')}; }}"]

    nvec = R // V if V > 1 else 0
    if nvec:
        L += ["#pragma unroll", f"    for (int v = 0; v < {nvec}; ++v) {{"]
        for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
            if kind == "v":
                vt = VEC16[dt][0] + "u"
                L.append(f"        const {vt} X{i} = *(const {vt}*)(row{i} + v * {V});")
        for e in range(V):
            L += element([f"X{i}[{e}]" if kind == "v" else f"c{i}"
                          for i, kind in enumerate(leaf_kind)])
        L.append("    }")
    if nvec * V < R:
        L += ["#pragma unroll", f"    for (int j = {nvec * V}; j < {R}; ++j) {{"]
        L += element([f"row{i}[j]" if kind == "v" else f"c{i}" for i, kind in enumerate(leaf_kind)])
        L.append("    }")
    L += ["    out[k] = acc;", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_group_rows(prog, leaf_kind, acc_dt, op, R, G, outer2=False):
    """Reduction over a unit-stride last dimension of R elements (a compile-time
    constant) by groups of G lanes (G a power of two, 8..64): a wave holds 64 / G rows at a
    time, lane j of a group takes the 16-byte units j, j + G, ... of its row (a group reads
    16 G contiguous bytes per step), and the group's lanes meet in log2 G butterfly steps.
    A whole wave per row leaves lanes idle whenever a row is not a multiple of 256 elements
    (200 floats: 22 % of the lanes, then six combining steps for one output); groups of
    eight waste a tenth as many unit slots, combine in three steps and store eight adjacent
    outputs per wave.

    leaf_kind  per leaf 'v' (unit stride along the row) or 'k' (constant along it)
    Parameters: leaf pointers, output pointer, scalars, K, then per leaf the stride
    between rows (elements)."""
    ct = CTYPE[acc_dt]
    nl = len(prog.leaves)
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    V = 16 // widths.pop() if len(widths) == 1 and widths <= {4, 8} else 1
    units = -(-R // V)                     # 16-byte units per row, the last one maybe partial
    steps = -(-units // G)
    per_wave = WAVE // G
    src = [PREAMBLE, emit_body(prog, [acc_dt])]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long K")
    params += [f"const long long sk{i}" for i in range(nl)]
    if outer2:
        params.append("const unsigned int K1")
        params += [f"const long long sj{i}" for i in range(nl)]
        src.append(ROW_AT)
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    shfl = "__shfl_xor(acc, off, 64)"
    if acc_dt in ("u1", "b1"):
        shfl = f"({ct})__shfl_xor((int)acc, off, 64)"
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    const int sub = threadIdx.x & {G - 1};",
         f"    const int grp = (threadIdx.x & {WAVE - 1}) >> {G.bit_length() - 1};",
         f"    const long long stride = (long long)gridDim.x * {BLOCK // WAVE * per_wave};",
         f"    for (long long first = ((long long)blockIdx.x * {BLOCK // WAVE} + (threadIdx.x >> 6)) * "
         f"{per_wave}; first < K; first += stride) {{",
         "        const long long row = first + grp;",
         "        const long long k = row < K ? row : K - 1;      // idle groups re-read the last row"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            L.append(f"        const {CTYPE[dt]}* row{i} = a{i} + {_row_at(outer2, i, 'k')};")
        else:
            L.append(f"        const {CTYPE[dt]} c{i} = a{i}[{_row_at(outer2, i, 'k')}];")
    L.append(f"        {ct} acc = {_identity(op, acc_dt)};")

    def element(args, pad):
        return (f"{pad}{{ {ct} t0; dr_body({', '.join(args + call_tail)}); "
                f"acc = {_combine(op, 'acc', 't0')}; }}")

    full = R // V                          # units that are whole
    for j in range(steps):
        lo = j * G                         # this step covers units lo .. lo + G - 1
        if lo + G <= full:
            cond, pad = None, "        "
        else:
            cond, pad = f"        if ({lo} + sub < {full}) {{", "            "
        if lo < full:
            if cond:
                L.append(cond)
            for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
                if kind == "v":
                    vt = (VEC16[dt][0] + "u") if V > 1 else CTYPE[dt]
                    L.append(f"{pad}const {vt} X{j}_{i} = *(const {vt}*)(row{i} + ({lo} + sub) * {V});")
            for e in range(V):
                L.append(element([(f"X{j}_{i}[{e}]" if V > 1 else f"X{j}_{i}") if kind == "v" else f"c{i}"
                                  for i, kind in enumerate(leaf_kind)], pad))
            if cond:
                L.append("        }")
        if full * V < R and lo <= full < lo + G:
            # the partial unit at the end of the row: its lane takes the elements one by one
            L.append(f"        if (sub == {full - lo}) {{")
            for r in range(full * V, R):
                L.append(element([f"row{i}[{r}]" if kind == "v" else f"c{i}"
                                  for i, kind in enumerate(leaf_kind)], "            "))
            L.append("        }")
    L += ["#pragma unroll",
          f"        for (int off = {G // 2}; off > 0; off >>= 1) {{",
          f"            const {ct} other = {shfl};",
          f"            acc = {_combine(op, 'acc', 'other')};",
          "        }",
          "        if (sub == 0 && row < K) out[row] = acc;",
          "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_col_stream(prog, leaf_kind, acc_dt, op, unroll=8, outer=False, stagger=True):
    """Reduction over the rows of a matrix whose kept dimension has unit stride: a block owns
    256 x V adjacent columns (V the elements of a 16-byte vector: 4 KB of every row) and a
    slice of rows, and walks the rows with `unroll` loads in flight per lane; every lane
    keeps its own V columns, so nothing is combined inside the block.  Blocks with adjacent
    column tiles are adjacent in launch order: together they read whole rows.

    leaf_kind  per leaf 'v' (unit stride along the kept dimension) or 'k' (constant along it)
    stagger    every block starts its walk at a different row of its slice and wraps round:
               slices whose first rows lie a power of two apart (8 x 8192 x 2048 float32
               summed over the middle axis) otherwise march over the same memory channels
               in step (measured 60 % of the HBM peak in step, 82 % staggered)
    outer      a second, outer kept dimension (the middle axis of a 3-D array reduced): its
               index is part of the block number, column tiles stay inside one row
    Parameters: leaf pointers, output pointer, scalars, K, R, S, RS, then per leaf the
    stride between rows (elements); with `outer` its extent KO and every leaf's stride
    along it follow.  Output layout [slice][outer][column]."""
    ct = CTYPE[acc_dt]
    nl = len(prog.leaves)
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    V = 16 // widths.pop()
    TK = BLOCK * V
    src = [PREAMBLE, emit_body(prog, [acc_dt])]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const long long K", "const long long R", "const long long S", "const long long RS"]
    params += [f"const long long sr{i}" for i in range(nl)]
    if outer:
        params.append("const long long KO")
        params += [f"const long long sko{i}" for i in range(nl)]
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    ident = _identity(op, acc_dt)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    const long long ktiles = (K + {TK - 1}) / {TK};"]
    if outer:
        L += ["    for (long long b = blockIdx.x; b < ktiles * KO * S; b += gridDim.x) {",
              "        const long long sl = b / (ktiles * KO);",
              "        const long long ko = (b - sl * ktiles * KO) / ktiles;",
              "        const long long kt = b - (sl * KO + ko) * ktiles;"]
        L += [f"        const {CTYPE[dt]}* A{i} = a{i} + ko * sko{i};" for i, dt in enumerate(prog.leaves)]
        L.append(f"        {ct}* O = out + (sl * KO + ko) * K;")
    else:
        L += ["    for (long long b = blockIdx.x; b < ktiles * S; b += gridDim.x) {",
              "        const long long sl = b / ktiles;",
              "        const long long kt = b - sl * ktiles;"]
        L += [f"        const {CTYPE[dt]}* A{i} = a{i};" for i, dt in enumerate(prog.leaves)]
        L.append(f"        {ct}* O = out + sl * K;")
    L += [f"        const long long g = kt * {TK} + (long long)threadIdx.x * {V};",
         "        const long long r_end = (sl + 1) * RS < R ? (sl + 1) * RS : R;",
         f"        const long long r_mid = sl * RS + {'(b * 37) % (r_end - sl * RS)' if stagger else '0'};",
         f"        {ct} acc[{V}];",
         "#pragma unroll",
         f"        for (int e = 0; e < {V}; ++e) acc[e] = {ident};",
         f"        if (g + {V} <= K) {{",
         "          for (int half = 0; half < 2; ++half) {",
         "            const long long ra = half ? sl * RS : r_mid, rb = half ? r_mid : r_end;",
         f"#pragma unroll {unroll}",
         "            for (long long r = ra; r < rb; ++r) {"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            vt = VEC16[dt][0] + "u"
            L.append(f"                const {vt} X{i} = __builtin_nontemporal_load((const {vt}*)(A{i} + g + r * sr{i}));")
        else:
            L.append(f"                const {CTYPE[dt]} c{i} = A{i}[r * sr{i}];")
    for e in range(V):
        vargs = [f"X{i}[{e}]" if kind == "v" else f"c{i}" for i, kind in enumerate(leaf_kind)]
        L.append(f"                {{ {ct} t0; dr_body({', '.join(vargs + call_tail)}); "
                 f"acc[{e}] = {_combine(op, f'acc[{e}]', 't0')}; }}")
    sargs = [f"A{i}[g + e + r * sr{i}]" if kind == "v" else f"A{i}[r * sr{i}]"
             for i, kind in enumerate(leaf_kind)]
    L += ["            }",
          "          }",
          "        } else if (g < K) {          // the vector that straddles the last column",
          "            for (long long r = sl * RS; r < r_end; ++r) {",
          "#pragma unroll",
          f"                for (int e = 0; e < {V}; ++e) {{",
          "                    if (g + e < K) {",
          f"                        {ct} t0; dr_body({', '.join(sargs + call_tail)});",
          f"                        acc[e] = {_combine(op, 'acc[e]', 't0')};",
          "                    }",
          "                }",
          "            }",
          "        }",
          "#pragma unroll",
          f"        for (int e = 0; e < {V}; ++e)",
          "            if (g + e < K) O[g + e] = acc[e];",
          "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_block_rows(prog, leaf_kind, acc_dt, op, unroll=4, outer=False, shared=(), outer2=False):
    """Reduction over a long unit-stride last dimension: a block per (row, slice) streams
    its stretch of the row like a flat reduction (256 lanes x 16 bytes x `unroll` per step,
    one accumulator per vector element), combines through `dr_block_reduce` and writes one
    value.  A wave per row reads 256 bytes per instruction and keeps far fewer bytes in
    flight (sum over axis 1 of 16384^2 float32: 74 % of the HBM peak against the 87 % of a
    flat reduction).

    leaf_kind  per leaf 'v' (unit stride along the row) or 'k' (constant along it)
    outer      a second, outer reduced dimension (sum over the first and last axis of a
               3-D array): a block then takes whole rows, a slice of the outer range
    shared     indices of 'v' leaves that every row reads again (the vector of a
               matrix-vector product): cached loads; the others are read once and
               non-temporal
    Parameters: leaf pointers, output pointer, scalars, K, R, S, RS, then per leaf the
    stride between rows (elements); with `outer` R is the row length, S and RS cut the
    outer extent RO, and RO and every leaf's outer stride follow.  Output layout
    [row][slice]."""
    ct = CTYPE[acc_dt]
    nl = len(prog.leaves)
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    V = 16 // widths.pop()
    src = [PREAMBLE, emit_body(prog, [acc_dt]), emit_block_reduce(op, acc_dt)]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const long long K", "const long long R", "const long long S", "const long long RS"]
    params += [f"const long long sk{i}" for i in range(nl)]
    if outer:
        params.append("const long long RO")
        params += [f"const long long so{i}" for i in range(nl)]
    if outer2:
        assert not outer
        params.append("const unsigned int K1")
        params += [f"const long long sj{i}" for i in range(nl)]
        src.append(ROW_AT)
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    ident = _identity(op, acc_dt)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         "    for (long long o = blockIdx.x; o < K * S; o += gridDim.x) {",
         "        const long long k = o / S;",
         "        const long long sl = o - k * S;",
         f"        {ct} acc[{V}];",
         "#pragma unroll",
         f"        for (int e = 0; e < {V}; ++e) acc[e] = {ident};"]
    if outer:
        L += ["        const long long q_end = (sl + 1) * RS < RO ? (sl + 1) * RS : RO;",
              "        const long long r_end = R;",
              f"#pragma unroll {unroll}",
              "        for (long long q = sl * RS; q < q_end; ++q) {"]
        base = lambda i: f"a{i} + k * sk{i} + q * so{i}"
        const = lambda i: f"a{i}[k * sk{i} + q * so{i}]"
        first, pad = f"(long long)threadIdx.x * {V}", "    "
    else:
        L.append("        const long long r_end = (sl + 1) * RS < R ? (sl + 1) * RS : R;")
        base = lambda i: f"a{i} + {_row_at(outer2, i, 'k')}"
        const = lambda i: f"a{i}[{_row_at(outer2, i, 'k')}]"
        first, pad = f"sl * RS + (long long)threadIdx.x * {V}", ""
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            L.append(f"{pad}        const {CTYPE[dt]}* row{i} = {base(i)};")
        else:
            L.append(f"{pad}        const {CTYPE[dt]} c{i} = {const(i)};")
    L += [f"{pad}        long long r = {first};",
          f"#pragma unroll {1 if outer else unroll}",
          f"{pad}        for (; r + {V} <= r_end; r += {BLOCK * V}) {{"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            vt = VEC16[dt][0] + "u"
            ptr = f"(const {vt}*)(row{i} + r)"
            L.append(f"{pad}            const {vt} X{i} = {_ld(i not in shared, ptr)};")
    for e in range(V):
        vargs = [f"X{i}[{e}]" if kind == "v" else f"c{i}" for i, kind in enumerate(leaf_kind)]
        L.append(f"{pad}            {{ {ct} t0; dr_body({', '.join(vargs + call_tail)}); "
                 f"acc[{e}] = {_combine(op, f'acc[{e}]', 't0')}; }}")
    L.append(f"{pad}        }}")
    # exactly one thread is left with r < r_end: the one whose next vector would straddle
    # the end of the stretch; it takes those elements one by one
    sargs = [f"row{i}[r]" if kind == "v" else f"c{i}" for i, kind in enumerate(leaf_kind)]
    L += [f"{pad}        for (; r < r_end; ++r) {{",
          f"{pad}            {ct} t0; dr_body({', '.join(sargs + call_tail)});",
          f"{pad}            acc[0] = {_combine(op, 'acc[0]', 't0')};",
          f"{pad}        }}"]
    if outer:
        L.append("        }")
    accs = [f"acc[{e}]" for e in range(V)]
    while len(accs) > 1:
        accs = [f"({_combine(op, accs[i], accs[i + 1])})" if i + 1 < len(accs) else accs[i]
                for i in range(0, len(accs), 2)]
    L += [f"        {ct} total = dr_block_reduce({accs[0]});",
          "        if (threadIdx.x == 0) out[o] = total;",
          "        __syncthreads();          // the block reduction's LDS words are reused",
          "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_block_rows_shared(prog, leaf_kind, acc_dt, op, shared, rows=4, unroll=2):
    """`emit_block_rows` for reductions in which some operand is the same for every row (the
    vector of a matrix-vector product): a block takes `rows` adjacent rows at once, loads
    the shared operands' vectors once per step and uses them for all of them, so a step
    issues rows + 1 loads for rows x V elements instead of 2 x rows.  Every row is summed
    in the order `emit_block_rows` uses, so the results are the same to the bit.

    leaf_kind  per leaf 'v' (unit stride along the row) or 'k' (constant along it)
    shared     indices of the 'v' leaves every row reads again (cached loads; the others
               are read once and non-temporal)
    Parameters: leaf pointers, output pointer, scalars, K (rows), R (row length), then per
    leaf the stride between rows (elements).  One output per row."""
    ct = CTYPE[acc_dt]
    nl = len(prog.leaves)
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    V = 16 // widths.pop()
    src = [PREAMBLE, emit_body(prog, [acc_dt]), emit_block_reduce(op, acc_dt)]
    params = [f"const {CTYPE[dt]}* __restrict__ a{i}" for i, dt in enumerate(prog.leaves)]
    params.append(f"{ct}* __restrict__ out")
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const long long K", "const long long R"]
    params += [f"const long long sk{i}" for i in range(nl)]
    call_tail = [f"s{i}" for i in range(len(prog.scalars))] + ["t0"]
    ident = _identity(op, acc_dt)
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    for (long long k0 = (long long)blockIdx.x * {rows}; k0 < K; k0 += (long long)gridDim.x * {rows}) {{",
         f"        {ct} acc[{rows}][{V}];",
         "#pragma unroll",
         f"        for (int j = 0; j < {rows}; ++j)",
         "#pragma unroll",
         f"            for (int e = 0; e < {V}; ++e) acc[j][e] = {ident};"]
    for j in range(rows):
        L.append(f"        const long long kr{j} = k0 + {j} < K ? k0 + {j} : K - 1;   // past the end: the last row again, not stored")
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v" and i in shared:
            continue
        for j in range(rows):
            if kind == "v":
                L.append(f"        const {CTYPE[dt]}* row{i}_{j} = a{i} + kr{j} * sk{i};")
            else:
                L.append(f"        const {CTYPE[dt]} c{i}_{j} = a{i}[kr{j} * sk{i}];")
    L += [f"        long long r = (long long)threadIdx.x * {V};",
          f"#pragma unroll {unroll}",
          f"        for (; r + {V} <= R; r += {BLOCK * V}) {{"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind != "v":
            continue
        vt = VEC16[dt][0] + "u"
        if i in shared:
            L.append(f"            const {vt} X{i} = *((const {vt}*)(a{i} + r));")
        else:
            for j in range(rows):
                L.append(f"            const {vt} X{i}_{j} = __builtin_nontemporal_load((const {vt}*)(row{i}_{j} + r));")

    def arg(i, kind, j, e):
        if kind == "v":
            return f"X{i}[{e}]" if i in shared else f"X{i}_{j}[{e}]"
        return f"c{i}_{j}"

    for j in range(rows):
        for e in range(V):
            vargs = [arg(i, kind, j, e) for i, kind in enumerate(leaf_kind)]
            L.append(f"            {{ {ct} t0; dr_body({', '.join(vargs + call_tail)}); "
                     f"acc[{j}][{e}] = {_combine(op, f'acc[{j}][{e}]', 't0')}; }}")
    L.append("        }")
    # the one thread whose next vector would straddle the end of the row takes the rest of
    # it element by element
    L.append("        for (; r < R; ++r) {")
    for j in range(rows):
        sargs = [(f"a{i}[r]" if i in shared else f"row{i}_{j}[r]") if kind == "v" else f"c{i}_{j}"
                 for i, kind in enumerate(leaf_kind)]
        L.append(f"            {{ {ct} t0; dr_body({', '.join(sargs + call_tail)}); "
                 f"acc[{j}][0] = {_combine(op, f'acc[{j}][0]', 't0')}; }}")
    L.append("        }")
    for j in range(rows):
        accs = [f"acc[{j}][{e}]" for e in range(V)]
        while len(accs) > 1:
            accs = [f"({_combine(op, accs[i], accs[i + 1])})" if i + 1 < len(accs) else accs[i]
                    for i in range(0, len(accs), 2)]
        L += [f"        {{ const {ct} total = dr_block_reduce({accs[0]});",
              f"          if (threadIdx.x == 0 && k0 + {j} < K) out[k0 + {j}] = total;",
              "          __syncthreads(); }"]
    L += ["    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


# ---- 2-D kernel with transposed operands ------------------------------------------

T_TILE = 64      # square tile edge: both the transposed read and the write coalesce


def emit_tile_transpose(prog, leaf_kind, out_dtypes, restrict=True, vec=0, nt_load=False,
                        nt_store=False, unaligned=False, tile=(T_TILE, T_TILE), nbatch=0):
    """2-D tiled kernel for expressions in which some operand is walked along the
    output's rows by its unit stride (a transposed view).

    leaf_kind  per leaf: ('t',) unit stride along output dimension 0: its tile (TR output
               rows x TC output columns, `tile`) is read along its own contiguous
               direction, TR elements at a time, into LDS and read back transposed
               (rows padded by one word, so neither side has bank conflicts); ('d',) unit stride along output dimension 1, read directly;
               ('b',) single element broadcast
    vec        0, or the number of elements in 16 bytes when every array has that
               element size, 16-byte aligned rows and row strides: tiles that lie
               wholly inside the output then move 16 bytes per lane on both sides
               (the transposition itself happens in LDS, one word at a time)
    nbatch     further output dimensions (every dimension but the two the tiles span): the
               matrices of a batch are transposed one after the other, a block's matrix
               comes from its index (`a.T` of a 3-D array is 1 batch dimension in the
               middle).
    Parameters: leaf pointers, output pointers, scalars, H, W, tiles_x, then per 't'
    leaf its stride along output columns, per 'd' leaf its row stride, per output its
    row stride, then per batch dimension its extent and the stride of every leaf and of
    every output along it."""
    rs = "__restrict__ " if restrict else ""
    n_out = len(out_dtypes)
    TR, TC = tile
    per_thread = TR * TC // BLOCK
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    sfx = "_" if nbatch else ""          # with a batch the kernel offsets the pointers first
    params = [f"const {CTYPE[dt]}* {rs}a{i}{sfx}" for i, dt in enumerate(prog.leaves)]
    params += [f"{CTYPE[dt]}* {rs}o{i}{sfx}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += ["const int H", "const int W", "const int tiles_x"]
    for i, k in enumerate(leaf_kind):
        if k[0] == "t":
            params.append(f"const long long cs{i}")
    for i, k in enumerate(leaf_kind):
        if k[0] == "d":
            params.append(f"const long long rs{i}")
    params += [f"const long long ors{o}" for o in range(n_out)]
    for d in range(nbatch):
        params.append(f"const long long bd{d}")
        params += [f"const long long bs{i}_{d}" for i in range(len(prog.leaves))]
        params += [f"const long long bos{o}_{d}" for o in range(n_out)]
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{"]
    for i, k in enumerate(leaf_kind):
        if k[0] == "t":
            L.append(f"    __shared__ {CTYPE[prog.leaves[i]]} tt{i}[{TC * (TR + 1)}];")
    blk = "blockIdx.x"
    if nbatch:
        L += [f"    const long long per_matrix = (long long)tiles_x * ((H + {TR - 1}) / {TR});",
              "    long long rem_b = blockIdx.x / per_matrix;",
              "    const int tile_id = (int)(blockIdx.x - rem_b * per_matrix);"]
        for i in range(len(prog.leaves)):
            L.append(f"    long long boff{i} = 0;")
        for o in range(n_out):
            L.append(f"    long long boo{o} = 0;")
        for d in reversed(range(nbatch)):
            L.append(f"    {{ const long long c = rem_b % bd{d}; rem_b /= bd{d};")
            L += [f"      boff{i} += c * bs{i}_{d};" for i in range(len(prog.leaves))]
            L += [f"      boo{o} += c * bos{o}_{d};" for o in range(n_out)]
            L.append("    }")
        L += [f"    const {CTYPE[dt]}* {rs}a{i} = a{i}_ + boff{i};" for i, dt in enumerate(prog.leaves)]
        L += [f"    {CTYPE[dt]}* {rs}o{o} = o{o}_ + boo{o};" for o, dt in enumerate(out_dtypes)]
        blk = "tile_id"
    # Diagonal order: blocks that run at the same time differ in both tile coordinates.
    # With row-major order they would share r0, and the transposed operand's tiles
    # (rows a power-of-two pitch apart) would all fall into the same few memory channels.
    L += [f"    const int band = {blk} / tiles_x;",
          f"    const int tx = {blk} - band * tiles_x;",
          f"    const int ty = (band + tx) % ((H + {TR - 1}) / {TR});",
          f"    const int r0 = ty * {TR};",
          f"    const int c0 = tx * {TC};"]
    if vec:
        V = vec
        vpr = TR // V                     # vectors per column of the tile (operand's rows)
        vpc = TC // V                     # vectors per row of the tile (output's rows)
        passes = TR * TC // V // BLOCK
        L += [f"    if (r0 + {TR} <= H && c0 + {TC} <= W) {{",
              "#pragma unroll",
              f"        for (int k = 0; k < {passes}; ++k) {{",
              f"            const int e = threadIdx.x + k * {BLOCK};",
              f"            const int lc = e / {vpr};",
              f"            const int vr = e - lc * {vpr};"]
        for i, k in enumerate(leaf_kind):
            if k[0] == "t":
                vt = VEC16[prog.leaves[i]][0] + ("u" if unaligned else "")
                ptr = f"(const {vt}*)(a{i} + (long long)(c0 + lc) * cs{i} + (r0 + vr * {V}))"
                L.append(f"            const {vt} w{i} = {_ld(nt_load, ptr)};")
                for q in range(V):
                    L.append(f"            tt{i}[lc * {TR + 1} + vr * {V} + {q}] = w{i}[{q}];")
        L += ["        }", "        __syncthreads();",
              "#pragma unroll",
              f"        for (int k = 0; k < {passes}; ++k) {{",
              f"            const int e = threadIdx.x + k * {BLOCK};",
              f"            const int lr = e / {vpc};",
              f"            const int vc = e - lr * {vpc};",
              "            const long long i = r0 + lr;",
              f"            const int j = c0 + vc * {V};"]
        for i, k in enumerate(leaf_kind):
            if k[0] == "d":
                vt = VEC16[prog.leaves[i]][0] + ("u" if unaligned else "")
                L.append(f"            const {vt} d{i} = "
                         f"{_ld(nt_load, f'(const {vt}*)(a{i} + i * rs{i} + j)')};")
        for o, dt in enumerate(out_dtypes):
            L.append(f"            {VEC16[dt][0]} R{o};")
        for q in range(V):
            vargs = []
            for i, k in enumerate(leaf_kind):
                if k[0] == "t":
                    vargs.append(f"tt{i}[(vc * {V} + {q}) * {TR + 1} + lr]")
                elif k[0] == "d":
                    vargs.append(f"d{i}[{q}]")
                else:
                    vargs.append(f"a{i}[0]")
            decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
            call = vargs + [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]
            sets = " ".join(f"R{o}[{q}] = t{o};" for o in range(n_out))
            L.append(f"            {{ {decl} dr_body({', '.join(call)}); {sets} }}")
        for o, dt in enumerate(out_dtypes):
            ovt = VEC16[dt][0] + ("u" if unaligned else "")
            L.append("            " + _st(nt_store, f"R{o}", f"({ovt}*)(o{o} + i * ors{o} + j)"))
        L += ["        }", "        return;", "    }"]
    L += [# transposed operands: consecutive threads walk output ROWS (their unit stride)
          "#pragma unroll",
          f"    for (int k = 0; k < {per_thread}; ++k) {{",
          f"        const int e = threadIdx.x + k * {BLOCK};",
          f"        const int lc = e / {TR};",
          f"        const int lr = e - lc * {TR};",
          "        if (r0 + lr < H && c0 + lc < W) {"]
    for i, k in enumerate(leaf_kind):
        if k[0] == "t":
            L.append(f"            tt{i}[lc * {TR + 1} + lr] = a{i}[(long long)(c0 + lc) * cs{i} + (r0 + lr)];")
    L += ["        }", "    }", "    __syncthreads();",
          "#pragma unroll",
          f"    for (int k = 0; k < {per_thread}; ++k) {{",
          f"        const int e = threadIdx.x + k * {BLOCK};",
          f"        const int lr = e / {TC};",
          f"        const int lc = e - lr * {TC};",
          "        const int i = r0 + lr;",
          "        const int j = c0 + lc;",
          "        if (i < H && j < W) {"]
    args = []
    for i, k in enumerate(leaf_kind):
        if k[0] == "t":
            args.append(f"tt{i}[lc * {TR + 1} + lr]")
        elif k[0] == "d":
            args.append(f"a{i}[(long long)i * rs{i} + j]")
        else:
            args.append(f"a{i}[0]")
    decl = " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes))
    call = args + [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]
    L.append(f"            {decl} dr_body({', '.join(call)});")
    for o in range(n_out):
        L.append(f"            o{o}[(long long)i * ors{o} + j] = t{o};")
    L += ["        }", "    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


def emit_thin_transpose(prog, leaf_kind, out_dtypes, short, short_rows, restrict=True):
    """Transposed operands in a matrix with one side of a few elements (`short`, a compile-time
    constant): points as rows of coordinates and the coordinate vectors.  No tile and no LDS: a
    lane takes one index of the long side and all `short` indices of the other.

    short_rows  the output has `short` rows (and the 't' operands rows of `short` contiguous
                elements): a lane reads those elements one after the other and stores one
                element into each output row, the wave's stores covering 256 contiguous bytes
                of it; otherwise the output has `short` columns: the lane reads one element of
                each of the operand's `short` rows (the wave 256 contiguous bytes) and stores
                its output row
    leaf_kind   per leaf ('t',) unit stride along the output's rows, ('d',) along its columns,
                ('b',) one element
    Parameters: leaf pointers, output pointers, scalars, n (the long extent), per 't' leaf its
    stride along output columns, per 'd' leaf its row stride, per output its row stride."""
    rs = "__restrict__ " if restrict else ""
    n_out = len(out_dtypes)
    src = [PREAMBLE, emit_body(prog, out_dtypes)]
    params = [f"const {CTYPE[dt]}* {rs}a{i}" for i, dt in enumerate(prog.leaves)]
    params += [f"{CTYPE[dt]}* {rs}o{i}" for i, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long n")
    params += [f"const long long cs{i}" for i, k in enumerate(leaf_kind) if k[0] == "t"]
    params += [f"const long long rs{i}" for i, k in enumerate(leaf_kind) if k[0] == "d"]
    params += [f"const long long ors{o}" for o in range(n_out)]
    L = [f'extern "C" __global__ __launch_bounds__({BLOCK})',
         f"void dr_kernel({', '.join(params)})", "{",
         f"    const long long i = (long long)blockIdx.x * {BLOCK} + threadIdx.x;",
         "    if (i >= n) return;"]
    # element (row, column) of the output: (r, i) with short rows, (i, r) with short columns
    row, col = ("r", "i") if short_rows else ("i", "r")
    for i, (dt, k) in enumerate(zip(prog.leaves, leaf_kind)):
        if k[0] == "b":
            L.append(f"    const {CTYPE[dt]} x{i} = a{i}[0];")
        else:
            L.append(f"    {CTYPE[dt]} x{i}[{short}];")
    L += ["#pragma unroll", f"    for (int r = 0; r < {short}; ++r) {{"]
    for i, k in enumerate(leaf_kind):
        if k[0] == "t":
            L.append(f"        x{i}[r] = a{i}[{col} * cs{i} + {row}];")
        elif k[0] == "d":
            L.append(f"        x{i}[r] = a{i}[{row} * rs{i} + {col}];")
    L += ["    }", "#pragma unroll", f"    for (int r = 0; r < {short}; ++r) {{"]
    args = [f"x{i}" if k[0] == "b" else f"x{i}[r]" for i, k in enumerate(leaf_kind)]
    args += [f"s{i}" for i in range(len(prog.scalars))] + [f"t{o}" for o in range(n_out)]
    L.append("        " + " ".join(f"{CTYPE[dt]} t{o};" for o, dt in enumerate(out_dtypes)))
    L.append(f"        dr_body({', '.join(args)});")
    for o in range(n_out):
        L.append(f"        o{o}[{row} * ors{o} + {col}] = t{o};")
    L += ["    }", "}"]
    src.append("\n".join(L))
    return "\n".join(src) + "\n"


# Rows counted over two levels, K = K0 * K1, that some operand does not walk as one sequence
# (a matrix repeated for every item of a batch): row k of operand i starts at
# (k / K1) * sk_i + (k % K1) * sj_i.  Kernels that take such rows have the parameters K1 and
# sj_i after their others.
ROW_AT = ("__device__ __forceinline__ long long dr_row_at(const long long k, const unsigned int K1, "
          "const long long s0, const long long s1)\n{\n"
          "    const unsigned int q = (unsigned int)k / K1;\n"
          "    return (long long)q * s0 + (long long)((unsigned int)k - q * K1) * s1;\n}")


def _row_at(outer2, i, k):
    return f"dr_row_at({k}, K1, sk{i}, sj{i})" if outer2 else f"{k} * sk{i}"


# ---- rows that are reduced and used again in one kernel -----------------------------

ROW_REDUCE = {"rowsum": "add", "rowmax": "maximum", "rowmin": "minimum"}
# 16-byte units a lane holds of one operand's row.  A block of 256 lanes takes rows of up to
# 64 KB; longer ones, up to 256 KB, a block of 512 lanes with up to 32 units each (rows of
# 128 KB: 16 units in 512 lanes move 71 % of the peak, 32 units in 256 lanes 68 %, with
# 150-165 registers; 1024 lanes leave each 128 registers and a layer normalisation of
# 50257 float32 then spills: 20 %).
ROW_STEPS_MAX = 16
ROW_STEPS_LONG = 32
ROW_BLOCKS = (256, 512)             # lanes of a block that holds one row


class RowFusionUnsupported(Exception):
    """The program or its operands do not fit the row kernel: the reductions inside the
    expression are evaluated on their own instead."""


def row_analysis(prog, leaf_kind):
    """Where each operation of a program with row reductions is computed.

    A row reduction (`rowsum`, `rowmax`, `rowmin` of a per-element value) yields one value
    per row.  level[i] counts the reductions on the longest path below operation i; a
    reduction whose operand has level s is made in stage s, after the stages before it.
    uniform[i]: the value is the same along a row.  Returns (level, uniform, stages) with
    stages[s] the reductions made in stage s."""
    level, uniform = [], []
    for name, _, _, args in prog.ops:
        lv, uni = 0, True
        for k, j in args:
            if k == "v":
                lv = max(lv, level[j])
                uni = uni and uniform[j]
            elif k == "l":
                uni = uni and leaf_kind[j] == "k"
        if name in ROW_REDUCE:
            if uni:
                raise RowFusionUnsupported("a reduction of a value that is constant along the row")
            lv, uni = lv + 1, True
        elif name in INDEX_OPS:
            raise RowFusionUnsupported("index-valued operands")
        level.append(lv)
        uniform.append(uni)
    stages = [[] for _ in range(max(level, default=0))]
    for i, (name, _, _, _) in enumerate(prog.ops):
        if name in ROW_REDUCE:
            stages[level[i] - 1].append(i)
    return level, uniform, stages


def _row_needed(prog, targets, held=None, pre=()):
    """Operations to compute for the values `targets` (refs), in order, the row
    reductions they read (those are handed in, not computed) and the leaves they read.
    `held` maps an operation to the leaf whose registers hold its value by now: such a
    value is read from that leaf's slot, and what it was computed from is not needed.
    `pre`: operations computed once per row beforehand, handed in like the reductions
    (a target is computed even when it is listed there)."""
    held = held or {}
    need, given = set(), set()
    leaves = {j for k, j in targets if k == "l"}
    stack = [j for k, j in targets if k == "v"]
    own = set(stack)
    while stack:
        i = stack.pop()
        if i in need or i in given:
            continue
        if prog.ops[i][0] in ROW_REDUCE or (i in pre and i not in own):
            given.add(i)
            continue
        if i in held:
            leaves.add(held[i])
            need.add(i)
            continue
        need.add(i)
        for k, j in prog.ops[i][3]:
            if k == "v":
                stack.append(j)
            elif k == "l":
                leaves.add(j)
    return sorted(need), sorted(given), leaves


def _row_function(prog, fname, targets, out_dtypes, held=None, pre=()):
    """Device function computing `targets` for one element (or one row, when every target
    is constant along the row): parameters are all leaf values, all scalars, the row
    reductions it reads, then one reference per target.  Returns (source, reductions read,
    leaves read)."""
    held = held or {}
    need, given, used = _row_needed(prog, targets, held, pre)
    params = [f"const {CTYPE[dt]} l{i}" for i, dt in enumerate(prog.leaves)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params += [f"const {CTYPE[prog.ops[i][2]]} v{i}" for i in given]
    params += [f"{CTYPE[dt]}& r{n}" for n, dt in enumerate(out_dtypes)]
    lines = [f"__device__ __forceinline__ void {fname}({', '.join(params)})", "{"]
    for i in need:
        if i in held:       # computed by an earlier stage and kept where its operand was
            lines.append(f"    const {CTYPE[prog.ops[i][2]]} v{i} = l{held[i]};")
        else:
            lines.append(_op_statement(prog, i))
    for n, ((k, j), dt) in enumerate(zip(targets, out_dtypes)):
        lines.append(f"    r{n} = {_conv(f'{k}{j}', prog.ref_dtype((k, j)), dt)};")
    lines.append("}")
    return "\n".join(lines), given, used


_ROW_CHEAP = frozenset(("add", "subtract", "multiply", "negative", "positive", "absolute", "fabs",
                        "maximum", "minimum", "fmax", "fmin", "cast", "copysign", "where", "square"))


def _row_carry(prog, need, later_targets, held, kept, uniform, pre=()):
    """Which value computed by this stage (operations `need`) to keep for the stages that
    follow, and where: (operation, leaf) or None.  A value qualifies when later stages read
    it, when it costs more than a few additions to compute again (an exponential, a
    quotient), and when there is an operand of its type that is held in registers and that
    the later stages read only through this value: its registers then hold the value
    instead.  softmax: exp(a - max) takes the place of a after the sum."""
    later_need, _, _ = _row_needed(prog, later_targets, held, pre)
    for v in sorted(set(need) & set(later_need), reverse=True):
        name, _, rdt, _ = prog.ops[v]
        if uniform[v] or v in held:
            continue
        # what computing v again would cost: the operations below it down to what is at hand
        below, _, leaves_of_v = _row_needed(prog, [("v", v)], held, pre)
        if all(prog.ops[i][0] in _ROW_CHEAP for i in below):
            continue
        for leaf in sorted(leaves_of_v & kept):
            if prog.leaves[leaf] != rdt or leaf in held.values():
                continue
            trial = dict(held)
            trial[v] = leaf
            _, _, still = _row_needed(prog, later_targets, trial, pre)
            # the leaf's slot may be read later only as the carried value
            reads_leaf_itself = any(
                ("l", leaf) in prog.ops[i][3]
                for i in _row_needed(prog, later_targets, trial, pre)[0] if i not in trial)
            if not reads_leaf_itself and not any(k == "l" and j == leaf for k, j in later_targets):
                return v, leaf
    return None


def row_vector(prog, leaf_kind, out_dtypes, out_uniform):
    """Elements per 16-byte unit, when everything that moves along the row has one item
    size (4 or 8 bytes); else 1."""
    widths = {ITEMSIZE[dt] for dt, k in zip(prog.leaves, leaf_kind) if k == "v"}
    widths |= {ITEMSIZE[dt] for dt, u in zip(out_dtypes, out_uniform) if not u}
    return 16 // widths.pop() if len(widths) == 1 and widths <= {4, 8} else 1


def emit_row_fused(prog, leaf_kind, out_dtypes, out_uniform, R, G, keep=None, nt_store=False,
                   fence=True, recompute=True, pipeline=True, carry_values=True, wave_map=False,
                   nt_load=False, hoist=True, outer2=False, restrict=True):
    """Rows that are reduced and used again: `a - max(a, axis=-1)`, softmax, the variance,
    layer normalisation.  A group of G lanes (1..64: part of a wave; 256 or 512: the block) owns a
    row of R elements (a compile-time constant, unit stride); lane j takes the 16-byte
    units j, j + G, ... of it.  An operand flagged in `keep` (default: all) has its share of
    the row in registers from one stage to the next, so the row is read from memory once;
    the others are loaded again by every stage that reads them (from the caches: operands
    that are the same for every row, rows that would not fit).  Stage s computes,
    per element, the operands of the reductions whose inputs depend on s earlier
    reductions (per-element values are computed again in every stage that needs them: no
    value is carried but the row itself), and the group combines them: butterfly of
    `__shfl_xor` inside the wave, then, for a block, the four waves' values through LDS
    (two slots in turn, so one barrier per reduction).  The last stage computes the roots
    and stores them; a root that is constant along the row is stored once per row.

    A value that a stage computes at some cost and later stages read (softmax's
    exponentials) takes the place of the operand it was computed from in those registers
    (`_row_carry`).
    `fence`: the compiler may not move instructions from one 16-byte unit's work to the
    next (left to itself it interleaves all sixteen units of a long row for the sake of
    instruction-level parallelism and needs 205 vector registers for a softmax of rows of
    16384, which leaves two waves per SIMD).

    leaf_kind    per leaf 'v' (unit stride along the row) or 'k' (constant along it)
    out_uniform  per root: one value per row
    Parameters: leaf pointers, output pointers, scalars, K (rows), per leaf the stride
    between rows, per output the stride between rows (all in elements)."""
    level, uniform, stages = row_analysis(prog, leaf_kind)
    V = row_vector(prog, leaf_kind, out_dtypes, out_uniform)
    units = -(-R // V)
    full, rem = R // V, R % V
    steps = -(-units // G)
    if steps > (ROW_STEPS_LONG if G > BLOCK else ROW_STEPS_MAX):
        raise RowFusionUnsupported("row too long")
    nl, ns, n_out = len(prog.leaves), len(prog.scalars), len(out_dtypes)
    block_row = G >= BLOCK
    B = G if block_row else BLOCK          # lanes of a block: 256, or 512 for one long row
    if B not in ROW_BLOCKS:
        raise RowFusionUnsupported("no such block")
    lanes = min(G, WAVE)
    per_wave = WAVE // lanes
    src = [PREAMBLE,
           mathlib.source(prog.own_math, soft_div=any(prog.ops[i][1] == "f8" and prog.ops[i][0] != "sqrt"
                                                      for i in prog.soft_div)),
           mathlib32.source(prog.own_math32, soft_div=any(prog.ops[i][1] == "f4" for i in prog.soft_div))]

    # one function per stage, one for the per-element roots, one for the per-row roots
    if keep is None:
        keep = [True] * nl
    kept = {i for i in range(nl) if keep[i] and leaf_kind[i] == "v"}
    elem_roots = [n for n in range(n_out) if not out_uniform[n]]
    row_roots = [n for n in range(n_out) if out_uniform[n]]
    final_targets = [prog.roots[n][0] for n in elem_roots]
    stage_targets = [[prog.ops[i][3][0] for i in reds] for reds in stages]
    # Values that are the same along a row and that per-element work reads (the mean
    # `sum / n`, `sqrt(var + eps)`, `log(sum)`) are computed once per row, as soon as the
    # reductions they depend on are made, and handed to the per-element functions like the
    # reductions themselves: left inside, the compiler computes them for every element (a
    # log-softmax of rows of 16384 issued 65 logarithms per lane for its 64 elements).
    pre = set()
    if hoist:
        for n, (name, _, _, args) in enumerate(prog.ops):
            if not uniform[n]:
                pre |= {j for k, j in args
                        if k == "v" and uniform[j] and prog.ops[j][0] not in ROW_REDUCE}
    pre_by_level = {}
    for i in sorted(pre):
        pre_by_level.setdefault(level[i], []).append(i)
    pre_fn = {}
    for lv, ops_lv in sorted(pre_by_level.items()):
        lower_pre = {i for i in pre if level[i] < lv}
        text, given, _ = _row_function(prog, f"dr_once{lv}", [("v", i) for i in ops_lv],
                                       [prog.ops[i][2] for i in ops_lv], pre=lower_pre)
        src.append(text)
        pre_fn[lv] = (ops_lv, given)
    stage_fn = []
    held = {}
    carried_leaves = set()
    for s, reds in enumerate(stages):
        targets = stage_targets[s]
        outs = [prog.ops[i][1] for i in reds]
        carry = None
        if carry_values:
            later = [t for ts in stage_targets[s + 1:] for t in ts] + final_targets
            need, _, _ = _row_needed(prog, targets, held, pre)
            carry = _row_carry(prog, need, later, held, kept, uniform, pre)
        if carry is not None:
            targets = targets + [("v", carry[0])]
            outs = outs + [prog.ops[carry[0]][2]]
        text, given, used = _row_function(prog, f"dr_stage{s}", targets, outs, held, pre)
        src.append(text)
        stage_fn.append((given, used, carry))
        if carry is not None:
            held[carry[0]] = carry[1]
            carried_leaves.add(carry[1])
    final_given = rowout_given = ()
    final_used = set()
    if elem_roots:
        text, final_given, final_used = _row_function(
            prog, "dr_final", final_targets, [out_dtypes[n] for n in elem_roots], held, pre)
        src.append(text)
    if row_roots:
        text, rowout_given, _ = _row_function(
            prog, "dr_rowout", [prog.roots[n][0] for n in row_roots], [out_dtypes[n] for n in row_roots])
        src.append(text)

    # combining a value over the group
    red_types = sorted({(ROW_REDUCE[prog.ops[i][0]], prog.ops[i][2]) for reds in stages for i in reds})
    n_red = sum(len(reds) for reds in stages)
    for op, dt in red_types:
        ct = CTYPE[dt]
        body = [f"__device__ __forceinline__ {ct} dr_group_{op}_{dt}({ct} v, {ct}* slot)", "{",
                "#pragma unroll",
                f"    for (int off = {lanes // 2}; off > 0; off >>= 1) {{",
                f"        const {ct} o = __shfl_xor(v, off, 64);",
                f"        v = {_combine(op, 'v', 'o')};",
                "    }"]
        if block_row:
            body += [f"    if ((threadIdx.x & {WAVE - 1}) == 0) slot[threadIdx.x >> 6] = v;",
                     "    __syncthreads();"]
            terms = [f"slot[{w}]" for w in range(B // WAVE)]
            if len(terms) == 4:
                terms = [f"({_combine(op, terms[t], terms[t + 1])})" for t in (0, 2)]
            level = 0
            while len(terms) > 2:       # the waves' values pairwise, in one order for every lane
                body += [f"    const {ct} w{level}_{t // 2} = {_combine(op, terms[t], terms[t + 1])};"
                         for t in range(0, len(terms), 2)]
                terms = [f"w{level}_{t}" for t in range(len(terms) // 2)]
                level += 1
            body.append(f"    v = {_combine(op, terms[0], terms[1])};")
        body.append("    return v;")
        body.append("}")
        src.append("\n".join(body))

    rq = "__restrict__ " if restrict else ""      # (not when a result is written over an operand)
    params = [f"const {CTYPE[dt]}* {rq}a{i}" for i, dt in enumerate(prog.leaves)]
    params += [f"{CTYPE[dt]}* {rq}o{n}" for n, dt in enumerate(out_dtypes)]
    params += [f"const {CTYPE[dt]} s{i}" for i, dt in enumerate(prog.scalars)]
    params.append("const long long K")
    params += [f"const long long sk{i}" for i in range(nl)]
    params += [f"const long long so{n}" for n in range(n_out)]
    if outer2:
        params.append("const unsigned int K1")
        params += [f"const long long sj{i}" for i in range(nl)]
        src.append(ROW_AT)

    def row_at(i, k):
        return _row_at(outer2, i, k)
    scal = [f"s{i}" for i in range(ns)]
    L = [f'extern "C" __global__ __launch_bounds__({B})',
         f"void dr_kernel({', '.join(params)})", "{"]
    def vtype(dt):
        return (VEC16[dt][0] + "u") if V > 1 else CTYPE[dt]

    # Which unit a lane takes in step j: `lo + sub`.  Lanes side by side over the whole
    # group (sub = lane, lo = j G), or, `wave_map`, every wave of the block its own quarter
    # of the row (sub = wave * quarter + lane, lo = 64 j): a wave then reads 16 KB of a
    # 64 KB row in sequence instead of sixteen pieces 4 KB apart, which the memory system
    # serves faster (copying rows of 64 KB: 75 % of the peak against 66 %; rows of 16 and
    # 32 KB: 74 against 76 % and 69 against 71 %).
    wave_map = bool(block_row and wave_map and steps > 1)
    seg = steps * WAVE
    step_units = WAVE if wave_map else G
    max_sub = (B // WAVE - 1) * seg + WAVE - 1 if wave_map else G - 1

    def holds(sub):
        """Whether some lane has this `sub`."""
        if sub < 0:
            return False
        return (sub % seg < WAVE and sub // seg < B // WAVE) if wave_map else sub < G

    # which lanes hold what in step j: whole units, the partial last unit, nothing
    def step_state(j):
        lo = j * step_units
        whole = "" if lo + max_sub < full else (f"{lo} + sub < {full}" if lo < full else None)
        part = f"sub == {full - lo}" if rem and holds(full - lo) else None
        return lo, whole, part

    def loads(j, pad, which, base="row", declare=True):
        """Loads of step j's units of the row operands in `which` from the rows at
        `base`<i>, into new variables or (`declare` False) into the ones at hand."""
        lo, whole, part = step_state(j)
        out = []
        for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
            if kind != "v" or i not in which:
                continue
            vt = vtype(dt)
            zero = "{0}" if V > 1 else "0"
            # a pointer that is the same for the wave plus a lane's unsigned 32-bit offset:
            # the load then takes its address from a scalar register pair and one vector
            # register, instead of a vector register pair per unit of the row
            # (an operand that stays in registers is read once: past the caches, `nt_load`)
            ld = _ld(nt_load and V > 1 and i in kept,
                     f"(const {vt}*)(({base}{i} + {lo * V}) + usub * {V}u)")
            if whole == "" and declare:
                const = "" if i in carried_leaves else "const "
                out.append(f"{pad}{const}{vt} X{j}_{i} = {ld};")
                continue
            if declare:
                out.append(f"{pad}{vt} X{j}_{i} = {zero};")
            if whole == "":
                out.append(f"{pad}X{j}_{i} = {ld};")
            elif whole is not None:
                out.append(f"{pad}if ({whole}) X{j}_{i} = {ld};")
            if part is not None:
                fill = " ".join(f"X{j}_{i}[{e}] = {base}{i}[{full * V + e}];" for e in range(rem))
                out.append(f"{pad}if ({part}) {{ {fill} }}")
        return out

    def row_pointers(pad, k, base="row", which=None):
        out = []
        for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
            if kind == "v" and (which is None or i in which):
                out.append(f"{pad}const {CTYPE[dt]}* {base}{i} = a{i} + {row_at(i, k)};")
        return out

    # Rows in turn: the registers that hold a row are filled for the next row as soon as
    # the last stage has used them, so the next row is on its way while this one is
    # finished and stored (`rotate`; the first row is loaded ahead of the loop).
    # (not when the last stage also loads operands that are not held: the wave would wait
    # for them behind the next row's loads, which return in order)
    unheld_in_final = {i for i in final_used if leaf_kind[i] == "v"} - kept
    rotate = bool(kept) and pipeline and not unheld_in_final
    if rotate:
        for j in range(steps):
            for i in sorted(kept):
                zero = "{0}" if V > 1 else "0"
                L.append(f"    {vtype(prog.leaves[i])} X{j}_{i} = {zero};")
    if block_row:
        widest = max((CTYPE[prog.ops[i][2]] for reds in stages for i in reds), default="float",
                     key=lambda c: 8 if c in ("double", "long long") else 4)
        L += [f"    __shared__ {widest} dr_slots[2][{max(n_red, 1)}][{B // WAVE}];",
              f"    const int sub = (threadIdx.x >> 6) * {seg} + (threadIdx.x & {WAVE - 1});" if wave_map
              else "    const int sub = threadIdx.x;",
              "    const unsigned int usub = sub;",
              "    int turn = 0;"]
        if rotate:
            L.append("    if (blockIdx.x < K) {")
            L += row_pointers("        ", "(long long)blockIdx.x", which=kept)
            for j in range(steps):
                L += loads(j, "        ", kept, declare=False)
            L.append("    }")
        L += ["    for (long long row = blockIdx.x; row < K; row += gridDim.x, turn ^= 1) {",
              "        const long long k = row;"]
        if rotate:
            L += ["        const bool more = row + gridDim.x < K;",
                  "        const long long nk = more ? row + gridDim.x : row;"]
    else:
        L += [f"    const int sub = threadIdx.x & {G - 1};",
              f"    const unsigned int usub = threadIdx.x & {G - 1};",
              f"    const int grp = (threadIdx.x & {WAVE - 1}) >> {G.bit_length() - 1};",
              f"    const long long stride = (long long)gridDim.x * {BLOCK // WAVE * per_wave};",
              f"    const long long start = ((long long)blockIdx.x * {BLOCK // WAVE} + (threadIdx.x >> 6)) * "
              f"{per_wave};"]
        if rotate:
            L.append("    if (start < K) {")
            L.append("        const long long k0 = start + grp < K ? start + grp : K - 1;")
            L += row_pointers("        ", "k0", which=kept)
            for j in range(steps):
                L += loads(j, "        ", kept, declare=False)
            L.append("    }")
        L += ["    for (long long first = start; first < K; first += stride) {",
              "        const long long row = first + grp;",
              "        const long long k = row < K ? row : K - 1;      // idle groups re-read the last row"]
        if rotate:
            L += ["        const bool more = first + stride < K;",
                  "        const long long nk = more ? (first + stride + grp < K ? first + stride + grp : K - 1) : k;"]
    for i, (dt, kind) in enumerate(zip(prog.leaves, leaf_kind)):
        if kind == "v":
            L.append(f"        const {CTYPE[dt]}* row{i} = a{i} + {row_at(i, 'k')};")
        else:
            L.append(f"        const {CTYPE[dt]} c{i} = a{i}[{row_at(i, 'k')}];")
    if rotate:
        L += row_pointers("        ", "nk", base="nrow", which=kept)

    def once(lv, pad):
        """The per-row values of level lv: computed by every lane (all get the same)."""
        if lv not in pre_fn:
            return []
        ops_lv, given = pre_fn[lv]
        args = [("0" if kind == "v" else f"c{i}") for i, kind in enumerate(leaf_kind)]
        args += [f"s{i}" for i in range(ns)] + [f"v{g}" for g in given] + [f"v{i}" for i in ops_lv]
        return [f"{pad}{CTYPE[prog.ops[i][2]]} v{i};" for i in ops_lv] + \
               [f"{pad}dr_once{lv}({', '.join(args)});"]
    L += once(0, "        ")

    def next_loads(j, pad):
        """The next row's units of step j, into the registers that step j has just used."""
        if not rotate:
            return []
        inner = loads(j, pad + "    ", kept, base="nrow", declare=False)
        return [f"{pad}if (more) {{"] + inner + [f"{pad}}}"] if inner else []

    def element_args(j, e, used):
        """Arguments for the leaves: an operand that the function does not read is a zero."""
        return [(("0" if i not in used else f"X{j}_{i}[{e}]" if V > 1 else f"X{j}_{i}")
                 if kind == "v" else f"c{i}") for i, kind in enumerate(leaf_kind)]

    def guarded(j, e, stmt, pad):
        """`stmt` for element e of step j, under the condition that the lane holds it."""
        lo, whole, part = step_state(j)
        conds = []
        if whole == "":
            return f"{pad}{stmt}"
        if whole is not None:
            conds.append(f"({whole})")
        if part is not None and e < rem:
            conds.append(f"({part})")
        if not conds:
            return None
        return f"{pad}if ({' || '.join(conds)}) {stmt}"

    pad = "        "

    def relabel(g, tag):
        """A copy of row value g that the compiler cannot tell is the same value: what one
        stage computed per element (`exp(x - max)` for the sum) is then not kept in
        registers for the next stage that computes it (for the quotient), but computed
        again; a row of 16384 held twice leaves two waves per SIMD."""
        if not recompute:
            return f"v{g}"
        ct = CTYPE[prog.ops[g][2]]
        if ITEMSIZE[prog.ops[g][2]] < 4:    # a byte (a mask) has no register class of its own
            L.append(f'{pad}{ct} v{g}_{tag}; {{ int w_ = v{g}; asm volatile("" : "+v"(w_)); '
                     f'v{g}_{tag} = ({ct})w_; }}')
        else:
            L.append(f'{pad}{ct} v{g}_{tag} = v{g}; asm volatile("" : "+v"(v{g}_{tag}));')
        return f"v{g}_{tag}"
    if not rotate:
        for j in range(steps):
            L += loads(j, pad, kept)
    slot = 0
    for s, reds in enumerate(stages):
        for i in reds:
            op, dt = ROW_REDUCE[prog.ops[i][0]], prog.ops[i][2]
            L.append(f"{pad}{CTYPE[dt]} acc{i} = {_identity(op, dt)};")
        given = []
        for g in stage_fn[s][0]:
            given.append(relabel(g, f"s{s}"))
        used = stage_fn[s][1]
        carry = stage_fn[s][2]
        again = {i for i in used if leaf_kind[i] == "v"} - kept
        outs = [f"t{i}" for i in reds]
        decl = " ".join(f"{CTYPE[prog.ops[i][1]]} t{i};" for i in reds)
        if carry is not None:
            outs.append("tc")
            decl += f" {CTYPE[prog.ops[carry[0]][2]]} tc;"
        for j in range(steps):
            body = []
            for e in range(V):
                acc = " ".join(f"acc{i} = {_combine(ROW_REDUCE[prog.ops[i][0]], f'acc{i}', f't{i}')};"
                               for i in reds)
                if carry is not None:       # the value takes its operand's place in the registers
                    acc += f" X{j}_{carry[1]}{f'[{e}]' if V > 1 else ''} = tc;"
                stmt = (f"{{ {decl} dr_stage{s}({', '.join(element_args(j, e, used) + scal + given + outs)}); "
                        f"{acc} }}")
                line = guarded(j, e, stmt, pad + ("    " if again else ""))
                if line:
                    body.append(line)
            if not body:
                continue
            if not again:
                L += body
            else:
                L += [f"{pad}{{"] + loads(j, pad + "    ", again) + body + [f"{pad}}}"]
            if fence and j + 1 < steps:
                L.append(f"{pad}__builtin_amdgcn_sched_barrier(0);")
        for i in reds:
            op, dt = ROW_REDUCE[prog.ops[i][0]], prog.ops[i][2]
            where = f"({CTYPE[dt]}*)dr_slots[turn][{slot}]" if block_row else "nullptr"
            L.append(f"{pad}const {CTYPE[dt]} v{i} = dr_group_{op}_{dt}(acc{i}, {where});")
            slot += 1
        L += once(s + 1, pad)
    # the roots
    store_guard = "" if block_row else "if (row < K) "
    if elem_roots:
        given = [relabel(g, "f") for g in final_given]
        for j in range(steps):
            lo, whole, part = step_state(j)
            if whole is None and part is None:
                continue
            inner = pad + "    "
            L.append(f"{pad}{{")
            L += loads(j, inner, {i for i in final_used if leaf_kind[i] == "v"} - kept)
            for n in elem_roots:
                L.append(f"{inner}{vtype(out_dtypes[n])} Y{n};")
            for e in range(V):
                outs = [(f"Y{n}[{e}]" if V > 1 else f"Y{n}") for n in elem_roots]
                # vector components cannot bind to references: through temporaries
                tmps = [f"y{n}" for n in elem_roots]
                decl = " ".join(f"{CTYPE[out_dtypes[n]]} y{n};" for n in elem_roots)
                copy = " ".join(f"{o} = {t};" for o, t in zip(outs, tmps))
                stmt = (f"{{ {decl} dr_final({', '.join(element_args(j, e, final_used) + scal + given + tmps)}); "
                        f"{copy} }}")
                line = guarded(j, e, stmt, inner)
                if line:
                    L.append(line)
            for n in elem_roots:
                dt = out_dtypes[n]
                base = f"o{n} + row * so{n}"
                st = _st(nt_store and V > 1, f"Y{n}", f"({vtype(dt)}*)(({base} + {lo * V}) + usub * {V}u)")
                if whole == "":
                    L.append(f"{inner}{store_guard}{st}")
                elif whole is not None:
                    cond = f"{whole}" if block_row else f"row < K && {whole}"
                    L.append(f"{inner}if ({cond}) {st}")
                if part is not None:
                    tail = " ".join(f"({base})[{full * V + e}] = Y{n}[{e}];" for e in range(rem))
                    cond = f"{part}" if block_row else f"row < K && {part}"
                    L.append(f"{inner}if ({cond}) {{ {tail} }}")
            L += next_loads(j, inner)
            L.append(f"{pad}}}")
            if fence and j + 1 < steps:
                L.append(f"{pad}__builtin_amdgcn_sched_barrier(0);")
    elif rotate:
        for j in range(steps):
            L += next_loads(j, pad)
    if row_roots:
        given = [f"v{g}" for g in rowout_given]
        outs = [f"z{n}" for n in row_roots]
        decl = " ".join(f"{CTYPE[out_dtypes[n]]} z{n};" for n in row_roots)
        # per-row values read no row operand: hand the function zeros for those
        args = [("0" if kind == "v" else f"c{i}") for i, kind in enumerate(leaf_kind)]
        cond = "sub == 0" if block_row else "sub == 0 && row < K"
        stores = " ".join(f"o{n}[row * so{n}] = z{n};" for n in row_roots)
        L.append(f"{pad}if ({cond}) {{ {decl} dr_rowout({', '.join(args + scal + given + outs)}); {stores} }}")
    L += ["    }", "}"]
    src.append("\n".join(L))
    return "\n".join(p for p in src if p) + "\n"
