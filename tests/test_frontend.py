"""Host logic of the lazy front end and of the code generator; no GPU needed.

Leaves are placeholder device arrays (geometry and dtype, no memory), so DAG
construction, tracing, lowering, source generation and hiprtc compilation are all
exercised here; nothing is launched.
"""
import ctypes
import os
import re

import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import codegen as cg
from delayrepay_amd import hip, hiprt, lowering, mathlib, mathlib32
from delayrepay_amd.delayarray import (BinaryFuncEx, BinaryNumpyEx, CastEx, FullEx, IotaEx, NPArray,
                                       ReduceEx, Scalar, UnaryFuncEx, Memoiser)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def leaf(shape, dtype=np.float32, **kw):
    return NPArray(hip.placeholder(shape, dtype, **kw))


# ---- C ABI ---------------------------------------------------------------------

def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "drhip.h")).read()
    declared = set(re.findall(r"\b(drhip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    lib = ctypes.CDLL(hiprt.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in drhip.h but not exported"
    assert declared == set(hiprt._SIGNATURES), "ctypes binding and header disagree"


def test_uninitialised_library_reports_errors_without_a_gpu():
    lib = hiprt.lib()
    p = ctypes.c_void_p()
    if not hiprt._initialised:
        assert lib.drhip_malloc(ctypes.byref(p), 1024) == 20001       # DRHIP_ENOTINIT
        assert b"drhip_init" in lib.drhip_last_error()
    assert lib.drhip_compile(None, b"x", None, 0, None) == 20002      # DRHIP_EINVAL


def test_compile_error_carries_the_hiprtc_log():
    with pytest.raises(hiprt.DrhipError) as err:
        hiprt.compile_only('extern "C" __global__ void k() { this is not C++; }', "bad.hip", [])
    assert err.value.code > 10000
    assert "error" in err.value.log


# ---- laziness and hash-consing (reference tests/test.py:145-162) -------------------

def test_memoise_leaf_and_expression_identity():
    arr = hip.placeholder((3,), np.float64)
    assert NPArray(arr) is NPArray(arr)
    a = leaf((3,))
    b = leaf((3,))
    assert a is not b
    assert np.sin(a) is np.sin(a)
    assert (a + b) is (a + b)
    assert (a + b) is not (b + a)


def test_scalar_keys_do_not_collide():
    assert Scalar(-1) is not Scalar(-2)          # hash((-1,)) == hash((-2,)) in CPython
    assert Scalar(2) is not Scalar(2.0)
    assert Scalar(0.0) is not Scalar(-0.0)
    assert Scalar(2) is Scalar(2)
    a = leaf((4,))
    assert isinstance(a ** 2.0, BinaryFuncEx)    # float exponent stays pow()
    assert isinstance(a ** 2, BinaryNumpyEx)


def test_hash_cons_table_holds_nodes_weakly():
    import gc
    def interior():      # nodes for numbers stay alive for a while (a bounded number of them)
        return sum(1 for key in Memoiser._cache.data if key[0] is not Scalar)
    a = leaf((8,))
    before = interior()
    tmp = [a * float(i) for i in range(50)]
    assert interior() >= before + 50
    del tmp
    gc.collect()
    assert interior() <= before + 2
    # the numbers kept alive are bounded
    tmp = [a * float(i) for i in range(2000)]
    del tmp
    gc.collect()
    assert sum(1 for key in Memoiser._cache.data if key[0] is Scalar) <= 512 + 2


def test_nothing_is_computed_while_building():
    a, b = leaf((1 << 20,)), leaf((1 << 20,))
    before = dict(hip.STATS)
    z = np.sqrt(a * 2.0 + b) / 3
    assert "array" not in z.__dict__
    assert hip.STATS == before
    assert z.shape == (1 << 20,) and z.dtype == np.float32


def test_rewrites_follow_the_reference():
    a = leaf((16,))
    sq = np.square(a)                            # delayarray.py:330-331
    assert isinstance(sq, BinaryNumpyEx) and sq.func is np.multiply
    assert sq.children[0] is a and sq.children[1] is a
    cube = a ** 3                                # delayarray.py:316-324: (a*a)*a
    assert cube.func is np.multiply and cube.children[1] is a
    assert cube.children[0].children[0] is a and cube.children[0].children[1] is a
    assert (a ** 1) is a
    assert isinstance(np.cos(a), UnaryFuncEx)
    assert isinstance(np.arctan2(a, a), BinaryFuncEx)
    assert isinstance(a / 2, BinaryNumpyEx)      # NumPy 2 calls the ufunc `divide`
    assert isinstance((a + 1).astype(np.float64), CastEx)   # lazy nodes cast lazily
    assert (a + 1).astype(np.float32) is (a + 1)
    assert a.astype(np.float32) is a                         # same dtype: same leaf


def test_powers_below_one_follow_numpy_not_the_reference():
    a = leaf((16,))
    zero = a ** 0                                # the reference would hand back `a`
    assert zero is not a and isinstance(zero, BinaryFuncEx) and zero.func is np.power
    inv = a ** -1
    assert isinstance(inv, UnaryFuncEx) and inv.func is np.reciprocal
    assert isinstance(a ** -2, BinaryFuncEx)
    ints = leaf((16,), np.int32)
    with pytest.raises(ValueError, match="negative integer powers"):
        ints ** -1
    ones = ints ** 0
    assert ones is not ints and ones.dtype == np.int32
    low, src = hip.lower_only(ones)
    hip.compile_source(src)


def test_bool_arithmetic_is_logical():
    p, q = leaf((64,), np.bool_), leaf((64,), np.bool_)
    _, src = hip.lower_only(p + q)
    assert "l0 | l1" in src.replace("(", " ").replace(")", " ") or "|" in src
    _, src = hip.lower_only(p * q)
    assert "&" in src
    with pytest.raises(TypeError, match="boolean"):
        hip.lower_only(UnaryFuncEx(np.negative, p))
    with pytest.raises(TypeError):
        p - q                                    # NumPy itself refuses to type this


def test_dtype_and_shape_inference_is_numpys():
    f32, f64, i64 = leaf((4, 5)), leaf((4, 5), np.float64), leaf((4, 5), np.int64)
    assert (f32 * 0.3).dtype == np.float32                 # weak Python scalar
    assert (f32 * np.float64(0.3)).dtype == np.float64     # NumPy scalars are not weak
    assert (f32 + f64).dtype == np.float64
    assert (i64 * 2).dtype == np.int64
    assert (i64 * 2.0).dtype == np.float64
    assert (i64 / i64).dtype == np.float64
    assert np.sqrt(i64).dtype == np.float64
    assert (f32 > 0).dtype == np.bool_
    row = leaf((1, 5))
    col = leaf((4, 1))
    assert (row + col).shape == (4, 5)
    with pytest.raises(ValueError):
        leaf((3,)) + leaf((4,))


def test_unsupported_operands_raise():
    a = leaf((4,))
    with pytest.raises(NotImplementedError):
        a + "text"
    with pytest.raises(NotImplementedError):
        np.add(a, 1, where=np.array([True] * 4))


def test_inplace_operator_rebinds_like_the_reference():
    a = leaf((4,))
    b = a
    b += 1
    assert b is not a and isinstance(b, BinaryNumpyEx)


# ---- tracing ---------------------------------------------------------------------

def trace(ex):
    t = hip.Tracer()
    root = t.visit(ex)
    return t, t.program([root])


def test_shared_subexpression_is_traced_once():
    a, b = leaf((64,), np.float64), leaf((64,), np.float64)
    d = a - b
    t, prog = trace(d * d * b)                   # the sum-of-squares body
    assert [op[0] for op in prog.ops] == ["subtract", "multiply", "multiply"]
    assert prog.ops[1][3] == (("v", 0), ("v", 0))
    assert len(t.leaves) == 2


def test_program_is_structural():
    """Two instances of the same expression over different arrays and scalar values
    give the same cache key (the reference's names embed a global counter and
    always differ, delayarray.py:150-152)."""
    def build(c0, c1):
        x, y = leaf((128,)), leaf((128,))
        return hip.lower_only(c0 * x + y * c1)[0].key
    assert build(2.0, 3.0) == build(-7.5, 0.25)
    x = leaf((128,))
    assert hip.lower_only(2.0 * x)[0].key != hip.lower_only(2.0 * leaf((128,), np.float64))[0].key


def test_scalars_become_typed_parameters():
    x = leaf((256,))
    t, prog = trace(0.3 * x + 1)
    assert prog.scalars == ("f4", "f4")
    import struct
    assert struct.pack("f", t.scalars[0]) == np.float32(0.3).tobytes()    # rounded as NumPy does
    big = struct.pack("@f", hip._scalar_value(1e60, "f4"))    # overflow -> inf, like np.float32(1e60)
    assert np.frombuffer(big, np.float32)[0] == np.inf
    assert hip._scalar_value(3, "i8") == 3 and hip._scalar_value(2, "f8") == 2.0
    src = hip.lower_only(0.3 * x + 1)[1]
    assert "0.3" not in src                      # never an inlined (double) literal


def test_same_geometry_views_are_one_leaf():
    base = hip.placeholder((16, 16), np.float32)
    v1, v2 = NPArray(base[1:-1, 1:-1]), NPArray(base[1:-1, 1:-1])
    assert v1 is v2                              # two view objects, one geometry, one leaf
    assert NPArray(base[1:-1, 1:-1]) is not NPArray(base[1:-1, 2:])
    t, _ = trace(v1 + NPArray(base[1:-1, 1:-1]))
    assert len(t.leaves) == 1


# ---- lowering: which kernel shape, which key -------------------------------------------

def test_contiguous_is_flat_and_vectorised():
    x, y = leaf((1 << 16,)), leaf((1 << 16,))
    low, src = hip.lower_only(2.0 * x + y)
    assert low.kind == "flat"
    assert "f4x4" in src and "__builtin_nontemporal" not in src      # small: stays cacheable
    big = hip.lower_only(2.0 * leaf((1 << 26,)) + leaf((1 << 26,)))[1]
    assert "__builtin_nontemporal_load" in big and "__builtin_nontemporal_store" in big
    # 2-D contiguous operands collapse to the same flat kernel
    assert hip.lower_only(2.0 * leaf((256, 256)) + leaf((256, 256)))[0].key == low.key


def test_misaligned_view_moves_vectors_at_element_alignment():
    base = hip.placeholder((1 << 12,), np.float32)
    low, src = hip.lower_only(NPArray(base[1:]) * 2.0)
    kernel = src.split('extern "C"')[1]
    assert low.kind == "flat" and "f4x4*)" not in kernel and "(const f4x4u*)a0" in kernel
    assert hip._kernel_name(low).startswith("dr_flat_") and hip._kernel_name(low) in src
    aligned = hip.lower_only(NPArray(base[4:]) * 2.0)[1].split('extern "C"')[1]
    assert "(const f4x4*)a0" in aligned and "f4x4u" not in aligned
    # rows whose pitch is not a multiple of 16 bytes: vector tiles all the same
    m = NPArray(hip.placeholder((2046, 2046), np.float32, strides=(2048, 1), offset=2049))
    low, src = hip.lower_only(m * 2.0 + m)
    assert low.key[0] == "tile2dv" and "(const f4x4u*)(a0" in src and "(f4x4u*)(o0" in src
    hip.compile_source(src)
    hip.set_tune(uvec=0)
    try:
        low, src = hip.lower_only(NPArray(base[1:]) * 2.0)
        assert "f4x4u*)" not in src.split('extern "C"')[1]
    finally:
        hip.set_tune(uvec=1)


def test_broadcast_scalar_leaf_and_mixed_dtypes():
    x = leaf((1 << 12,), np.float32)
    s = leaf((), np.float64)
    low, src = hip.lower_only(x * s)
    assert low.kind == "flat" and "a1[0]" in src
    assert "(double)l0" in src
    hip.compile_source(src)


def test_strided_and_broadcast_operands_use_nd():
    a, b = leaf((64, 1, 1320), np.float64), leaf((1, 48, 1320), np.float32)
    low, src = hip.lower_only(a * b + 1)         # unit inner stride: tiled, rows = 64 * 48
    assert low.kind == "tile2d" and "rem_o / e1" in src
    hip.compile_source(src)
    col = leaf((64, 1))
    low, src = hip.lower_only(leaf((64, 1320)) * col)        # column broadcast: one load per row
    assert low.kind == "tile2d" and ("r",) in low.key[2]
    hip.compile_source(src)
    # rows of at most 4 KB: the row kernel, a group of lanes per row, also over two levels
    a, b = leaf((64, 1, 32), np.float64), leaf((1, 48, 32), np.float32)
    low, src = hip.lower_only(a * b + 1)
    assert low.kind == "rows" and "dr_row_at" in src and "dr_final" in src and "dr_stage" not in src
    hip.compile_source(src)
    low, src = hip.lower_only(leaf((1 << 20, 3)) * leaf((3,)) + leaf((1 << 20, 1)))
    assert low.kind == "rows" and low.key[6] == 1 and low.key[2] == ("v", "v", "k")
    hip.compile_source(src)
    lowering.TUNE["rows_elem"] = 0
    try:
        assert hip.lower_only(leaf((1 << 20, 5)) * leaf((5,)))[0].kind == "tile2d"
    finally:
        lowering.TUNE["rows_elem"] = 4096
    dst = hip.placeholder((64, 32), np.float32, strides=(64, 1))           # a destination with
    low, src = hip.lower_only(leaf((64, 32)) * col, dst=dst)               # its own pitch
    assert low.kind == "rows" and low.tail[:4] == [64, 32, 1, 64]
    hip.compile_source(src)
    dst3 = hip.placeholder((4, 16, 32), np.float32, strides=(2048, 64, 1))  # rows on two levels
    assert hip.lower_only(leaf((4, 16, 32)) * 2.0, dst=dst3)[0].kind == "tile2d"
    m = hip.placeholder((100, 200), np.float32)
    low, src = hip.lower_only(NPArray(m.T) * 2.0)           # transposed operand: through LDS
    assert low.kind == "tile2dt" and "__shared__ float tt0[" in src
    hip.compile_source(src)
    assert hip.lower_only(NPArray(m[::2, ::3]) * 2.0)[0].kind == "nd"


def test_views_without_shared_rows_stream_row_by_row():
    """No halo group: a block takes one stretch of one row (up to 1024 float32), the streams
    are non-temporal beyond the cache sizes, and the first and last column group of a row
    load whole vectors where the operand's buffer allows."""
    n = 16384
    m = NPArray(hip.placeholder((n, n), np.float32))
    low, src = hip.lower_only(m[1:-1, 1:-1] * 2.0)
    assert low.kind == "tile2d" and low.key[0] == "tile2dv"
    gpr, rpt, ntl, nts = low.key[8:12]
    assert (gpr, rpt, ntl, nts) == (256, 1, True, True)
    assert low.grid == 16 * (n - 2) and "lo0" in src and "__builtin_nontemporal_load" in src
    assert low.tail[-2:] == [-(n + 1), n * n - (n + 1)]
    hip.compile_source(src)
    u = NPArray(hip.placeholder((64, 64, 64), np.float32))       # short rows: 62 -> 16 groups
    dst = hip.placeholder((62, 62, 62), np.float32, strides=(4096, 64, 1), offset=4096 + 64 + 1)
    low, src = hip.lower_only(u[1:-1, 1:-1, 1:-1] * 2.0, dst=dst)
    assert low.key[8:10] == (16, 1) and "__builtin_nontemporal_load" not in src
    hip.compile_source(src)
    row = NPArray(hip.placeholder((n,), np.float32))             # repeats from row to row:
    low, src = hip.lower_only(m + row)                            # the taller tile shares it
    assert low.key[0] == "tile2dv" and low.key[8:10] == (64, 2)


def test_lowering_is_remembered_by_structure_and_geometry():
    """The same expression over fresh arrays of the same layout reuses the kernel choice,
    with the new buffers and scalar values filled in; another layout, alignment, buffer
    size, sharing of buffers or tunable is another entry."""
    def build(c, **kw):
        x, y = leaf((300, 1000), **kw), leaf((300, 1000))
        return hip.lower_only(x * c + y)[0], x, y
    first, x1, y1 = build(2.0)
    hits = hip.STATS["lowering_hits"]
    again, x2, y2 = build(-7.5)
    assert hip.STATS["lowering_hits"] == hits + 1
    assert again is not first and again.key == first.key and again.tail == first.tail
    assert [b for b, _ in again.srcs] == [x2.array.buf, y2.array.buf] and again.scal == [np.float32(-7.5)]
    assert [b for b, _ in first.srcs] == [x1.array.buf, y1.array.buf] and first.scal == [np.float32(2.0)]
    shifted, _, _ = build(2.0, offset=3)                       # another alignment
    assert hip.STATS["lowering_hits"] == hits + 1 and shifted.key != first.key
    a = leaf((64, 64))
    hip.lower_only(a[1:, :-1] + a[:-1, 1:])                     # two views of one buffer ...
    hits = hip.STATS["lowering_hits"]
    b, c = leaf((64, 64)), leaf((64, 64))
    low = hip.lower_only(b[1:, :-1] + c[:-1, 1:])[0]            # ... are not two buffers
    assert hip.STATS["lowering_hits"] == hits and all(k[0] != "g" for k in low.key[2])
    old = lowering.TUNE["unroll"]
    try:
        lowering.TUNE["unroll"] = 4
        tuned, _, _ = build(2.0)
        assert tuned.key != first.key
    finally:
        lowering.TUNE["unroll"] = old


def test_bitwise_operations_lower_with_numpy_result_types():
    """`&`, `|`, `^`, `~` and shifts fuse for masks and integers; their result types are
    NumPy's, and float operands get NumPy's TypeError when the expression is traced."""
    P = lambda dt: NPArray(hip.placeholder((5003,), dt))
    a, b = P(np.float32), P(np.float32)
    for dt in (np.int32, np.int64, np.uint32, np.uint8):
        x, y = P(dt), P(dt)
        for e, want in [((a > b) & (a < 1.0), np.bool_), ((a > b) | ~(b < 0.5), np.bool_), (x & y, dt),
                        (~x, dt), (x ^ 15, dt), (x << 3, dt), (np.right_shift(x, y), dt),
                        (x & (a > 0), dt)]:
            assert e.dtype == np.dtype(want)
            low, src = hip.lower_only(e)
            assert low.kind == "flat" and len(hip.compile_source(src)) > 0
    assert "(unsigned int)" in hip.lower_only(P(np.int32) << P(np.int32))[1]
    with pytest.raises(TypeError):
        hip.lower_only(a & b)
    with pytest.raises(TypeError):
        hip.lower_only(~a)


def test_shifted_views_lower_to_lds_stencil():
    n = 512
    u = NPArray(hip.placeholder((n, n), np.float32))
    rhs = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
    # a fresh output has rows of 510: the tiles follow the 16-byte boundaries of the grid's
    # buffer and the stores are vectors at element alignment
    low, src = hip.lower_only(rhs)
    assert low.kind == "tile2d" and low.key[0] == "tile2dv" and low.key[-1] is True
    assert "__shared__ f4x4 tile[" in src and "(f4x4u*)(o0 +" in src and "(const f4x4*)(gp + lin)" in src
    kinds = low.key[2]
    assert sorted(k[1:] for k in kinds) == [(0, 0), (1, -1), (1, 1), (2, 0)]
    hip.compile_source(src)
    # a grid whose own rows are not 16-byte periodic: element loads into LDS
    odd = NPArray(hip.placeholder((n - 1, n - 1), np.float32))
    low, src = hip.lower_only(0.25 * (odd[:-2, 1:-1] + odd[2:, 1:-1] + odd[1:-1, :-2] + odd[1:-1, 2:]))
    assert low.key[0] == "tile2d" and "__shared__ float tile[" in src and "__syncthreads" in src
    hip.compile_source(src)
    # written back into the grid's interior, rows stay 16-byte periodic: vector variant
    dst = hip.placeholder((n - 2, n - 2), np.float32, strides=(n, 1), offset=n + 1)
    low, vsrc = hip.lower_only(rhs, dst=dst)
    assert low.key[0] == "tile2dv" and "__shared__ f4x4 tile[" in vsrc
    assert "(f4x4*)(o0 +" in vsrc and "(const f4x4*)(gp + lin)" in vsrc
    hip.compile_source(vsrc)
    src = vsrc
    # association of the sum is the user's: ((up + down) + left) + right, then 0.25 *
    body = src.split("dr_body")[1]
    assert re.search(r"v0 = l0 \+ l1;\s+const float v1 = v0 \+ l2;\s+const float v2 = v1 \+ l3;"
                     r"\s+const float v3 = s0 \* v2;", body)


def test_reduction_lowers_to_fused_tail_with_finalize():
    x, y, w = (leaf((1 << 20,), np.float64) for _ in range(3))
    low, src = hip.lower_only(ReduceEx(np.add, (x - y) ** 2 * w))
    assert low.kind == "flat" and low.fin_count == low.grid
    assert "__shfl_down" in src and "_fin(" in src and "atomic" not in src
    assert hip._kernel_name(low).startswith("dr_flat_reduce_")
    hip.compile_source(src)
    assert ReduceEx(np.add, leaf((8,), np.int32)).dtype == np.int32
    low, src = hip.lower_only(ReduceEx(np.add, leaf((1 << 12,), np.int32)))
    assert "long long* __restrict__ partial" in src          # integer sums accumulate in int64


def test_two_roots_share_one_kernel():
    S, K, T = (leaf((1 << 16,), np.float64) for _ in range(3))
    from oracle import numpy_oracle as orc    # expression text only; nothing is evaluated
    call, put = orc.black_scholes_expr(dr, S, K, T, 0.02, 0.30)
    low, src = hip.lower_only([call, put])
    assert low.kind == "flat"
    body = src[src.index("void dr_body("):src.index("void dr_body_pack(")]
    assert body.count("dr_erf_f8_1(") == 2 and body.count("dr_exp_f8_1(") == 1   # once per use
    # (the square root reaches the prices through `erf` only: the short form)
    assert body.count("dr_log_f8_1(") == 1 and body.count("dr_sqrt_near_f8_1(") == 1
    assert "double& r0, double& r1" in src
    # the main loop passes four options per thread through the functions in lock step
    pack = src[src.index("void dr_body_pack("):src.index('extern "C" __global__')]
    assert pack.count("dr_erf_f8<4>(") == 2 and pack.count("dr_exp_f8<4>(") == 1
    assert pack.count("dr_log_f8<4>(") == 1 and pack.count("dr_sqrt_near_f8<4>(") == 1
    assert "double (&r0)[4], double (&r1)[4]" in pack and "dr_body_pack(P0, P1, P2," in src
    hip.compile_source(src)


_INTEGER_ONLY = set(cg._BITWISE) | set(cg._SHIFTS) | {"invert"}


@pytest.mark.parametrize("name", sorted(cg.SUPPORTED_UFUNCS - {"square"} - _INTEGER_ONLY))
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_every_supported_ufunc_generates_compilable_source(name, dtype):
    fn = getattr(np, name, None)
    if fn is None:
        import scipy.special
        fn = getattr(scipy.special, name)
    a, b = leaf((1 << 10,), dtype), leaf((1 << 10,), dtype)
    ex = fn(a) if fn.nin == 1 else fn(a, b)
    low, src = hip.lower_only(ex)
    hip.compile_source(src)
    expect = ("f" if dtype == np.float32 else "")
    if dtype == np.float64 and name in mathlib.FUNCTIONS:
        assert f"{mathlib.FUNCTIONS[name][0]}<" in src and f"{mathlib.FUNCTIONS[name][0]}_1(" in src
    elif dtype == np.float32 and name in mathlib32.FUNCTIONS:
        assert f"{mathlib32.FUNCTIONS[name][0]}(" in src
    elif name in cg._FLOAT_FUNCS1:
        assert f"{cg._FLOAT_FUNCS1[name]}{expect}(" in src


def test_flags_keep_mul_add_separate_and_unpacked():
    assert "-ffp-contract=off" in hip.COMPILE_OPTS
    joined = " ".join(hip.COMPILE_OPTS)
    assert "-target-feature -Xclang -packed-fp32-ops" in joined


def test_unfusable_ufunc_is_rejected_clearly():
    a = leaf((16,))
    with pytest.raises(NotImplementedError, match="cannot be fused"):
        hip.lower_only(np.logaddexp(a, a))


def test_launching_on_placeholders_is_refused():
    a = leaf((16,))
    with pytest.raises(Exception):
        (a + 1).get()


def test_generated_leaves_cost_no_operand():
    """`zeros/ones/full` are scalar parameters, `arange/linspace` are computed from the
    element index: neither adds a pointer to the kernel."""
    n = 1 << 20
    x = leaf((n,), np.float32)
    grid = dr.linspace(-2.0, 2.0, n, dtype=np.float32)
    low, src = hip.lower_only(grid * x + dr.ones(n, dtype=np.float32))
    assert low.kind == "flat" and len(low.srcs) == 1
    assert "const long long dr_i" in src and "(double)dr_i" in src
    assert src.count("const float* __restrict__ a") == 1
    hip.compile_source(src)
    low, src = hip.lower_only(dr.arange(n))                      # no operand at all
    assert low.kind == "flat" and len(low.srcs) == 0 and "(long long)dr_i" in src
    hip.compile_source(src)
    low, src = hip.lower_only(dr.zeros((1 << 10, 1 << 10), dtype=np.float32))
    assert low.kind == "flat" and len(low.srcs) == 0 and "dr_i" not in src
    hip.compile_source(src)
    # element-wise use next to a 2-d array: still no operand for the constant
    m = leaf((1 << 10, 1 << 10), np.float32)
    low, src = hip.lower_only(dr.zeros((1 << 10, 1 << 10), dtype=np.float32) + m * 2)
    assert low.kind == "flat" and len(low.srcs) == 1


def test_generated_leaves_are_never_shared_and_small_ones_are_eager():
    a, b = dr.zeros(1 << 16), dr.zeros(1 << 16)
    assert type(a) is FullEx and a is not b and (a + 1) is not (b + 1)
    assert type(dr.arange(1 << 16).children[1].children[0]) is IotaEx
    assert dr.arange(0, 1 << 16, 2).shape == (1 << 15,) and dr.arange(0.0, 10.0, 0.001).dtype == np.float64
    assert dr.linspace(0, 1, 1 << 16).shape == (1 << 16,)
    assert dr.linspace(0, 1, 1 << 16, dtype=np.float32).dtype == np.float32


def test_views_of_lazy_expressions_are_pushed_to_the_leaves():
    a, b = leaf((512, 1024)), leaf((1024,))
    e = a * 2 + b
    r = e[1:-1, 4:-4]
    assert type(r) is BinaryNumpyEx and r.shape == (510, 1016) and "array" not in e.__dict__
    low, src = hip.lower_only(r)
    assert len(low.srcs) == 2 and low.kind in ("tile2d", "rows")
    # shifted slices of one expression become one LDS stencil over the expression's leaf
    s = a + 1.0
    lap = s[:-2, 1:-1] + s[2:, 1:-1] + s[1:-1, :-2] + s[1:-1, 2:]
    low, src = hip.lower_only(lap)
    assert low.kind in ("tile2d", "tile2dv") and "__shared__" in src and len(low.srcs) == 1
    hip.compile_source(src)
    # transposes: the leaves are read through the LDS transpose tile
    low, src = hip.lower_only((a * 2).T)
    assert low.kind == "tile2dt"
    assert e.T.shape == (1024, 512) and "array" not in e.__dict__


def test_three_dimensional_shifted_views_lower_to_the_lds_window():
    n = 128
    u = NPArray(hip.placeholder((n, n, n), np.float32))
    rhs = (u[:-2, 1:-1, 1:-1] + u[2:, 1:-1, 1:-1] + u[1:-1, :-2, 1:-1] + u[1:-1, 2:, 1:-1]
           + u[1:-1, 1:-1, :-2] + u[1:-1, 1:-1, 2:]) * (1 / 6.0)
    dst = hip.placeholder((n - 2,) * 3, np.float32, strides=(n * n, n, 1), offset=n * n + n + 1)
    low, src = hip.lower_only(rhs, dst=dst)
    assert low.kind == "tile3d" and len(low.srcs) == 1 and "__shared__ f4x4 tile[" in src
    shifts = sorted(k[1:] for k in low.key[2])
    assert shifts == [(0, 0, 0), (1, -1, 0), (1, 0, -1), (1, 0, 1), (1, 1, 0), (2, 0, 0)]
    hip.compile_source(src)
    odd = NPArray(hip.placeholder((n, n, n - 1), np.float32))      # rows not 16-byte multiples
    low, src = hip.lower_only(odd[:-2, 1:-1, 1:-1] + odd[2:, 1:-1, 1:-1])
    assert low.kind == "tile2d"


def test_device_random_numbers_cost_no_operand():
    """`random.device(seed)`: the Philox stream is computed from the element index, so an
    expression over its arrays reads nothing; successive draws continue the stream."""
    from delayrepay_amd.delayarray import RandEx
    gen = dr.random.device(2024)
    u = gen.random(1 << 16)
    v = gen.uniform(-1.0, 1.0, 1 << 16)
    assert isinstance(u, RandEx) and "array" not in u.__dict__
    assert (u.pos, v.children[1].children[1].pos) == (0, 0)      # each draw starts on its own block
    assert v.children[1].children[1].counter == u.counter + (1 << 14)
    low, src = hip.lower_only(u * u + v)
    assert low.kind == "flat" and low.srcs == []                 # 0 bytes read per element
    assert src.count("dr_philox(") == 3 and "unsigned __int128" in src
    hip.compile_source(src)
    odd = dr.random.device(1)
    odd.random(3)
    w = odd.random_raw(1 << 12)                                   # starts in the middle of a block
    assert (w.pos, w.dtype) == (3, np.int64)
    hip.compile_source(hip.lower_only(w)[1])
    f = dr.random.device(9).random(1 << 14, dtype=np.float32)     # eight floats per block
    low, src = hip.lower_only(f * 2)
    assert f.dtype == np.float32 and low.kind == "flat" and low.srcs == [] and src.count("dr_philox_block(") == 3
    hip.compile_source(src)
    gen = dr.random.device(9)
    gen.random(3, dtype=np.float32)                              # leaves the high half of output 1 waiting
    assert gen._half == 1 and gen.pos == 2                       # (taken first by the next float32 draw)
    with pytest.raises(ValueError):
        dr.random.device(-1)


# ---- structures met before (hip._scan) -----------------------------------------------

def test_scan_writes_down_what_tracing_and_lowering_look_at():
    """Two expressions get the same key exactly when tracing and lowering them gives the
    same kernel and the same places for buffers and numbers: same functions, same operand
    identities (x*x is not x*y), same number types, same leaf geometry."""
    def key(*roots, head=("run",)):
        scan = hip._scan(roots, head)
        return None if scan is None else scan[0]
    a, b, c = leaf((64,)), leaf((64,)), leaf((64,))
    a2, b2 = leaf((64,)), leaf((64,))
    assert key(2.0 * a + b) == key(3.5 * a2 + b2)            # other arrays, another number
    assert key(2.0 * a + b) != key(2 * a + b)                 # a Python int is another type
    assert key(2.0 * a + b) != key(np.float32(2.0) * a + b)   # and so is a NumPy scalar
    assert key(a * a + b) != key(a * b + b)                   # which operand is which
    assert key(a * b + b) == key(a2 * b2 + b2)
    assert key(a * b + c) != key(a * b + b)
    assert key(a + b) != key(a - b)
    assert key(a + b) != key(a + leaf((64,), np.float64))     # dtype
    assert key(a + b) != key(leaf((32,)) + leaf((32,)))       # shape
    assert key(a + b) != key(a + leaf((1,)))                  # a broadcast operand
    d = a - b
    assert key(d * d) == key((a2 - b2) * (a2 - b2))           # hash-consed: one node, met twice
    k0, k1 = key(2.0 * a, 2.0 * a + b, head=("multi",)), key(2.0 * a2, 2.0 * a2 + b2, head=("multi",))
    assert k0 == k1 and k0 != key(2.0 * a + b, 2.0 * a, head=("multi",))
    # views of one buffer are told from views of two
    base = hip.placeholder((66,), np.float32)
    from delayrepay_amd.delayarray import NPArray
    v0, v1 = NPArray(base[:-2]), NPArray(base[2:])
    assert key(v0 + v1) != key(a + b)
    # what the tracer has to look at itself is not scanned
    assert key(np.where(a > 0, a, b)) is None
    assert key((a + b).astype(np.float64) * 2.0) is None
    assert key(a) is None


def test_scan_leaves_nothing_behind():
    """Nothing on the nodes changes and no reference cycle is made by looking."""
    import gc
    import weakref
    a, b = leaf((64,)), leaf((64,))
    ex = (a - b) * (a - b) + 2.0
    before = {k: dict(n.__dict__) for k, n in (("ex", ex), ("a", a))}
    gc.collect()
    gc.disable()
    try:
        scan = hip._scan((ex,), ("run",))
        ref = weakref.ref(ex)
        assert {k: dict(n.__dict__) for k, n in (("ex", ex), ("a", a))} == before
        del scan, ex, before
        assert ref() is None
    finally:
        gc.enable()


def test_long_rows_take_a_block_of_512_lanes_and_compile():
    """Lowering of softmax by row length: a lane group or a block of 256 lanes up to 64 KB,
    a block of 512 lanes up to 256 KB (with the waves' partial results combined over eight
    slots), and nothing beyond (`RowFusionUnsupported`: the caller evaluates the reductions
    on their own).  The generated source goes through hiprtc here, without a device."""
    def soft(a):
        e = np.exp(a - a.max(axis=1, keepdims=True))
        return e / e.sum(axis=1, keepdims=True)
    for R, dtype, lanes in ((16384, np.float32, 256), (16385, np.float32, 512), (50257, np.float32, 512),
                            (65536, np.float32, 512), (32768, np.float64, 512), (8192, np.float64, 256)):
        low, src = hip.lower_only(soft(leaf((64, R), dtype)))
        assert low.kind == "rows" and lowering.block_lanes(low) == lanes, (R, dtype)
        assert f"__launch_bounds__({lanes})" in src and f"[{lanes // 64}];" in src
        if lanes == 512:
            assert "slot[7]" in src and "slot[8]" not in src
            hip.compile_source(src)
    for R, dtype in ((65537, np.float32), (32769, np.float64)):
        with pytest.raises(cg.RowFusionUnsupported):
            hip.lower_only(soft(leaf((64, R), dtype)))
    low, _ = hip.lower_only(leaf((64, 50257)) * 2.0)
    assert lowering.block_lanes(low) == cg.BLOCK


def test_every_axis_reduction_kernel_shape_is_emitted_and_compiles():
    """One case per strategy of the reductions along axes (a block, a lane group or a wave
    per output row, a thread per output column, streams over a middle axis, the narrow and
    short forms): lowered over placeholders, the source generated and put through hiprtc."""
    cases = {"axis_block": ((16384, 16384), (1,)), "axis_stream": ((256, 512, 1024), (1,)),
             "axis_group": ((1342177, 200), (1,)), "axis_row": ((37, 70, 129), (0, 2)),
             "axis_col": ((129, 70), (0,)), "axis_narrow": ((1 << 22, 8), (0,)),
             "axis_short": ((1 << 20, 4), (1,))}
    for kind, (shape, axes) in cases.items():
        for func, dtype in ((np.add, np.float32), (np.maximum, np.float64)):
            low, src = hip.lower_only(ReduceEx(func, leaf(shape, dtype) * 2.0, axes))
            assert low.kind == kind, (kind, low.kind, dtype)
            hip.compile_source(src)


def test_reductions_along_rows_of_a_batch_with_a_shared_operand_keep_the_row_wise_kernels():
    """`sum(x + m, axis=-1)`, x (batch, rows, columns), m (rows, columns): two levels of
    kept dimensions; the lane, lane-group and block kernels take them with the row number
    split by the inner level (`dr_row_at`), and their sources compile."""
    for (B, N, R), kind in (((256, 8192, 8), "axis_short"), ((256, 8192, 64), "axis_group"),
                            ((64, 1000, 1000), "axis_group"), ((16, 512, 16384), "axis_block")):
        low, src = hip.lower_only(ReduceEx(np.add, leaf((B, N, R)) + leaf((N, R)), (2,)))
        assert low.kind == kind and "dr_row_at(k, K1, sk0, sj0)" in src, (B, N, R, low.kind)
        assert low.tail[-3:] == [N, R, R] and low.fmt.endswith("Iqq")
        hip.compile_source(src)
        plain, src1 = hip.lower_only(ReduceEx(np.add, leaf((B, N, R)) * 2.0, (2,)))
        assert plain.kind == kind and "dr_row_at" not in src1


def test_masks_that_are_the_same_along_a_row_compile_in_the_row_kernel():
    """A comparison of per-row values (`row maximum > 0`, a mask per row from a column) is
    a byte that is computed once per row and handed on; bytes have no vector register class
    of their own, so they are passed through a word where the kernel hides a value from
    the optimiser."""
    a = leaf((1000, 300))
    mx = a.max(axis=1, keepdims=True)
    for ex in (np.where(mx > 0, a / mx, a),
               np.where(a.sum(axis=1, keepdims=True) > mx, a, -a) * (mx > 1),
               np.where((leaf((1 << 20,)) > 0)[:, None], leaf((1 << 20, 3)), 0.0)):
        low, src = hip.lower_only(ex)
        assert low.kind == "rows" and "unsigned char" in src
        hip.compile_source(src)


def test_thin_transposes_are_a_lane_per_index_of_the_long_side():
    """A transposed operand in a matrix with a side of at most 16 elements that is no power of
    two: no tile; both orientations, a directly read operand beside the transposed one."""
    for shape, short_rows in (((1 << 20, 3), True), ((3, 1 << 20), False), ((1 << 18, 12), True)):
        x, o = leaf(shape), leaf(shape[::-1])
        low, src = hip.lower_only(x.T * 2.0 + o)
        assert low.kind == "thin_t" and low.key[-2:] == (min(shape), short_rows)
        assert "__shared__" not in src and low.tail[0] == max(shape) and low.grid == max(shape) // 256
        hip.compile_source(src)
    assert hip.lower_only(leaf((1 << 20, 4)).T * 2.0)[0].kind == "tile2dt"      # a power of two
    assert hip.lower_only(leaf((1000, 3)).T * 2.0)[0].kind == "tile2dt"         # a short long side
    assert hip.lower_only(leaf((1 << 20, 24)).T * 2.0)[0].kind == "tile2dt"
