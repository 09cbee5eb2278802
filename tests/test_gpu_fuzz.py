"""Seeded random expressions over random views, compared bit for bit with the
NumPy oracle.  Every operation used is exact in IEEE arithmetic (+ - * / sqrt abs
negate maximum minimum comparisons where casts), so any difference is a bug in
tracing, lowering (flat / tile2d / tile2dv / tile2dt / nd / reductions) or code
generation, not rounding.  Operand layouts: dense, offset slices, strided slices,
transposes, row / column / scalar broadcasts; dtypes float32, float64, int32, int64."""
import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import hip
from oracle.numpy_oracle import OracleArray
from tests.helpers import bits_equal

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64, np.float32, np.float64, np.int32, np.int64]


def make_host(rs, shape, dtype):
    if np.dtype(dtype).kind == "i":
        return rs.randint(-4, 5, shape).astype(dtype)
    vals = rs.uniform(-2, 2, shape)
    vals[rs.uniform(size=shape) < 0.03] = 0.0
    return vals.astype(dtype)


def random_leaf(rs, shape):
    """(device lazy array, oracle array) of broadcast-compatible shape."""
    dtype = DTYPES[rs.randint(len(DTYPES))]
    kind = rs.randint(8)
    if len(shape) == 1:
        (n,) = shape
        if kind in (0, 1, 2):
            host, key = make_host(rs, (n,), dtype), np.s_[:]
        elif kind in (3, 4):
            off = rs.randint(1, 6)
            host, key = make_host(rs, (n + off + 2,), dtype), np.s_[off:off + n]
        elif kind == 5:
            step = rs.randint(2, 4)
            host, key = make_host(rs, (n * step,), dtype), np.s_[::step]
        elif kind == 6:
            host, key = make_host(rs, (1,), dtype), np.s_[:]
        else:
            host, key = make_host(rs, (n,), dtype), np.s_[::-1]
        return dr.array(host)[key], OracleArray(host.copy())[key]
    h, w = shape
    if kind in (0, 1):
        host, key, t = make_host(rs, (h, w), dtype), np.s_[:, :], False
    elif kind == 2:
        a, b = rs.randint(0, 3), rs.randint(0, 5)
        host, key, t = make_host(rs, (h + a + 1, w + b + 2), dtype), np.s_[a:a + h, b:b + w], False
    elif kind == 3:
        host, key, t = make_host(rs, (h * 2, w * 3), dtype), np.s_[::2, ::3], False
    elif kind == 4:
        host, key, t = make_host(rs, (w, h), dtype), np.s_[:, :], True
    elif kind == 5:
        host, key, t = make_host(rs, (1, w), dtype), np.s_[:, :], False
    elif kind == 6:
        host, key, t = make_host(rs, (h, 1), dtype), np.s_[:, :], False
    else:
        host, key, t = make_host(rs, (w,), dtype), np.s_[:], False
    d, o = dr.array(host)[key], OracleArray(host.copy())[key]
    return (d.T, OracleArray(o.a.T)) if t else (d, o)


UNARY = [np.negative, np.absolute, lambda x: np.sqrt(np.absolute(x)), lambda x: x * x,
         lambda x: x.astype(np.float32), lambda x: x.astype(np.float64), lambda x: 0.5 * x,
         lambda x: x + 1, lambda x: 3 - x, lambda x: x / 2.0]
BINARY = [np.add, np.subtract, np.multiply, np.true_divide, np.maximum, np.minimum,
          lambda a, b: np.where(a > b, a, b * 2), lambda a, b: np.where(a < 0, b, a),
          lambda a, b: (a >= b).astype(np.float32) + a]


def random_expr(rs, shape, depth):
    if depth == 0 or rs.uniform() < 0.15:
        return random_leaf(rs, shape)
    if rs.uniform() < 0.35:
        fn = UNARY[rs.randint(len(UNARY))]
        d, o = random_expr(rs, shape, depth - 1)
        return fn(d), fn(o)
    fn = BINARY[rs.randint(len(BINARY))]
    d1, o1 = random_expr(rs, shape, depth - 1)
    d2, o2 = random_expr(rs, shape, depth - 1)
    return fn(d1, d2), fn(o1, o2)


def full_shape_leaf(rs, shape):
    """A leaf that really has `shape` (so the expression's shape is not all-broadcast)."""
    host = make_host(rs, shape, DTYPES[rs.randint(4)])
    return dr.array(host), OracleArray(host.copy())


@pytest.mark.parametrize("seed", range(120))
def test_random_expression(seed):
    rs = np.random.RandomState(1000 + seed)
    if rs.uniform() < 0.4:
        shape = (int(rs.choice([1, 5, 63, 64, 257, 1000, 4099])),)
    else:
        shape = (int(rs.choice([1, 3, 8, 33, 64, 130])), int(rs.choice([1, 4, 7, 64, 129, 260, 1300])))
    with np.errstate(all="ignore"):
        d, o = random_expr(rs, shape, depth=int(rs.randint(1, 5)))
        anchor_d, anchor_o = full_shape_leaf(rs, shape)
        d, o = d + anchor_d, o + anchor_o
        mode = rs.randint(5)
        if mode <= 1:
            got, ref = d.get(), o.get()
        elif mode == 2:                      # fused full reduction (exact for max/min)
            got = np.asarray(dr.max(d).get())
            ref = np.asarray(np.max(o.a))
        elif mode == 3 and len(shape) == 2:  # axis reduction (max: order-independent)
            axis = int(rs.randint(2))
            got, ref = dr.max(d, axis=axis).get(), np.max(o.a, axis=axis)
        else:                                # fused assignment into a view of a bigger array
            pad = tuple(s + 3 for s in shape)
            host = make_host(rs, pad, np.float64)
            dst_d, dst_o = dr.array(host), host.copy()
            key = tuple(slice(1, 1 + s) for s in shape)
            dst_d[key] = d
            dst_o[key] = o.a
            got, ref = dst_d.get(), dst_o
    assert bits_equal(got, np.asarray(ref)), (seed, shape, mode)


@pytest.mark.parametrize("seed", range(40))
def test_random_expression_on_skinny_matrices(seed):
    """Many rows, few columns: the shapes that have reduction kernels of their own."""
    rs = np.random.RandomState(5000 + seed)
    shape = (int(rs.choice([4096, 4100, 9001])), int(rs.choice([2, 3, 7, 16, 33, 64])))
    with np.errstate(all="ignore"):
        d, o = random_expr(rs, shape, depth=int(rs.randint(1, 4)))
        anchor_d, anchor_o = full_shape_leaf(rs, shape)
        d, o = d + anchor_d, o + anchor_o
        mode = rs.randint(4)
        if mode == 0:
            got, ref = d.get(), o.get()
        else:
            axis = int(rs.randint(2))
            fn = (dr.max, np.max) if mode == 1 else (dr.min, np.min)
            got, ref = fn[0](d, axis=axis).get(), fn[1](o.a, axis=axis)
    assert bits_equal(got, np.asarray(ref)), (seed, shape, mode)


def test_fuzz_reached_every_kernel_shape():
    """Runs after the cases above: the kernel cache must hold every shape kind."""
    kinds = {}
    for key in hip._KERNELS:
        kinds[key[0]] = kinds.get(key[0], 0) + 1
    print("kernel kinds compiled:", kinds)
    for kind in ("flat", "nd", "tile2dv", "tile2dt", "axis", "axis_short", "axis_narrow",
                 "axis_group", "rows"):
        assert kinds.get(kind, 0) > 0, kind


# ---- random view geometries: offsets, row pitches, steps, transposes, broadcast axes ------------

GEO_DTYPES = [np.float32, np.float64, np.int32, np.int64]


def geo_leaf(rs, shape, dtype):
    """(lazy leaf, host array) with the same random geometry on both sides."""
    nd = len(shape)
    kind = rs.randint(7)

    def both(host, view):
        dev = dr.array(host)
        return view(dev), view(host)

    if kind == 1:                                   # starts off a 16-byte boundary
        off = int(rs.randint(1, 4))
        n = int(np.prod(shape))
        host = make_host(rs, (n + off,), dtype)
        return both(host, lambda a: a[off:].reshape(shape))
    if kind == 2 and nd >= 2:                       # rows with a pitch, shifted start
        pad = int(rs.randint(1, 6))
        host = make_host(rs, shape[:-1] + (shape[-1] + pad,), dtype)
        lo = int(rs.randint(0, pad + 1))
        return both(host, lambda a: a[..., lo:lo + shape[-1]])
    if kind == 3:                                   # stretched along one axis
        k = int(rs.randint(nd))
        host = make_host(rs, tuple(1 if i == k else d for i, d in enumerate(shape)), dtype)
        return both(host, lambda a: a)
    if kind == 4 and nd >= 2:                       # lower rank
        host = make_host(rs, shape[1:], dtype)
        return both(host, lambda a: a)
    if kind == 5 and nd == 2:                       # transposed
        host = make_host(rs, (shape[1], shape[0]), dtype)
        return both(host, lambda a: a.T)
    if kind == 6:                                   # every second element
        host = make_host(rs, tuple(2 * d for d in shape), dtype)
        key = tuple(slice(int(rs.randint(2)), None, 2) for _ in shape)
        return both(host, lambda a: a[key])
    host = make_host(rs, shape, dtype)
    return both(host, lambda a: a)


def geo_expr(rs, shape, depth):
    if depth == 0:
        return geo_leaf(rs, shape, GEO_DTYPES[rs.randint(len(GEO_DTYPES))])
    op = rs.randint(8)
    d, h = geo_expr(rs, shape, depth - 1)
    if op == 0:
        return d * 2.5, h * 2.5
    if op == 1:
        return np.sqrt(np.abs(d) + 1.0), np.sqrt(np.abs(h) + 1.0)
    if op == 2:
        return dr.where(d > 0, d, 1), np.where(h > 0, h, 1)
    if op == 3:
        return (d + 0).astype(np.float32), (h + 0).astype(np.float32)
    d2, h2 = geo_expr(rs, shape, depth - 1)
    if op == 4:
        return d + d2, h + h2
    if op == 5:
        return d * d2, h * h2
    if op == 6:
        return np.maximum(d, d2), np.maximum(h, h2)
    return d - d2, h - h2


@pytest.mark.parametrize("seed", range(80))
def test_random_geometry_matches_numpy(seed):
    rs = np.random.RandomState(9000 + seed)
    nd = int(rs.randint(1, 4))
    shape = tuple(int(rs.choice([1, 3, 16, 33, 64, 130, 1030])) for _ in range(nd))
    if np.prod(shape) > 1 << 21:
        shape = shape[:2]
    with np.errstate(all="ignore"):
        d, h = geo_expr(rs, shape, int(rs.randint(0, 4)))
        anchor = make_host(rs, shape, np.float32)
        d, h = d + dr.array(anchor), h + anchor
        mode = rs.randint(4)
        if mode == 0 or len(shape) < 2:
            got, ref = d.get(), h
        elif mode == 1:
            got, ref = np.asarray(dr.max(d).get()), np.asarray(np.max(h))
        elif mode == 2:
            axis = int(rs.randint(len(shape)))
            got, ref = dr.min(d, axis=axis).get(), np.min(h, axis=axis)
        else:                                       # into a view with a pitch
            pad = tuple(s + 2 for s in shape)
            host = make_host(rs, pad, np.float64)
            dst_d, dst_h = dr.array(host), host.copy()
            key = tuple(slice(1, 1 + s) for s in shape)
            dst_d[key] = d
            dst_h[key] = h
            got, ref = dst_d.get(), dst_h
    assert got.dtype == np.asarray(ref).dtype and bits_equal(got, np.asarray(ref)), (seed, shape, mode)


# ---- the same with flipped axes and combined masks ------------------------------------------------

def flip_leaf(rs, shape, dtype):
    d, h = geo_leaf(rs, shape, dtype)
    how = rs.randint(4)
    if how == 0 or d.shape != tuple(shape):          # (lower-rank leaves flip along their own axes)
        return d, h
    if how == 1:
        key = (Ellipsis, slice(None, None, -1))
    elif how == 2:
        key = (slice(None, None, -1),)
    else:
        key = tuple(slice(None, None, -1) for _ in shape)
    return d[key], h[key]


def flip_expr(rs, shape, depth):
    if depth == 0:
        return flip_leaf(rs, shape, GEO_DTYPES[rs.randint(len(GEO_DTYPES))])
    op = rs.randint(7)
    d, h = flip_expr(rs, shape, depth - 1)
    if op == 0:
        return d * 2.5, h * 2.5
    if op == 1:
        return dr.where((d > 0) & (d < 50), d, 1), np.where((h > 0) & (h < 50), h, 1)
    if op == 2:
        return (d + 0).astype(np.float32), (h + 0).astype(np.float32)
    d2, h2 = flip_expr(rs, shape, depth - 1)
    if op == 3:
        return d + d2, h + h2
    if op == 4:
        return dr.where((d > d2) | ~(d2 > 0), d, d2), np.where((h > h2) | ~(h2 > 0), h, h2)
    if op == 5:
        return np.minimum(d, d2), np.minimum(h, h2)
    return d - d2, h - h2


@pytest.mark.parametrize("seed", range(60))
def test_random_geometry_with_flips_and_masks(seed):
    rs = np.random.RandomState(12000 + seed)
    nd = int(rs.randint(1, 4))
    shape = tuple(int(rs.choice([1, 3, 16, 33, 64, 130, 1030])) for _ in range(nd))
    if np.prod(shape) > 1 << 21:
        shape = shape[:2]
    with np.errstate(all="ignore"):
        d, h = flip_expr(rs, shape, int(rs.randint(0, 4)))
        anchor = make_host(rs, shape, np.float32)
        if rs.randint(2):
            d, h = d + dr.array(anchor)[..., ::-1], h + anchor[..., ::-1]
        else:
            d, h = d + dr.array(anchor), h + anchor
        mode = rs.randint(3)
        if mode == 0 or len(shape) < 2:
            got, ref = d.get(), h
        elif mode == 1:
            axis = int(rs.randint(len(shape)))
            got, ref = dr.max(d, axis=axis).get(), np.max(h, axis=axis)
        else:
            pad = tuple(s + 2 for s in shape)
            host = make_host(rs, pad, np.float64)
            dst_d, dst_h = dr.array(host), host.copy()
            key = tuple(slice(1, 1 + s) for s in shape)
            dst_d[key] = d
            dst_h[key] = h
            got, ref = dst_d.get(), dst_h
    assert got.dtype == np.asarray(ref).dtype and bits_equal(got, np.asarray(ref)), (seed, shape, mode)


def test_short_rows_with_repeated_operands_into_every_kind_of_destination():
    """Random element-wise expressions over a matrix or a batch of matrices with short rows
    and operands that repeat along or across them (a row, a column, a matrix per batch, a
    vector per item, a scalar), evaluated into a new array, an existing dense array, a view
    with a pitch, and over the first operand: bit-equal to NumPy in all of them."""
    bad = 0
    kinds = {}
    for seed in range(160):
        rs = np.random.RandomState(1000 + seed)
        dtype = [np.float32, np.float64, np.int32, np.int64][rs.randint(4)]
        R = int(rs.choice([1, 2, 3, 5, 8, 16, 33, 64, 70, 200, 500, 1000, 1024]))
        three = rs.randint(3) == 0
        lead = (int(rs.choice([1, 2, 5])), int(rs.choice([1, 7, 40]))) if three else (int(rs.choice([1, 3, 100, 1001])),)
        shape = lead + (R,)
        def mk(s):
            if np.dtype(dtype).kind == "f":
                return (rs.standard_normal(s) * 4).astype(dtype)
            return rs.randint(-20, 20, s).astype(dtype)
        ops = {"x": mk(shape), "v": mk((R,)), "c": mk(lead + (1,)), "s": mk(())}
        if three:
            ops["m"] = mk(lead[1:] + (R,)); ops["b"] = mk((lead[0], 1, R))
        names = list(ops)
        dev = {k: dr.array(v) for k, v in ops.items()}
        def build(env, xp):
            e = env["x"]
            for _ in range(rs_local.randint(1, 5)):
                o = env[names[rs_local.randint(len(names))]]
                k = rs_local.randint(6)
                if k == 0: e = e + o
                elif k == 1: e = e - o
                elif k == 2: e = e * o
                elif k == 3: e = xp.maximum(e, o)
                elif k == 4: e = xp.where(e > o, e, o)
                else: e = xp.minimum(e, o) - e
            return e
        st = rs.randint(1 << 30)
        rs_local = np.random.RandomState(st); ref = build(ops, np)
        rs_local = np.random.RandomState(st); ex = build(dev, dr)
        mode = rs.randint(4)
        try:
            if mode == 0:
                k = hip.lower_only(ex)[0].kind
                got = ex.get()
            elif mode == 1:                       # dense existing destination
                dst = dr.zeros(shape, dtype=ref.dtype); k = "w"; dst[...] = ex; got = dst.get()
            elif mode == 2:                       # pitched view
                big = dr.zeros(lead + (R + 7,), dtype=ref.dtype); k = "p"; big[..., 3:R + 3] = ex
                got = big.get()[..., 3:R + 3]
                assert not big.get()[..., :3].any() and not big.get()[..., R + 3:].any()
            else:                                 # over the operand
                k = "i"
                if ref.dtype == ops["x"].dtype and ref.shape == shape:
                    dev["x"][...] = ex; got = dev["x"].get()
                else:
                    got = ex.get()
            kinds[k] = kinds.get(k, 0) + 1
            ok = got.dtype == ref.dtype and got.shape == ref.shape and got.tobytes() == np.ascontiguousarray(ref).tobytes()
        except Exception as e:
            ok = False; print("seed", seed, "raised", type(e).__name__, str(e)[:100])
        if not ok:
            bad += 1; print("MISMATCH seed", seed, np.dtype(dtype).name, shape, "mode", mode, flush=True)


    print("destinations and kernels:", kinds)
    assert bad == 0
