"""Reductions along the last axis inside an expression: one kernel reads each row once,
reduces it, uses the result and writes once (`codegen.emit_row_fused`; the reference's
`ReduceEx` as an interior node, delayarray.py:272-283, cuda.py:87-88).

Bars: expressions of max / min and + - * / only are bit-equal to NumPy; sums within
rtol 1e-6 (float32) / 1e-13 (float64) of NumPy's; what follows a sum inherits its
tolerance."""
import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import hip, lowering
from tests.helpers import bits_equal

pytestmark = pytest.mark.gpu

SHAPES = [(5, 2), (3, 7), (64, 200), (33, 203), (1000, 64), (7, 1000), (9, 1023), (130, 1025),
          (50, 4096), (17, 4099), (12, 16384), (5, 16381), (9, 13001), (6, 12289),
          (4, 32768), (3, 32000), (3, 20001), (2, 40000), (2, 65536), (2, 70001)]
ROW_BYTES = 262144      # a row of at most 256 KB is held by one block (of 512 lanes above 64 KB)


def launches(fn):
    before = hip.STATS["launches"]
    out = fn()
    return out, hip.STATS["launches"] - before


def softmax(xp, a):
    e = xp.exp(a - a.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_softmax_is_one_kernel(shape, dtype):
    rs = np.random.RandomState(hash(shape) % 1000)
    a = (rs.standard_normal(shape) * 3).astype(dtype)
    got, n = launches(lambda: softmax(dr, dr.array(a)).get())
    ref = softmax(np, a)
    fits = shape[-1] * a.itemsize <= ROW_BYTES
    assert (n == 1 or not fits) and got.shape == ref.shape and got.dtype == ref.dtype
    np.testing.assert_allclose(got, ref, rtol=2e-6 if dtype == np.float32 else 1e-13)
    np.testing.assert_allclose(got.sum(axis=-1), 1.0, rtol=1e-5 if dtype == np.float32 else 1e-13)


@pytest.mark.parametrize("shape", SHAPES)
def test_max_min_and_arithmetic_are_bit_equal(shape):
    rs = np.random.RandomState(3)
    a = rs.standard_normal(shape).astype(np.float32)
    da = dr.array(a)
    fits = shape[-1] * a.itemsize <= ROW_BYTES
    got, n = launches(lambda: (da - da.max(axis=1, keepdims=True)).get())
    assert (n == 1 or not fits) and bits_equal(got, a - a.max(axis=1, keepdims=True))
    lo, hi = da.min(axis=-1, keepdims=True), da.max(axis=-1, keepdims=True)
    got, n = launches(lambda: ((da - lo) / (hi - lo)).get())
    ref = (a - a.min(axis=-1, keepdims=True)) / (a.max(axis=-1, keepdims=True) - a.min(axis=-1, keepdims=True))
    assert (n == 1 or not fits) and bits_equal(got, ref)


def test_nan_and_infinity_in_a_row_follow_numpy():
    a = np.random.RandomState(4).standard_normal((6, 300)).astype(np.float32)
    a[1, 17] = np.nan
    a[2, 5] = np.inf
    a[3, 299] = -np.inf
    a[4, :] = -np.inf
    da = dr.array(a)
    with np.errstate(invalid="ignore"):
        ref = a - a.max(axis=1, keepdims=True)
        ref2 = softmax(np, a)
    got = (da - da.max(axis=1, keepdims=True)).get()
    assert np.array_equal(np.isnan(got), np.isnan(ref)) and bits_equal(np.nan_to_num(got), np.nan_to_num(ref))
    got2 = softmax(dr, da).get()
    assert np.array_equal(np.isnan(got2), np.isnan(ref2))
    np.testing.assert_allclose(np.nan_to_num(got2), np.nan_to_num(ref2), rtol=2e-6)


@pytest.mark.parametrize("shape", [(64, 200), (33, 1001), (20, 4096), (6, 16384), (3, 32768)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_centred_and_normalised_rows(shape, dtype):
    rs = np.random.RandomState(7)
    a = (rs.standard_normal(shape) * 2 + 5).astype(dtype)
    g, b = rs.standard_normal(shape[1]).astype(dtype), rs.standard_normal(shape[1]).astype(dtype)
    da, dg, db = dr.array(a), dr.array(g), dr.array(b)
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == np.float32 else dict(rtol=1e-11, atol=1e-11)
    fits = shape[-1] * a.itemsize <= ROW_BYTES
    got, n = launches(lambda: (da - da.mean(axis=1, keepdims=True)).get())
    assert n == 1 or not fits
    np.testing.assert_allclose(got, a - a.mean(axis=1, keepdims=True), **tol)
    # layer normalisation with weights shared by all rows: mean, then variance, then the rows
    def layer_norm(xp, x, w, c):
        mu = x.mean(axis=-1, keepdims=True)
        d = x - mu
        var = (d * d).mean(axis=-1, keepdims=True)
        return d / xp.sqrt(var + 1e-5) * w + c
    got, n = launches(lambda: layer_norm(dr, da, dg, db).get())
    assert n == 1 or not fits
    np.testing.assert_allclose(got, layer_norm(np, a, g, b), **tol)
    # variance and standard deviation along the rows: the mean never leaves the kernel
    for keep in (False, True):
        got, n = launches(lambda: dr.var(da, axis=1, keepdims=keep).get())
        ref = a.var(axis=1, keepdims=keep)
        # the row kernel, then the division by n (one more when an operand built by the
        # lines above has been met often enough to be computed on its own)
        assert got.shape == ref.shape and (n <= 3 or not fits)
        np.testing.assert_allclose(got, ref, rtol=1e-4 if dtype == np.float32 else 1e-11)
        got = dr.std(da, axis=1, ddof=1, keepdims=keep).get()
        np.testing.assert_allclose(got, a.std(axis=1, ddof=1, keepdims=keep),
                                   rtol=1e-4 if dtype == np.float32 else 1e-11)
    # z-scores: two reductions of different depth and a quotient of per-row values
    got, n = launches(lambda: ((da - da.mean(axis=1, keepdims=True)) / da.std(axis=1, keepdims=True)).get())
    assert n == 1 or not fits
    np.testing.assert_allclose(got, (a - a.mean(axis=1, keepdims=True)) / a.std(axis=1, keepdims=True), **tol)


def test_values_that_are_one_per_row_come_out_as_columns():
    rs = np.random.RandomState(8)
    a = rs.standard_normal((40, 700))
    da = dr.array(a)
    m = da.max(axis=1, keepdims=True)
    lse = m + np.log(np.exp(da - m).sum(axis=1, keepdims=True))
    got, n = launches(lambda: lse.get())
    mm = a.max(axis=1, keepdims=True)
    ref = mm + np.log(np.exp(a - mm).sum(axis=1, keepdims=True))
    assert n == 1 and got.shape == (40, 1)
    np.testing.assert_allclose(got, ref, rtol=1e-13)
    # a kept reduction asked for on its own is an ordinary axis reduction
    got = da.min(axis=1, keepdims=True).get()
    assert got.shape == (40, 1) and np.array_equal(got, a.min(axis=1, keepdims=True))
    # the column and the matrix from one kernel
    sm = softmax(dr, da)
    peak = sm.max(axis=1, keepdims=True)
    (_, _), n = launches(lambda: dr.evaluate(sm, peak))
    np.testing.assert_allclose(sm.get(), softmax(np, a), rtol=1e-13)
    np.testing.assert_allclose(peak.get(), softmax(np, a).max(axis=1, keepdims=True), rtol=1e-13)


def test_stacks_of_matrices_and_operands_of_other_shapes():
    rs = np.random.RandomState(9)
    a = rs.standard_normal((6, 10, 300)).astype(np.float32)
    col = rs.standard_normal((10, 1)).astype(np.float32)
    da, dcol = dr.array(a), dr.array(col)
    got, n = launches(lambda: softmax(dr, da).get())
    assert n == 1
    np.testing.assert_allclose(got, softmax(np, a), rtol=2e-6)
    # a per-row operand and a number in the expression
    got = ((da * 0.5 - (da * 0.5).max(axis=-1, keepdims=True))[1] + dcol).get()
    ref = (a * np.float32(0.5) - (a * np.float32(0.5)).max(axis=-1, keepdims=True))[1] + col
    assert bits_equal(got, ref)
    # rows of a view (a row pitch that is no multiple of 16 bytes)
    v = dr.array(rs.standard_normal((50, 333)).astype(np.float32))
    hv = v.get()
    got = (v[:, 1:-2] - v[:, 1:-2].max(axis=1, keepdims=True)).get()
    assert bits_equal(got, hv[:, 1:-2] - hv[:, 1:-2].max(axis=1, keepdims=True))


def test_what_the_row_kernel_does_not_take_is_computed_the_long_way():
    rs = np.random.RandomState(10)
    a = rs.standard_normal((8, 70000)).astype(np.float32)          # rows too long to hold
    da = dr.array(a)
    got, n = launches(lambda: (da - da.max(axis=1, keepdims=True)).get())
    assert n >= 2 and bits_equal(got, a - a.max(axis=1, keepdims=True))
    b = rs.standard_normal((300, 40))
    db = dr.array(b)
    got = (db - db.max(axis=0, keepdims=True)).get()                # not along the rows
    assert bits_equal(got, b - b.max(axis=0, keepdims=True))
    t = dr.array(rs.standard_normal((64, 96)))
    ht = t.get()
    got = (t.T - t.T.max(axis=1, keepdims=True)).get()              # rows without unit stride
    assert bits_equal(got, ht.T - ht.T.max(axis=1, keepdims=True))
    i = dr.array(rs.randint(0, 100, (20, 30)))
    hi = i.get()
    got = (i - i.max(axis=1, keepdims=True)).get()                  # integers
    assert np.array_equal(got, hi - hi.max(axis=1, keepdims=True))
    wide = dr.array(rs.standard_normal((16, 64)))
    hw = wide.get()
    other = dr.array(rs.standard_normal((16, 1)))
    ho = other.get()
    got = (other * 2.0 + wide.sum(axis=1, keepdims=True)).get()     # nothing left that has rows
    np.testing.assert_allclose(got, ho * 2.0 + hw.sum(axis=1, keepdims=True), rtol=1e-13)


def test_the_unfused_mode_and_the_tunables_agree():
    rs = np.random.RandomState(11)
    a = rs.standard_normal((70, 5000)).astype(np.float32)
    ref = softmax(np, a)
    base = softmax(dr, dr.array(a)).get()
    for tune in (dict(row_recompute=0), dict(row_fence=0), dict(row_regs=0), dict(row_lanes=64),
                 dict(row_lanes=256, row_bpc=2), dict(rowfuse=0), dict(row_pipe=0), dict(row_carry=0),
                 dict(row_wavemap=1), dict(row_wavemap=0, row_lanes=256)):
        old = {k: hip.TUNE[k] for k in tune}
        hip.set_tune(**tune)
        try:
            got = softmax(dr, dr.array(a)).get()
        finally:
            hip.set_tune(**old)
        np.testing.assert_allclose(got, ref, rtol=2e-6)
        if not {"row_lanes", "rowfuse", "row_wavemap"} & set(tune):
            assert bits_equal(got, base), tune      # same order of additions
    hip.set_fused(False)
    try:
        got = softmax(dr, dr.array(a)).get()
    finally:
        hip.set_fused(True)
    np.testing.assert_allclose(got, ref, rtol=2e-6)


def test_softmax_full_size():
    """16384 rows of 16384 float32: every row sums to one, agrees with NumPy on sampled rows."""
    rs = np.random.RandomState(12)
    a = rs.standard_normal((16384, 16384)).astype(np.float32)
    got, n = launches(lambda: softmax(dr, dr.array(a)).get())
    assert n == 1
    np.testing.assert_allclose(got.sum(axis=1, dtype=np.float64), 1.0, rtol=1e-5)
    rows = rs.randint(0, 16384, 64)
    np.testing.assert_allclose(got[rows], softmax(np, a[rows]), rtol=2e-6)
    assert np.array_equal(got.argmax(axis=1), a.argmax(axis=1))


# ---- seeded random expressions with row maxima and minima inside ----------------------------

def _fuzz_leaf(rs, shape):
    """(lazy leaf, host array) of a shape that broadcasts to `shape`: dense, a view with a row
    pitch, one row for all, one value per row, every second column (which the row kernel
    does not take: the reductions are then evaluated on their own)."""
    dtype = [np.float32, np.float64][rs.randint(2)]
    rows, R = shape
    kind = rs.randint(7)

    def host(s):
        v = rs.uniform(-2, 2, s)
        v[rs.uniform(size=s) < 0.02] = 0.0
        return v.astype(dtype)
    if kind == 3:
        h = host((rows, R + 5))
        lo = int(rs.randint(0, 6))
        return dr.array(h)[:, lo:lo + R], h[:, lo:lo + R]
    if kind == 4:
        h = host((1, R))
        return dr.array(h), h
    if kind == 5:
        h = host((rows, 1))
        return dr.array(h), h
    if kind == 6 and R * 2 * rows < (1 << 22):
        h = host((rows, 2 * R))
        return dr.array(h)[:, ::2], h[:, ::2]
    h = host(shape)
    return dr.array(h), h


_FUZZ_UNARY = [np.negative, np.absolute, lambda x: x * x, lambda x: 0.5 * x, lambda x: x + 1, lambda x: 3 - x,
               lambda x: np.sqrt(np.absolute(x))]
_FUZZ_BINARY = [np.add, np.subtract, np.multiply, np.true_divide, np.maximum, np.minimum,
                lambda a, b: np.where(a > b, a, b * 2)]


def _fuzz_expr(rs, shape, depth, reductions):
    """Random expression; with probability growing towards the root a sub-expression is
    replaced by its maximum or minimum along the row (exact, whatever the order)."""
    if depth == 0:
        return _fuzz_leaf(rs, shape)
    if reductions and rs.uniform() < 0.3:
        d, o = _fuzz_expr(rs, shape, depth - 1, reductions - 1)
        if o.shape != shape:        # reduce something that has whole rows
            d2, o2 = _fuzz_leaf(rs, shape)
            while o2.shape != shape:
                d2, o2 = _fuzz_leaf(rs, shape)
            d, o = d + d2, o + o2
        if rs.randint(2):
            return d.max(axis=-1, keepdims=True), o.max(axis=-1, keepdims=True)
        return d.min(axis=-1, keepdims=True), o.min(axis=-1, keepdims=True)
    if rs.uniform() < 0.3:
        fn = _FUZZ_UNARY[rs.randint(len(_FUZZ_UNARY))]
        d, o = _fuzz_expr(rs, shape, depth - 1, reductions)
        return fn(d), fn(o)
    fn = _FUZZ_BINARY[rs.randint(len(_FUZZ_BINARY))]
    d1, o1 = _fuzz_expr(rs, shape, depth - 1, reductions)
    d2, o2 = _fuzz_expr(rs, shape, depth - 1, reductions)
    return fn(d1, d2), fn(o1, o2)


@pytest.mark.parametrize("seed", range(80))
def test_random_expressions_with_row_maxima_inside_are_bit_equal(seed):
    rs = np.random.RandomState(7000 + seed)
    shape = (int(rs.choice([1, 3, 64, 130, 1000])),
             int(rs.choice([2, 3, 5, 16, 33, 64, 100, 257, 1000, 4099, 9000, 20000])))
    if shape[0] * shape[1] > (1 << 22):
        shape = (64, shape[1])
    with np.errstate(all="ignore"):
        d, o = _fuzz_expr(rs, shape, depth=int(rs.randint(2, 6)), reductions=3)
        anchor_d, anchor_o = _fuzz_leaf(rs, shape)
        d, o = d + anchor_d, o + anchor_o
        got = d.get()
    ref = np.broadcast_to(o, got.shape) if o.shape != got.shape else o
    assert got.shape == np.broadcast_shapes(o.shape, got.shape) and bits_equal(got, np.asarray(ref)), (seed, shape)


def test_the_random_expressions_reached_the_row_kernel():
    """Runs after the cases above: many of them must have taken the row kernel, in
    several lane-group sizes, and some the fallback (reductions evaluated on their own)."""
    groups = {}
    for key in hip._KERNELS:
        if key[0] == "rows":
            groups[key[6]] = groups.get(key[6], 0) + 1
    print("row kernels by lanes per row:", groups)
    assert sum(groups.values()) >= 20 and len(groups) >= 4, groups


def test_the_usual_spellings_of_a_normalisation_are_one_kernel_too():
    """`a.sum(axis=1)` stays lazy; `[:, None]`, `.reshape(-1, 1)` and `expand_dims(..., -1)`
    turn it into its kept twin, so these expressions take the row kernel like their
    `keepdims=True` forms; used in any other way the reduction is evaluated on its own."""
    rs = np.random.RandomState(8)
    a = rs.uniform(0.5, 2.0, (300, 1000)).astype(np.float32)
    da = dr.array(a)
    got, n = launches(lambda: (da / da.sum(axis=1)[:, None]).get())
    assert n == 1
    np.testing.assert_allclose(got, a / a.sum(axis=1)[:, None], rtol=2e-6)
    got, n = launches(lambda: (da - da.max(axis=1).reshape(-1, 1)).get())
    assert n == 1 and bits_equal(got, a - a.max(axis=1).reshape(-1, 1))
    got, n = launches(lambda: (da - np.expand_dims(da.min(axis=-1), -1) * 2.0).get())
    assert n == 1 and bits_equal(got, a - np.expand_dims(a.min(axis=-1), -1) * 2.0)
    e = np.exp(da - da.max(axis=1)[:, None])
    got, n = launches(lambda: (e / e.sum(axis=1)[:, None]).get())
    ref = np.exp(a - a.max(axis=1)[:, None])
    assert n == 1
    np.testing.assert_allclose(got, ref / ref.sum(axis=1)[:, None], rtol=2e-6)
    # on its own, sliced, or inside an expression of its own shape: evaluated as before
    s = da.sum(axis=1)
    np.testing.assert_allclose(s.get(), a.sum(axis=1), rtol=1e-5)
    np.testing.assert_allclose((s * 2 + 1)[5:9].get(), (a.sum(axis=1) * 2 + 1)[5:9], rtol=1e-5)
    assert bits_equal(da.max(axis=1).get(), a.max(axis=1))
    t3 = rs.standard_normal((7, 9, 130))
    d3 = dr.array(t3)
    got, n = launches(lambda: (d3 - d3.max(axis=-1)[..., None]).get())
    assert n == 1 and bits_equal(got, t3 - t3.max(axis=-1)[..., None])


def test_rows_held_by_a_block_of_512_lanes_replay_with_that_block():
    """Rows of 64 to 256 KB take a block of 512 lanes; recorded launches and the HIP graph
    made of them must launch that many (a replay with 256 would leave half of every row
    unwritten)."""
    rs = np.random.RandomState(12)
    a = rs.standard_normal((24, 50257)).astype(np.float32)
    b = rs.standard_normal((24, 50257)).astype(np.float32)
    da = dr.array(a)
    low, src = hip.lower_only(softmax(dr, da))
    assert low.kind == "rows" and lowering.block_lanes(low) == 512 and "__launch_bounds__(512)" in src
    with hip.record() as rep:
        out = hip.run(softmax(dr, da))
    assert len(rep.launches) == 1
    ref = softmax(np, a)
    np.testing.assert_allclose(out.get(), ref, rtol=2e-6)
    da[...] = b                                        # same buffers, new values
    rep()
    np.testing.assert_allclose(out.get(), softmax(np, b), rtol=2e-6)
    rep.as_graph()
    for k in range(3):
        da[...] = (a, b)[k % 2]
        rep()
        hip.synchronize()
        np.testing.assert_allclose(out.get(), (ref, softmax(np, b))[k % 2], rtol=2e-6)
    # fresh arrays through the same expression: plans made from the remembered structure
    hits = hip.STATS["seen_hits"]
    for k in range(6):
        h = rs.standard_normal((24, 50257)).astype(np.float32)
        got, n = launches(lambda: softmax(dr, dr.array(h)).get())
        assert n == 1
        np.testing.assert_allclose(got, softmax(np, h), rtol=2e-6)
    assert hip.STATS["seen_hits"] > hits


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_values_computed_once_per_row_give_the_same_bits_as_per_element(dtype):
    """The mean `sum / n`, `sqrt(var + eps)`, `log(sum)` are the same along a row: computed
    once per row and handed to the per-element work, or computed for every element
    (`row_hoist=0`), the results are the same bits; both agree with NumPy."""
    rs = np.random.RandomState(13)
    a = (rs.standard_normal((40, 3001)) * 2 + 1).astype(dtype)
    w = rs.standard_normal(3001).astype(dtype)
    col = rs.standard_normal((40, 1)).astype(dtype)

    def layer_norm(xp, x, g):
        mu = x.mean(axis=-1, keepdims=True)
        d = x - mu
        return d / xp.sqrt((d * d).mean(axis=-1, keepdims=True) + 1e-5) * g

    def log_softmax(xp, x, g):
        s = x - x.max(axis=-1, keepdims=True)
        return s - xp.log(xp.exp(s).sum(axis=-1, keepdims=True))

    def scaled(xp, x, g, c):            # a value per row that no reduction feeds: level 0
        return x * xp.exp(c) + x.sum(axis=-1, keepdims=True) / xp.exp(c)
    tol = dict(rtol=3e-5, atol=3e-5) if dtype == np.float32 else dict(rtol=1e-11, atol=1e-11)
    for fn, extra in ((layer_norm, ()), (log_softmax, ()), (scaled, (col,))):
        got = {}
        for hoist in (1, 0):
            # the same lanes per row both times (the choice counts per-element work, which
            # differs between the two, and the order of a sum follows the lanes)
            hip.set_tune(row_hoist=hoist, row_lanes=256)
            try:
                args = [dr.array(a), dr.array(w)] + [dr.array(e) for e in extra]
                low, src = hip.lower_only(fn(dr, *args))
                assert low.kind == "rows" and ("dr_once" in src) == bool(hoist), fn.__name__
                got[hoist], n = launches(lambda: fn(dr, *args).get())
                assert n == 1
            finally:
                hip.set_tune(row_hoist=1, row_lanes=0)
        assert bits_equal(got[0], got[1]), fn.__name__
        np.testing.assert_allclose(got[1], fn(np, a, w, *extra), **tol)


def test_rows_beyond_2_to_31_elements():
    """Row kernels address with 64 bits: 70000 rows of 32768 float32 (2.29e9 elements,
    9.2 GB in, 9.2 GB out, a block of 512 lanes per row); rows on both sides of the
    2^31-element boundary and the last row agree with NumPy."""
    K, R = 70000, 32768
    rs = np.random.RandomState(14)
    x = dr.zeros((K, R), dtype=np.float32)
    edge = (1 << 31) // R                       # first row that starts at element 2^31
    picked = {0: None, edge - 1: None, edge: None, edge + 1: None, K - 1: None}
    for k in picked:
        picked[k] = rs.standard_normal(R).astype(np.float32)
        x[k] = picked[k]
    out, n = launches(lambda: hip.run(softmax(dr, x)))
    assert n == 1 and out.shape == (K, R)
    for k, row in picked.items():
        np.testing.assert_allclose(out[k].get(), softmax(np, row[None])[0], rtol=2e-6, err_msg=str(k))
    np.testing.assert_allclose(out[edge + 7].get(), np.full(R, 1.0 / R, np.float32), rtol=1e-6)
    del out
    small, n = launches(lambda: hip.run(x[:, :96] - x[:, :96].max(axis=1, keepdims=True)))
    assert n == 1                               # lane groups, rows 128 KB apart
    for k, row in picked.items():
        assert bits_equal(small[k].get(), row[:96] - row[:96].max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_operands_repeated_over_a_batch_stay_in_the_row_kernel(dtype):
    """`softmax(scores + mask)` with a mask per (row, column) shared by every item of the
    batch, `layer_norm(x + positions)`, a vector per batch item: the rows are counted over two
    levels (batch, row) that the repeated operand does not walk as one sequence; one
    kernel, which splits the row number."""
    rs = np.random.RandomState(15)
    B, N = 6, 37
    for R in (40, 257, 1000, 5000):
        x = rs.standard_normal((B, N, R)).astype(dtype)
        mask = np.where(rs.uniform(size=(N, R)) < 0.2, -np.inf, 0.0).astype(dtype)
        mask[:, 0] = 0.0                                       # no row without a finite entry
        pos = rs.standard_normal((N, R)).astype(dtype)
        per_item = rs.standard_normal((B, 1, R)).astype(dtype)
        dx, dm, dp, dv = dr.array(x), dr.array(mask), dr.array(pos), dr.array(per_item)
        got, n = launches(lambda: softmax(dr, dx + dm).get())
        assert n == 1, R
        np.testing.assert_allclose(got, softmax(np, x + mask), rtol=2e-6 if dtype == np.float32 else 1e-13)
        got, n = launches(lambda: ((dx + dp) - (dx + dp).max(axis=-1, keepdims=True)).get())
        assert n == 1 and bits_equal(got, (x + pos) - (x + pos).max(axis=-1, keepdims=True))
        got, n = launches(lambda: ((dx * dv + dp) - (dx * dv + dp).min(axis=-1, keepdims=True)).get())
        ref = (x * per_item + pos) - (x * per_item + pos).min(axis=-1, keepdims=True)
        assert n == 1 and bits_equal(got, ref)

        def layer_norm(xp, a, p):
            s = a + p
            d = s - s.mean(axis=-1, keepdims=True)
            return d / xp.sqrt((d * d).mean(axis=-1, keepdims=True) + 1e-5)
        got, n = launches(lambda: layer_norm(dr, dx, dp).get())
        assert n == 1
        tol = dict(rtol=3e-5, atol=3e-5) if dtype == np.float32 else dict(rtol=1e-11, atol=1e-11)
        np.testing.assert_allclose(got, layer_norm(np, x, pos), **tol)
        # the batch as a view: every second item, rows still two levels
        got, n = launches(lambda: softmax(dr, dx[::2] + dm).get())
        assert n == 1
        np.testing.assert_allclose(got, softmax(np, x[::2] + mask), rtol=2e-6 if dtype == np.float32 else 1e-13)
    # three levels that do not merge: the long way, same values
    y = rs.standard_normal((3, 4, 5, 64)).astype(dtype)
    m2 = rs.standard_normal((4, 1, 64)).astype(dtype)
    dy, dm2 = dr.array(y), dr.array(m2)
    got = ((dy + dm2) - (dy + dm2).max(axis=-1, keepdims=True)).get()
    assert bits_equal(got, (y + m2) - (y + m2).max(axis=-1, keepdims=True))


def test_masks_that_are_the_same_along_a_row():
    """`where(row maximum > 0, a / maximum, a)`, a mask per row from a vector: the per-row
    comparison is a byte computed once per row; bit-equal to NumPy."""
    rs = np.random.RandomState(19)
    a = rs.standard_normal((500, 300)).astype(np.float32)
    a[::7] -= 10.0                                         # rows whose maximum is negative
    da = dr.array(a)
    mx, hmx = da.max(axis=1, keepdims=True), a.max(axis=1, keepdims=True)
    got, n = launches(lambda: np.where(mx > 0, da / mx, da).get())
    assert n == 1 and bits_equal(got, np.where(hmx > 0, a / hmx, a))
    got, n = launches(lambda: (np.where(da.min(axis=1, keepdims=True) < -3, da, -da) * (mx > 1)).get())
    assert n == 1 and bits_equal(got, np.where(a.min(axis=1, keepdims=True) < -3, a, -a) * (hmx > 1))
    w = rs.standard_normal(100003).astype(np.float32)
    x = rs.standard_normal((100003, 3)).astype(np.float32)
    got, n = launches(lambda: np.where((dr.array(w) > 0)[:, None], dr.array(x), 0.0).get())
    assert n == 1 and bits_equal(got, np.where((w > 0)[:, None], x, np.float32(0.0)))
