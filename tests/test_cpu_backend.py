"""The `DELAY_CPU` backend (NumPy node by node, like the reference's cpu.py), which
is chosen at import time and therefore runs in a child process."""
import os
import subprocess
import sys
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCRIPT = textwrap.dedent("""
    import numpy as np
    import delayrepay as dnp
    from delayrepay import NPArray, array, full, ones, sum
    assert dnp.backend.__name__.endswith(".cpu")

    # reference tests/test.py:21-67 on the NumPy backend
    arr, np_arr = ones(64), np.ones(64)
    assert isinstance(arr + 1, dnp.DelayArray) and "array" not in (arr + 1).__dict__
    assert np.array_equal((arr + 1).get(), np_arr + 1)
    assert np.array_equal((8 * arr + 9).get(), 8 * np_arr + 9)
    assert np.array_equal((arr + arr * 3 + 9).get(), np_arr + np_arr * 3 + 9)
    assert np.array_equal(np.cos(arr).get(), np.cos(np_arr))
    a32 = arr.astype(np.float32)
    assert (a32 ** 2).get().dtype == np.float32
    x = np.random.RandomState(0).uniform(-3, 3, 1000).astype(np.float32)
    assert (array(x) ** 3).get().tobytes() == ((x * x) * x).tobytes()      # delayarray.py:316-324
    assert np.array_equal((np.sin(arr) ** 2 + np.cos(arr) ** 2).get(),
                          np.sin(np_arr) * np.sin(np_arr) + np.cos(np_arr) * np.cos(np_arr))
    # tests/test.py:70-111
    v, w = full((64,), 7).astype(np.float32), full((64,), 3).astype(np.float32)
    assert np.all((v + w).get() == 10) and np.all((v * w).get() == 21)
    assert sum(v) == 448 and float(v.dot(w)) == 7 * 3 * 64 and float(v @ w) == 1344
    m = full((64, 64), 7).astype(np.float32)
    assert np.array_equal((m @ v).get(), np.full((64, 64), 7, np.float32) @ np.full(64, 7, np.float32))
    # tests/test.py:143-162
    raw = np.array([1, 2, 3])
    assert NPArray(raw) is NPArray(raw)
    z = array([1, 2, 3])
    assert np.sin(z) is np.sin(z)

    # slices, fused assignment, reductions, several roots: same front end, NumPy underneath
    u0 = np.zeros((20, 30), np.float32)
    u0[1:-1, 1:-1] = np.random.RandomState(1).uniform(0, 1, (18, 28))
    u, ref = array(u0.copy()), u0.copy()
    for _ in range(3):
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
        ref[1:-1, 1:-1] = 0.25 * (ref[:-2, 1:-1] + ref[2:, 1:-1] + ref[1:-1, :-2] + ref[1:-1, 2:])
    assert u.get().tobytes() == ref.tobytes()
    a = array(np.arange(12.0).reshape(3, 4))
    assert np.array_equal(dnp.sum(a * 2, axis=0).get(), (np.arange(12.0).reshape(3, 4) * 2).sum(axis=0))
    assert float(dnp.mean(a)) == 5.5 and float(dnp.max(a)) == 11
    p, q = dnp.evaluate(a + 1, a * 2)
    assert np.array_equal(p.get(), np.arange(12.0).reshape(3, 4) + 1)
    assert np.array_equal(np.where(a > 5, a, 0.0).get(), np.where(np.arange(12.0).reshape(3, 4) > 5,
                                                                   np.arange(12.0).reshape(3, 4), 0.0))

    # the device generator's stream is NumPy's Philox stream, call after call
    gen, ref = dnp.random.device(99), np.random.Generator(np.random.Philox(key=99))
    for size in (5, 4096, 3, (6, 7)):
        assert np.array_equal(gen.random(size).get(), ref.random(size))
    assert np.array_equal(gen.uniform(-3.0, 5.0, 1001).get(), ref.uniform(-3.0, 5.0, 1001))
    raw = gen.random_raw(10).get()
    assert raw.dtype == np.int64 and np.array_equal(raw.view(np.uint64), ref.bit_generator.random_raw(10))
    # float32: two numbers from every output, the low half first; the high half of the last
    # output waits for the next float32 draw, whatever else is drawn in between
    gen, ref = dnp.random.device(5), np.random.Generator(np.random.Philox(key=5))
    for size, dt in ((7, np.float32), (3, np.float64), (4, np.float32), (1001, np.float32), (2, np.float64),
                     ((5, 3), np.float32), (1, np.float32), (64, np.float32)):
        got, want = gen.random(size, dtype=dt).get(), ref.random(size, dtype=dt)
        assert got.dtype == want.dtype and np.array_equal(got, want), (size, dt)
    big = dnp.random.device(3, counter=(1 << 256) - 2)
    assert np.array_equal(big.random(20).get(),
                          np.random.Generator(np.random.Philox(key=3, counter=(1 << 256) - 2)).random(20))

    # generated leaves: long constant / index arrays stay lazy and give NumPy's exact bits
    from delayrepay.delayarray import FullEx, WhereEx, BinaryNumpyEx
    same = lambda got, ref: (got.dtype == ref.dtype and got.shape == ref.shape
                             and got.tobytes() == ref.tobytes())
    for args in [(10000,), (3, 20000), (0.0, 1000.0, 0.1), (1.5, 9000.25, 0.7), (5000, 0, -1),
                 (10.0, -700.0, -0.07), (0.1, 1e4, 0.3)]:
        for kw in ({}, {"dtype": np.float32}, {"dtype": np.float64}, {"dtype": np.int64}):
            if kw.get("dtype") == np.int64 and any(isinstance(v, float) for v in args):
                continue
            lazy = dnp.arange(*args, **kw)
            assert type(lazy) in (WhereEx, BinaryNumpyEx), (args, kw)
            assert same(lazy.get(), np.arange(*args, **kw)), (args, kw)
    for lo, hi, n, ep in [(0, 1, 10000, True), (-2.0, 2.0, 65537, True), (0.1, 1e6, 5000, False),
                          (3, -3, 4096, True)]:
        for dt in (None, np.float32, np.float64):
            lazy = dnp.linspace(lo, hi, n, endpoint=ep, dtype=dt)
            assert not isinstance(lazy, NPArray)
            assert same(lazy.get(), np.linspace(lo, hi, n, endpoint=ep, dtype=dt)), (lo, hi, n, ep, dt)
    assert isinstance(dnp.arange(10), NPArray) and isinstance(dnp.linspace(0, 1, 50), NPArray)
    assert isinstance(dnp.arange(np.float32(0), 9000), NPArray)          # NumPy scalars: eager
    assert same(dnp.linspace(0, 1, 5000, retstep=False, dtype=np.int64).get(),
                np.linspace(0, 1, 5000, dtype=np.int64))
    z = dnp.zeros((100, 100))
    assert type(z) is FullEx and z.shape == (100, 100) and z.dtype == np.float64
    assert dnp.zeros((100, 100)) is not z                                 # never shared
    y = z + 1.5
    assert same(y.get(), np.full((100, 100), 1.5))
    z[1:3, 1:3] = 7.0                                                     # becomes a real array
    expect = np.zeros((100, 100)); expect[1:3, 1:3] = 7.0
    assert same(z.get(), expect) and same((z + 1).get(), expect + 1)
    assert same(dnp.ones_like(y).get(), np.ones((100, 100)))
    assert same(dnp.full((5000,), 3, dtype=np.int32).get(), np.full(5000, 3, np.int32))
    assert same(dnp.full_like(y, 2.5, dtype=np.float32).get(), np.full((100, 100), 2.5, np.float32))
    assert isinstance(dnp.zeros(8), NPArray) and isinstance(dnp.full((3,), "a"), NPArray)

    # views of unevaluated expressions are the expression over views of its leaves
    rs = np.random.RandomState(2)
    ha, hb = rs.uniform(-1, 1, (50, 70)), rs.uniform(-1, 1, 70)
    A, B = array(ha), array(hb)
    e, ref = A * 2 + B, ha * 2 + hb
    r = e[1:-1, ::2]
    assert not isinstance(r, NPArray) and r.shape == (48, 35) and "array" not in e.__dict__
    assert same(r.get(), ref[1:-1, ::2]) and same(e[3].get(), ref[3])
    assert same(e[:, None, 5].get(), ref[:, None, 5]) and same(e[..., -1].get(), ref[..., -1])
    assert same(e.T.get(), ref.T) and same(np.transpose(e, (1, 0))[2:4].get(), ref.T[2:4])
    assert same(np.roll(e, 7, axis=1).get(), np.roll(ref, 7, axis=1))
    assert same(np.roll(e, -3, axis=0).get(), np.roll(ref, -3, axis=0))
    assert same(np.roll(A[0] + 1, 5).get(), np.roll(ha[0] + 1, 5)) and "array" not in e.__dict__
    s1, r1 = A + 1, ha + 1
    lap = s1[:-2, 1:-1] + s1[2:, 1:-1] + s1[1:-1, :-2] + s1[1:-1, 2:]
    assert same(lap.get(), r1[:-2, 1:-1] + r1[2:, 1:-1] + r1[1:-1, :-2] + r1[1:-1, 2:])
    assert "array" not in s1.__dict__
    assert same((dnp.zeros((50, 70)) + A)[2:5].get(), ha[2:5])
    big = A
    for _ in range(60):
        big = big + 1.0
    assert isinstance(big[1:3], NPArray) and "array" in big.__dict__       # too large: evaluated once
    # out= on a ufunc writes into the destination and returns it (tests/test.py has no such case;
    # the reference ignores the keyword, delayarray.py:46-61)
    dst, src = array(np.zeros(64)), array(np.arange(64.0))
    back = np.multiply(src, 3.0, out=dst)
    assert back is dst and np.array_equal(dst.get(), np.arange(64.0) * 3.0)
    assert np.sqrt(src, out=dst) is dst and np.array_equal(dst.get(), np.sqrt(np.arange(64.0)))
    try:
        np.add(src, 1.0, out=array(np.zeros(64, dtype=np.int32)))
        raise SystemExit("a float result must not be cast into an integer destination")
    except TypeError:
        pass
    # any / all / count_nonzero / std / isclose / allclose / linalg.norm: compositions of the
    # fused reductions (none is registered by the reference, delayarray.py:485-615)
    h0 = np.random.RandomState(3).standard_normal((50, 70))
    h1 = h0 + 1e-9
    d0, d1 = array(h0), array(h1)
    assert bool(np.any(d0 > 3)) == (h0 > 3).any() and bool(np.all(d0 > -5)) == (h0 > -5).all()
    assert np.array_equal(np.any(d0 > 2, axis=1).get(), (h0 > 2).any(axis=1))
    assert np.array_equal(np.all(d0 > -2, axis=0).get(), (h0 > -2).all(axis=0))
    assert np.allclose(d0, d1) is True and np.allclose(d0, d1 + 1) is False
    assert np.array_equal(np.isclose(d0, d1, rtol=0, atol=5e-10).get(), np.isclose(h0, h1, rtol=0, atol=5e-10))
    assert abs(float(np.linalg.norm(d0)) - np.linalg.norm(h0)) < 1e-12
    assert np.allclose(np.linalg.norm(d0, axis=1).get(), np.linalg.norm(h0, axis=1), rtol=1e-14)
    assert abs(float(np.std(d0)) - h0.std()) < 1e-14 and int(np.count_nonzero(d0 > 0)) == np.count_nonzero(h0 > 0)
    # flips, differences, axis manipulation, concatenation: indexing, arithmetic and fused writes
    rs_ = np.random.RandomState(0)
    h, g = rs_.standard_normal((4, 5, 6)), rs_.standard_normal((4, 5, 6))
    a, b = array(h), array(g)
    eq = lambda x, y: np.array_equal(x.get(), y)
    assert eq(np.flip(a), np.flip(h)) and eq(np.flip(a + 1, (0, 2)), np.flip(h + 1, (0, 2)))
    assert eq(np.flipud(a), np.flipud(h)) and eq(np.fliplr(a), np.fliplr(h))
    assert eq(np.diff(a), np.diff(h)) and eq(np.diff(a * 2, n=2, axis=0), np.diff(h * 2, n=2, axis=0))
    assert eq(np.diff(a > 0, axis=1), np.diff(h > 0, axis=1))
    assert eq(np.outer(a[0, 0], b[1, 1]), np.outer(h[0, 0], g[1, 1])) and eq(np.ptp(a, axis=1), np.ptp(h, axis=1))
    assert eq(np.expand_dims(a + b, (0, -1)), np.expand_dims(h + g, (0, -1)))
    assert eq(np.squeeze(np.expand_dims(a, 2)), h) and eq(np.squeeze(a[:1] * 2, axis=0), h[0] * 2)
    assert eq(np.swapaxes(a, 0, 2), np.swapaxes(h, 0, 2))
    assert eq(np.moveaxis(a + 1, (0, 1), (2, 0)), np.moveaxis(h + 1, (0, 1), (2, 0)))
    assert eq(np.reshape(a, (20, 6)), h.reshape(20, 6)) and eq(np.ravel(a * b), (h * g).ravel())
    assert eq(np.concatenate([a, b * 2, a + b], axis=1), np.concatenate([h, g * 2, h + g], axis=1))
    assert eq(np.concatenate([a, b], axis=None), np.concatenate([h, g], axis=None))
    mixed = np.concatenate([a, b.astype(np.float32)], axis=-1)
    assert mixed.dtype == np.float64 and eq(mixed, np.concatenate([h, g.astype(np.float32)], axis=-1))
    assert eq(np.stack([a, b + 1], axis=2), np.stack([h, g + 1], axis=2))
    assert eq(np.vstack([a[0, 0], b[0, 0]]), np.vstack([h[0, 0], g[0, 0]]))
    assert eq(np.hstack([a[0], b[0]]), np.hstack([h[0], g[0]]))
    # ndarray's methods on lazy arrays
    hm = np.random.RandomState(4).standard_normal((5, 7))
    am = array(hm)
    assert abs(float(am.std()) - hm.std()) < 1e-14 and bool((am > -9).all()) and not bool((am > 9).any())
    assert np.array_equal(am.clip(-1, 1).get(), hm.clip(-1, 1)) and np.array_equal(am.cumsum().get(), hm.cumsum())
    assert np.array_equal(am.swapaxes(0, 1).get(), hm.T) and np.array_equal(am[:1].squeeze().get(), hm[0])
    assert am[1, 2].item() == hm[1, 2] and am.tolist() == hm.tolist() and am.nbytes == hm.nbytes
    bm = array(np.zeros(8))
    bm.fill(3.5)
    assert np.all(bm.get() == 3.5) and float(am.ptp()) == np.ptp(hm)
    # a loop of x = f(x) that never asks for a value: the expression stops growing at
    # MAX_DEPTH operations (its deepest operand is evaluated), so nothing recurses too far
    x, hx = array(np.full(32, 1.0)), np.full(32, 1.0)
    for _ in range(3000):
        x, hx = x * 0.999 + 0.5, hx * 0.999 + 0.5
        assert x._depth <= dnp.delayarray.MAX_DEPTH
    assert "array" not in x.__dict__ and np.array_equal(x.get(), hx)
    print("cpu-backend-ok")
""")


def run_cpu(script):
    """stdout of `script` run under DELAY_CPU in a child process."""
    env = dict(os.environ, DELAY_CPU="1", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", textwrap.dedent(script)], env=env, capture_output=True,
                         text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-3000:]
    return out.stdout


def test_delay_cpu_backend_runs_the_reference_suite():
    env = dict(os.environ, DELAY_CPU="1", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", SCRIPT], env=env, capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "cpu-backend-ok" in out.stdout


def test_hip_backend_is_the_default_and_fails_loudly_without_the_library(tmp_path):
    """No silent host fall-back: without libdrhip.so the default backend refuses to import."""
    pkg = tmp_path / "delayrepay_amd"
    pkg.mkdir()
    for name in os.listdir(os.path.join(ROOT, "delayrepay_amd")):
        if name.endswith(".py"):
            (pkg / name).write_text(open(os.path.join(ROOT, "delayrepay_amd", name)).read())
    env = {k: v for k, v in os.environ.items() if k != "DELAY_CPU"}
    env["PYTHONPATH"] = str(tmp_path)
    out = subprocess.run([sys.executable, "-c", "import delayrepay_amd"], env=env, cwd=str(tmp_path),
                         capture_output=True, text=True, timeout=300)
    assert out.returncode != 0
    assert "libdrhip.so is missing" in out.stderr and "no host fall-back" in out.stderr


def test_reductions_that_keep_their_axis_stay_lazy_and_give_numpys_values():
    """`a.max(axis=-1, keepdims=True)` of a float array is a node, not a value: the HIP
    backend fuses it with what is built on it; this backend applies NumPy's reduction."""
    script = r"""
import numpy as np
import delayrepay_amd as dr
from delayrepay_amd.delayarray import ReduceEx, DelayArray
rs = np.random.RandomState(0)
a = rs.standard_normal((13, 57))
da = dr.array(a)
m = da.max(axis=1, keepdims=True)
assert isinstance(m, ReduceEx) and m.shape == (13, 1) and "array" not in m.__dict__
e = np.exp(da - m)
sm = e / e.sum(axis=-1, keepdims=True)
ref_e = np.exp(a - a.max(axis=1, keepdims=True))
assert np.array_equal(sm.get(), ref_e / ref_e.sum(axis=-1, keepdims=True))
assert np.array_equal(m.get(), a.max(axis=1, keepdims=True))
assert np.array_equal(dr.var(da, axis=1).get(), ((a - a.mean(axis=1, keepdims=True)) ** 2).sum(axis=1) / 57)
assert np.allclose(dr.std(da, axis=1, keepdims=True).get(), a.std(axis=1, keepdims=True), rtol=1e-14)
# not along the last axis, integers: evaluated at once, as before
assert not isinstance(da.max(axis=0, keepdims=True), ReduceEx)
assert not isinstance(dr.array(np.arange(12).reshape(3, 4)).max(axis=1, keepdims=True), ReduceEx)
# along the last axis without keepdims: lazy too, and putting the axis back gives the kept twin,
# so the usual spellings of a normalisation fuse as well
s = da.sum(axis=1)
assert isinstance(s, ReduceEx) and s.shape == (13,) and "array" not in s.__dict__
for kept in (s[:, None], s[..., None], s[:, np.newaxis], s.reshape(-1, 1), s.reshape(13, 1), np.expand_dims(s, -1),
             np.expand_dims(s, 1)):
    assert isinstance(kept, ReduceEx) and kept.keepdims and kept.shape == (13, 1) and kept is s[:, None]
assert "array" not in s.__dict__
assert np.array_equal((da / da.sum(axis=1)[:, None]).get(), a / a.sum(axis=1)[:, None])
assert np.array_equal((da - da.mean(axis=1).reshape(-1, 1)).get(), a - a.mean(axis=1).reshape(-1, 1))
mx = (da.max(axis=1) * 2.0)[:, None]            # an expression over the reduction
assert isinstance(mx, DelayArray) and mx.shape == (13, 1) and "array" not in mx.__dict__
assert np.array_equal((da - mx).get(), a - (a.max(axis=1) * 2.0)[:, None])
assert np.array_equal(s.get(), a.sum(axis=1)) and np.array_equal(s[3:7].get(), a.sum(axis=1)[3:7])
assert np.array_equal((s * 2 + 1).get(), a.sum(axis=1) * 2 + 1) and float(s[2]) == a.sum(axis=1)[2]
t3 = dr.array(rs.standard_normal((3, 4, 5)))
assert np.array_equal((t3 / t3.sum(axis=-1)[..., None]).get(), t3.get() / t3.get().sum(axis=-1)[..., None])
# keywords that change the result are refused, not dropped
for call in (lambda: np.sum(da, initial=10.0), lambda: np.any(da, where=np.ones((13, 57), bool)),
             lambda: np.max(da, initial=0.0)):
    try:
        call()
    except NotImplementedError:
        pass
    else:
        raise AssertionError("keyword accepted")
assert np.sum(da, where=True) == a.sum()
# any / all of nothing
z = dr.array(np.zeros((0, 4)))
assert bool(np.any(z)) is False and bool(np.all(z)) is True
assert np.array_equal(np.all(z, axis=0).get(), np.ones(4, bool))
assert np.array_equal(np.any(z, axis=0, keepdims=True).get(), np.zeros((1, 4), bool))
print("ok")
"""
    assert run_cpu(script).strip().endswith("ok")


def test_a_result_written_to_by_hand_is_an_array_of_its_own():
    """After `b = a * 2; b[0] = 100` the node of `a * 2` holds a value that is no longer
    `a * 2`: the same expression built again is a new node, and what is built on `b` sees
    the write (this backend walks through evaluated nodes; it must stop at this one)."""
    script = r"""
    import numpy as np
    import delayrepay_amd as dr
    a = dr.array(np.arange(5.0))
    b = a * 2
    b.run()
    b[0] = 100.0
    c = a * 2
    assert c is not b and np.array_equal(c.get(), np.arange(5.0) * 2)
    assert np.array_equal((b + 1).get(), np.array([101.0, 3, 5, 7, 9]))
    # an explicit out= that is also the first operand writes into it
    x = dr.array(np.arange(5.0)); y = dr.array(np.ones(5))
    back = np.add(x, y, out=x)
    assert back is x and np.array_equal(x.get(), np.arange(5.0) + 1)
    # several results evaluated together are leaves of what is built on them
    p, q = dr.evaluate(x * 3, x + 7)
    assert p._depth == 0 and q._depth == 0
    print("ok")
    """
    assert run_cpu(script).strip().endswith("ok")


def test_an_evaluated_result_follows_its_leaves_on_this_backend_too():
    """The device backend computes an evaluated result again when a leaf under it has been
    written to (its buffers carry versions).  NumPy's arrays carry none, so the front end
    counts writes: asked for directly or used as an operand, a result evaluated before the
    latest write is computed again, and the two backends agree on the same program
    (the same cases run on the device in tests/test_gpu_reference_suite.py)."""
    script = r"""
    import numpy as np
    import delayrepay_amd as dr
    a = dr.array(np.ones(16))
    b = a * 2 + 1
    assert np.all(b.get() == 3) and b.get() is b.get()      # nothing written: the same array
    c = b + 1
    assert np.all(c.get() == 4)
    p, q = dr.evaluate(b * 2, b - 1)
    assert np.all(p.get() == 6) and np.all(q.get() == 2)
    a[:] = 5.0
    assert np.all(c.get() == 12) and np.all(b.get() == 11)
    assert np.all(p.get() == 22) and np.all(q.get() == 10)
    # reductions along the rows are expressions like any other
    m = dr.array(np.arange(24.0).reshape(4, 6))
    s, k = m.sum(axis=1), m.max(axis=1, keepdims=True)
    assert s.get()[1] == 51 and k.get()[1, 0] == 11
    m[1, 1] = -50.0
    assert s.get()[1] == -6 and k.get()[1, 0] == 11
    m[1, 5] = 99.0
    assert k.get()[1, 0] == 99
    # a result written to by hand keeps the write whatever happens to its operands
    h = a * 3
    h.run()
    h[0] = -1.0
    a[:] = 2.0
    assert h.get()[0] == -1 and h.get()[1] == 15
    print("ok")
    """
    assert run_cpu(script).strip().endswith("ok")
