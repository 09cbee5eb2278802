"""Device runtime (libdrhip through ctypes) and the device array class."""
import ctypes

import numpy as np
import pytest

from delayrepay_amd import hip, hiprt
from delayrepay_amd.devarray import ndarray

pytestmark = pytest.mark.gpu


def test_device_is_gfx950():
    info = hiprt.device_info()
    assert info["arch"].startswith("gfx950")
    assert info["wavefront_size"] == 64 and info["compute_units"] >= 200


def test_pool_recycles_blocks():
    hiprt.init()
    before = hiprt.pool_stats()
    p = hiprt.malloc(3 << 20)
    hiprt.free(p)
    q = hiprt.malloc((3 << 20) + 5)       # same 2 MiB-granular class
    assert q == p
    hiprt.free(q)
    after = hiprt.pool_stats()
    assert after["n_pool_hits"] >= before["n_pool_hits"] + 1
    assert after["bytes_in_use"] == before["bytes_in_use"]
    assert hiprt.lib().drhip_free(ctypes.c_void_p(12345)) == 20002   # foreign pointer rejected


def test_copies_fill_and_copy_kernel_roundtrip():
    host = np.random.RandomState(0).standard_normal(1 << 16).astype(np.float32)
    a = ndarray.from_host(host)
    b = ndarray(a.shape, a.dtype)
    hiprt.copy_kernel(b.ptr, a.ptr, a.nbytes)
    assert np.array_equal(b.get(), host)
    hiprt.memcpy_d2d(b.ptr, a.ptr, a.nbytes // 2)
    hiprt.fill32(b.ptr, 0x3F800000, 100)
    got = b.get()
    assert np.all(got[:100] == 1.0) and np.array_equal(got[100:], host[100:])
    c = ndarray((1000,), np.float64)
    hiprt.fill64(c.ptr, np.float64(-2.5).view(np.uint64).item(), 1000)
    assert np.all(c.get() == -2.5)
    with pytest.raises(hiprt.DrhipError):
        hiprt.copy_kernel(b.ptr + 4, a.ptr, 64)       # misaligned


def test_events_time_the_library_stream():
    a = ndarray((1 << 24,), np.float32)
    b = ndarray((1 << 24,), np.float32)
    e0, e1 = hiprt.Event(), hiprt.Event()
    e0.record()
    for _ in range(5):
        hiprt.copy_kernel(b.ptr, a.ptr, a.nbytes)
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_ms(e1)
    assert 0.01 < ms < 100


def test_compile_cache_levels(tmp_path, monkeypatch):
    monkeypatch.setenv("DELAYREPAY_CACHE_DIR", str(tmp_path))
    src = ('extern "C" __global__ void dr_kernel(float* o, long long n) '
           '{ if (threadIdx.x == 0) o[0] = 42.0f + (float)n; }\n')
    before = dict(hip.STATS)
    hip._load_or_compile(src)
    assert hip.STATS["compiles"] == before["compiles"] + 1
    assert len(list(tmp_path.glob("*.co"))) == 1
    mod = hip._load_or_compile(src)                    # second time: code object from disk
    assert hip.STATS["disk_hits"] == before["disk_hits"] + 1
    fn = hiprt.get_function(mod, "dr_kernel")
    out = ndarray((1,), np.float32)
    import struct
    args = struct.pack("@Pq", out.ptr, 8)
    hiprt.launch(fn, 1, 64, 0, args, len(args))
    assert out.get()[0] == 50.0
    with pytest.raises(hiprt.DrhipError):
        hiprt.launch(fn, 0, 64, 0, args, len(args))    # bad geometry is refused on the host


def test_unwritable_cache_directory_is_reported_once(tmp_path, monkeypatch):
    blocker = tmp_path / "file_not_dir"
    blocker.write_text("x")                          # a file where the directory should be
    monkeypatch.setenv("DELAYREPAY_CACHE_DIR", str(blocker / "cache"))
    monkeypatch.setitem(hip.STATS, "disk_write_failures", 0)
    src = 'extern "C" __global__ void dr_kernel(float* o) { o[0] = %d.0f; }\n'
    with pytest.warns(RuntimeWarning, match="cannot write the kernel cache"):
        hip._load_or_compile(src % 1)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        hip._load_or_compile(src % 2)                # second failure: counted, not repeated
    assert hip.STATS["disk_write_failures"] == 2


def test_views_follow_numpy_basic_indexing():
    host = np.arange(7 * 9 * 5, dtype=np.float64).reshape(7, 9, 5)
    dev = ndarray.from_host(host)
    keys = [np.s_[1:-1], np.s_[:, 2], np.s_[..., ::2], np.s_[::-1, 1:8:3, 4], np.s_[3],
            np.s_[None, 2, :, None, 1], np.s_[-1, -1, -1], np.s_[5:2], np.s_[1:6:2, ::-2, 1:]]
    for key in keys:
        assert np.array_equal(dev[key].get(), host[key]), key
        assert dev[key].shape == host[key].shape
        assert dev[key].strides == host[key].strides or host[key].size <= 1
    with pytest.raises(IndexError):
        dev[7]
    with pytest.raises(IndexError):
        dev[0, 0, 0, 0]
    with pytest.raises(NotImplementedError):
        dev[[1, 2]]


def test_setitem_fill_copy_astype_reshape():
    host = np.zeros((6, 8), np.float32)
    dev = ndarray.from_host(host)
    dev[1:-1, ::2] = 3
    host[1:-1, ::2] = 3
    dev[0] = np.arange(8, dtype=np.float32)
    host[0] = np.arange(8, dtype=np.float32)
    dev[:, 7] = dev[:, 0]
    host[:, 7] = host[:, 0]
    dev[5, 1:4] = np.array([1.5, 2.5, 3.5])           # float64 source, converted on assignment
    host[5, 1:4] = np.array([1.5, 2.5, 3.5])
    assert np.array_equal(dev.get(), host)
    assert np.array_equal(dev.T.copy().get(), host.T)
    assert dev.T.copy().is_contiguous
    assert np.array_equal(dev.astype(np.float64).get(), host.astype(np.float64))
    assert np.array_equal(dev.astype(np.int32).get(), host.astype(np.int32))
    assert np.array_equal(dev.reshape(8, 6).get(), host.reshape(8, 6))
    assert np.array_equal(dev[:, ::2].reshape(-1).get(), host[:, ::2].reshape(-1))
    assert float(dev[0, 3]) == 3.0 and dev[0, 3].item() == 3.0
    empty = ndarray((0, 4), np.float32)
    assert empty.get().shape == (0, 4)


def test_recorded_launches_replay_as_a_hip_graph():
    """A graph of recorded kernels must give the eager result on every replay, with
    the program's own eager work and synchronisations in between."""
    import delayrepay_amd as dr
    from oracle import numpy_oracle as orc
    rs = np.random.RandomState(21)
    u0 = np.zeros((130, 258), np.float32)
    u0[1:-1, 1:-1] = rs.uniform(0, 1, (128, 256))
    x0 = rs.standard_normal(5000)
    u = dr.array(u0)
    x = dr.array(x0)

    def sweep():
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])

    sweep()
    sweep()                                  # warm: shadow buffer exists, plan cached
    with hip.record() as plan:
        sweep()
        sweep()                              # ping-pong pair: back in the same allocation
        total = dr.sum(x * x)                # a reduction (two kernels) in the same graph
    done = 4
    assert len(plan.launches) == 4
    expect_total = float(np.sum(x0 * x0))
    assert abs(float(total) - expect_total) <= 1e-13 * expect_total
    plan.as_graph()
    for rep in range(4):
        hiprt.fill64(total.ptr, 0, 1)        # eager work between replays
        plan()
        done += 2
        hiprt.sync()
        assert np.array_equal(u.get(), orc.jacobi(u0, done)), rep
        assert abs(float(total) - expect_total) <= 1e-13 * expect_total
        y = (x * 2.0).get()                  # unrelated eager kernel + copy
        assert np.array_equal(y, x0 * 2.0)
    # the library refuses what a capture cannot hold
    hiprt.Graph.begin()
    try:
        with pytest.raises(hiprt.DrhipError):
            hiprt.sync()
        with pytest.raises(hiprt.DrhipError):
            hiprt.memcpy_d2d(total.ptr, total.ptr, 8)
    finally:
        hiprt.Graph.end()


def test_replays_invalidate_cached_results_and_keep_ping_pong_parity():
    import delayrepay_amd as dr
    from oracle import numpy_oracle as orc
    rs = np.random.RandomState(22)
    u0 = np.zeros((66, 130), np.float32)
    u0[1:-1, 1:-1] = rs.uniform(0, 1, (64, 128))
    u = dr.array(u0)

    def sweep():
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])

    sweep()
    with pytest.raises(RuntimeError, match="pairs"):
        with hip.record():
            sweep()                          # one aliasing update: would end in the other allocation
    done = 2
    with hip.record() as plan:
        sweep()
        sweep()
    done += 2
    doubled = u * 2.0
    assert np.array_equal(doubled.get(), orc.jacobi(u0, done) * np.float32(2))
    plan()
    done += 2
    # the replay wrote u: the result cached on `doubled` is stale and is recomputed
    assert np.array_equal(doubled.get(), orc.jacobi(u0, done) * np.float32(2))
    sweep()                                  # an eager update leaves u in its other allocation
    done += 1
    with pytest.raises(RuntimeError, match="swapped"):
        plan()
    sweep()
    done += 1
    plan()
    done += 2
    assert np.array_equal(u.get(), orc.jacobi(u0, done))
    # a plain (non-aliasing) recorded write bumps the version as well
    v = dr.array(np.zeros(1000))
    w = dr.array(np.arange(1000.0))
    with hip.record() as fill:
        v[:] = w + 1.0
    total = v.sum()
    assert float(total) == float(np.sum(np.arange(1000.0) + 1))
    w[:] = 5.0
    fill()
    assert np.all(v.get() == 6.0) and float(v.sum()) == 6000.0


def test_recent_roots_are_bounded_by_the_memory_their_results_hold(monkeypatch):
    import delayrepay_amd as dr
    x = dr.array(np.ones(1 << 18))                       # 2 MiB results
    monkeypatch.setattr(hip, "_RECENT_BYTES", 5 << 20)
    hip.forget()
    kept = []
    for k in range(8):
        node = x * float(k + 2)
        kept.append(node.get()[0])
        del node
    assert kept == [float(k + 2) for k in range(8)]
    held = sum(n.__dict__["array"].nbytes for n in hip._RECENT if "array" in n.__dict__)
    assert len(hip._RECENT) <= 4 and held <= (5 << 20) + (2 << 20)
    hip.forget()


def test_pool_survives_finalisers_running_on_other_threads():
    """Foreign calls drop the interpreter lock, so frees issued by another thread's
    garbage collection can overlap the driving thread's allocations."""
    import threading
    hiprt.init()
    before = hiprt.pool_stats()
    errors = []

    def churn(seed):
        try:
            sizes = [256 << (k % 9) for k in range(seed, seed + 400)]
            held = []
            for n in sizes:
                held.append(hiprt.malloc(n))
                if len(held) > 16:
                    hiprt.free(held.pop(0))
            for p in held:
                hiprt.free(p)
        except Exception as exc:      # noqa: BLE001
            errors.append(exc)
    threads = [threading.Thread(target=churn, args=(k,)) for k in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    after = hiprt.pool_stats()
    assert not errors
    assert after["bytes_in_use"] == before["bytes_in_use"]
    assert after["n_mallocs"] - before["n_mallocs"] == 6 * 400


@pytest.mark.parametrize("dtype,tol", [(np.float32, 3e-6), (np.float64, 1e-14)])
def test_matrix_product_on_the_matrix_cores(dtype, tol):
    """Full and ragged 128x128 tiles, short and long inner dimensions, both kernels."""
    import delayrepay_amd as dr
    rs = np.random.RandomState(8)
    for m, k, n in [(128, 16, 128), (64, 8, 64), (130, 33, 257), (600, 777, 513), (65, 1000, 300),
                    (256, 7, 256), (63, 100, 500), (1, 64, 64), (300, 5, 1)]:
        a, b = rs.standard_normal((m, k)).astype(dtype), rs.standard_normal((k, n)).astype(dtype)
        got = dr.array(a).dot(dr.array(b)).get()
        ref = a.astype(np.float64) @ b.astype(np.float64)
        assert got.shape == ref.shape and got.dtype == dtype
        assert np.abs(got - ref).max() <= tol * max(1.0, k / 64) * np.abs(ref).max(), (m, k, n)
    v = rs.standard_normal(777).astype(dtype)
    a = rs.standard_normal((600, 777)).astype(dtype)
    assert np.allclose((dr.array(a) @ dr.array(v)).get(), a @ v, rtol=1e-4 if dtype == np.float32 else 1e-12,
                       atol=1e-4 if dtype == np.float32 else 1e-12)


def test_a_deep_chain_of_stale_results_is_brought_up_to_date_without_recursion():
    """Three iterates, each 120 operations deep and each evaluated, then a write to the
    array they started from: the last iterate is asked for again and would be re-walked
    through all 360 operations, more frames than the interpreter allows; the stale
    operands are then recomputed one by one, deepest first."""
    import sys
    import delayrepay_amd as dr
    h0 = np.linspace(0.0, 1.0, 5000)
    base = dr.array(h0.copy())

    def grow(x):
        for _ in range(60):
            x = x * 0.999 + 0.25
        return x
    x1 = grow(base); x1.run()
    x2 = grow(x1); x2.run()
    x3 = grow(x2); x3.run()
    want_old = grow(grow(grow(h0)))
    assert np.array_equal(x3.get(), want_old)
    base[:] = base * 2.0 + 1.0
    from delayrepay_amd import delayarray
    calls = []
    refresh = delayarray._refresh_operands
    delayarray._refresh_operands = lambda root: (calls.append(root), refresh(root))
    limit = sys.getrecursionlimit()
    sys.setrecursionlimit(1000)
    try:
        got = x3.get()
    finally:
        sys.setrecursionlimit(limit)
        delayarray._refresh_operands = refresh
    assert calls, "the chain was walked in one go: make it deeper"
    assert np.array_equal(got, grow(grow(grow(h0 * 2.0 + 1.0))))
    assert np.array_equal(x1.get(), grow(h0 * 2.0 + 1.0))


def test_a_loop_of_functional_updates_holds_a_bounded_history():
    """`x = f(x)` evaluated every pass: results computed from results are a chain; past
    `hip.MAX_GENERATIONS` links the older result becomes an array in its own right, so the
    chain, its dependency lists and the device memory of earlier iterates stay bounded."""
    import gc
    import delayrepay_amd as dr
    from delayrepay_amd import hip
    n = 1 << 18
    hx, hy = np.full(n, 1.0, np.float32), np.full(n, 0.25, np.float32)
    y = dr.array(hy)
    x = dr.array(hx)
    gc.collect()
    base = hiprt.pool_stats()["bytes_in_use"]
    longest = 0
    hist = [hx]
    for k in range(300):
        x = x * 0.5 + y
        x.run()
        hx = hx * np.float32(0.5) + hy
        hist.append(hx)
        longest = max(longest, len(x.__dict__["_deps"]))
        assert x.__dict__["_gen"] <= hip.MAX_GENERATIONS
    assert longest <= 2 * (hip.MAX_GENERATIONS + 1)
    assert np.array_equal(x.get(), hx)
    gc.collect()
    held = hiprt.pool_stats()["bytes_in_use"] - base
    # the chain itself, and the last evaluated roots that are kept for plan reuse
    assert held <= (hip.MAX_GENERATIONS + 2 + hip._RECENT.maxlen) * 4 * n, held
    # the links above the last iterate that became an array in its own right still follow
    # their inputs: y changes, and x is computed afresh from that iterate
    links = x.__dict__["_gen"]
    y[:] = 1.0
    want = hist[-1 - links]
    for _ in range(links):
        want = want * np.float32(0.5) + np.float32(1.0)
    assert np.array_equal(x.get(), want)


def test_an_expression_never_asked_for_stops_growing():
    import delayrepay_amd as dr
    from delayrepay_amd import delayarray
    n = 4096
    hx, hy = np.full(n, 1.0), np.linspace(0, 1, n)
    x, y = dr.array(hx), dr.array(hy)
    for _ in range(700):
        x = x * 0.999 + y
        hx = hx * 0.999 + hy
        assert x._depth <= delayarray.MAX_DEPTH
    assert abs(float(dr.sum(x)) - hx.sum()) <= 1e-9 * hx.sum()
    assert np.allclose(x.get(), hx, rtol=1e-12)


def test_a_carried_expression_that_is_only_ever_reduced_is_evaluated_on_third_sight():
    """`x = f(x)` carried through a loop that only asks for `sum(g(x))`: the reduction walks
    through x's whole expression.  Once that expression is `hip.REUSE_DEPTH` operations deep
    and is met in a third evaluation, it is computed once on its own and is a leaf from then
    on, so the work per pass and the number of kernel structures stay bounded."""
    import delayrepay_amd as dr
    n = 1 << 14
    hx, hy = np.linspace(0.0, 1.0, n), np.linspace(1.0, 2.0, n)
    x, y = dr.array(hx), dr.array(hy)
    structures = set()
    before = len(hip._KERNELS)
    carried = []
    for k in range(60):
        x = x * 0.5 + y
        hx = hx * 0.5 + hy
        got = float(dr.sum(x * x))
        want = float(np.sum(hx * hx))
        assert abs(got - want) <= 1e-12 * want, k
        carried.append(x)
    assert len(hip._KERNELS) - before <= 12                  # not one structure per pass
    evaluated = sum("array" in node.__dict__ for node in carried)
    assert evaluated >= 40                                    # most iterates became leaves
    assert np.allclose(x.get(), hx, rtol=1e-14)
    # shallow shared operands are computed again rather than written and read back
    a, b = dr.array(hx), dr.array(hy)
    d = a - b
    r1, r2 = float(dr.sum(d * d)), float(dr.sum(abs(d)))
    assert "array" not in d.__dict__
    assert abs(r1 - np.sum((hx - hy) ** 2)) <= 1e-12 * r1 and abs(r2 - np.sum(np.abs(hx - hy))) <= 1e-12 * r2


def test_evaluations_leave_no_reference_cycles_behind():
    """Device memory must be freed with its last user, not whenever the cycle collector gets
    round to it: with the collector switched off, a long loop of fresh results still holds a
    bounded number of arrays, and a collection afterwards finds no tracer to free."""
    import gc
    import delayrepay_amd as dr
    n = 1 << 18
    y = dr.array(np.ones(n, np.float32))
    x = dr.array(np.zeros(n, np.float32))
    gc.collect()
    base = hiprt.pool_stats()["bytes_in_use"]
    gc.disable()
    try:
        for k in range(200):
            x = x * 0.999 + y
            x.run()
            if k % 3 == 0:
                float(dr.sum(x))
        held = hiprt.pool_stats()["bytes_in_use"] - base
    finally:
        gc.enable()
    assert held <= (hip.MAX_GENERATIONS + 2 + hip._RECENT.maxlen) * 4 * n, held
    gc.collect()
    assert not [o for o in gc.get_objects() if isinstance(o, hip.Tracer)]
    # the other entry points: several roots at once, updates in place, slices of lazy
    # expressions, eager helpers
    u = dr.array(np.zeros((300, 300), np.float32))

    def work(k):
        nonlocal x
        a, b = dr.evaluate(x * 0.5 + y, x - y * float(k))
        x = a
        u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:]) + float(k)
        dr.var(u, axis=1)
        dr.roll(a * 2.0, 3)
        (u.T * 2.0).run()
        (a * 2.0 + b)[5:-5].run()
        np.concatenate([a, b])
        float(np.linalg.norm(a))
    for k in range(5):
        work(k)
    gc.collect()
    for k in range(20):
        work(k + 5)
    assert gc.collect() <= 10


def test_rebuilding_a_multi_root_expression_reuses_its_plan():
    """A step that builds call and put prices anew every time and evaluates them together:
    the nodes are the hash-consed ones of the step before, the cached plan is found, one
    kernel runs, and no shared operand is computed on its own."""
    import delayrepay_amd as dr
    from oracle import numpy_oracle as orc
    rs = np.random.RandomState(12)
    S, K, T = (dr.array(rs.uniform(0.5, 2.0, 1 << 14)) for _ in range(3))
    for step in range(4):
        call, put = orc.black_scholes_expr(dr, S, K, T, 0.02, 0.3)
        launches, hits = hip.STATS["launches"], hip.STATS["plan_hits"]
        outs = hip.run_multi([call, put])
        del call, put
        assert hip.STATS["launches"] == launches + 1, step
        if step:
            assert hip.STATS["plan_hits"] == hits + 1, step
    # asked for one after the other (over fresh arrays: operands nobody has walked through
    # yet), the two prices still share nothing that is written out
    S2, K2, T2 = (dr.array(a.get()) for a in (S, K, T))
    call, put = orc.black_scholes_expr(dr, S2, K2, T2, 0.02, 0.3)
    launches = hip.STATS["launches"]
    c2 = hip.run(call)
    p2 = hip.run(put)
    assert hip.STATS["launches"] == launches + 2
    assert np.array_equal(c2.get(), outs[0].get()) and np.array_equal(p2.get(), outs[1].get())


def test_a_structure_met_before_keeps_its_plan_over_fresh_arrays():
    """Batches of new data through one expression: from the second batch on nothing is
    traced or lowered (`seen_hits`), and every batch gets its own arrays' and numbers'
    result.  Operand identities, number types and geometry tell structures apart."""
    import delayrepay_amd as dr
    from delayrepay_amd.delayarray import ReduceEx
    rs = np.random.RandomState(5)
    n = 1 << 12

    def batch():
        return [rs.uniform(-1, 1, n).astype(np.float32) for _ in range(3)]
    cases = [
        ("saxpy", lambda k, x, y, w: k * x + y, lambda k, x, y, w: np.float32(k) * x + y),
        ("square", lambda k, x, y, w: x * x + y, lambda k, x, y, w: x * x + y),
        ("mixed", lambda k, x, y, w: x * y + y, lambda k, x, y, w: x * y + y),
        ("shared", lambda k, x, y, w: (x - y) * (x - y) * w + k, lambda k, x, y, w: (x - y) * (x - y) * w + np.float32(k)),
        ("unary", lambda k, x, y, w: np.sqrt(np.abs(x)) / (k + y * y), lambda k, x, y, w: np.sqrt(np.abs(x)) / (np.float32(k) + y * y)),
    ]
    for name, lazy, eager in cases:
        for step in range(4):
            hx, hy, hw = batch()
            k = 1.5 + step
            x, y, w = dr.array(hx), dr.array(hy), dr.array(hw)
            seen, launches = hip.STATS["seen_hits"], hip.STATS["launches"]
            got = hip.run(lazy(k, x, y, w)).get()
            assert hip.STATS["launches"] == launches + 1
            if step:        # (the first batch may meet a structure that an earlier test left)
                assert hip.STATS["seen_hits"] == seen + 1, (name, step)
            assert got.tobytes() == eager(k, hx, hy, hw).astype(np.float32).tobytes(), (name, step)
    # a reduction root and two roots at once
    for step in range(3):
        hx, hy, hw = (a.astype(np.float64) for a in batch())
        x, y, w = dr.array(hx), dr.array(hy), dr.array(hw)
        seen = hip.STATS["seen_hits"]
        s = hip.run(ReduceEx(np.add, (x - y) ** 2 * w)).get()
        p, q = (r.get() for r in hip.run_multi([x * y + w, x - y * w]))
        if step:
            assert hip.STATS["seen_hits"] == seen + 2
        assert np.isclose(s, ((hx - hy) ** 2 * hw).sum(), rtol=1e-13)
        assert p.tobytes() == (hx * hy + hw).tobytes() and q.tobytes() == (hx - hy * hw).tobytes()
    # rows that are reduced and used again: the row kernel's plan is kept as well, per row
    # length and per way the rows are laid out
    for shape in ((64, 64), (32, 128), (64, 64)):
        for step in range(3):
            ha = rs.uniform(-2, 2, shape).astype(np.float32)
            hb = rs.uniform(1, 2, (shape[0] + 2, shape[1] + 4)).astype(np.float32)
            a, b = dr.array(ha), dr.array(hb)[1:-1, 2:-2]
            seen, launches = hip.STATS["seen_hits"], hip.STATS["launches"]
            e = np.exp(a - a.max(axis=1, keepdims=True))
            got = hip.run(e / e.sum(axis=1, keepdims=True) * b).get()
            assert hip.STATS["launches"] == launches + 1
            if step:
                assert hip.STATS["seen_hits"] == seen + 1, (shape, step)
            ref = np.exp(ha - ha.max(axis=1, keepdims=True))
            np.testing.assert_allclose(got, ref / ref.sum(axis=1, keepdims=True) * hb[1:-1, 2:-2], rtol=3e-6)
            seen = hip.STATS["seen_hits"]
            got = hip.run(a / a.max(axis=1)[:, None]).get()
            assert got.tobytes() == (ha / ha.max(axis=1)[:, None]).tobytes()
            if step:
                assert hip.STATS["seen_hits"] == seen + 1, (shape, step)
    # an operand evaluated beforehand is a leaf, whatever its structure's plan said
    hx, hy, hw = batch()
    x, y, w = dr.array(hx), dr.array(hy), dr.array(hw)
    t = x * y
    t.run()
    assert hip.run(t + w).get().tobytes() == (hx * hy + hw).tobytes()
    hx2, hy2, hw2 = batch()
    x2, y2, w2 = dr.array(hx2), dr.array(hy2), dr.array(hw2)
    assert hip.run(x2 * y2 + w2).get().tobytes() == (hx2 * hy2 + hw2).tobytes()
    # a view with another offset or stride is another geometry
    big = dr.array(np.concatenate(batch()))
    hb = big.get()
    for lo in (0, 4, 5):
        assert hip.run(big[lo:lo + n] * 2.0 + big[lo + n:lo + 2 * n]).get().tobytes() == \
            (hb[lo:lo + n] * np.float32(2.0) + hb[lo + n:lo + 2 * n]).tobytes()
    # switching the tunables makes every remembered plan stale
    hip.set_tune(nts=0)
    try:
        seen = hip.STATS["seen_hits"]
        assert hip.run(2.5 * x + y).get().tobytes() == (np.float32(2.5) * hx + hy).tobytes()
        assert hip.STATS["seen_hits"] == seen
    finally:
        hip.set_tune(nts=1)


def test_writes_by_hand_aliasing_out_and_stretched_views():
    """The same program as on the CPU backend gives the same values here; a view that
    repeats elements is read-only."""
    import delayrepay_amd as dr
    a = dr.array(np.arange(5.0))
    b = a * 2
    b.run()
    b[0] = 100.0
    c = a * 2
    assert c is not b and np.array_equal(c.get(), np.arange(5.0) * 2)
    assert np.array_equal((b + 1).get(), np.array([101.0, 3, 5, 7, 9]))
    x, y = dr.array(np.arange(5.0)), dr.array(np.ones(5))
    back = np.add(x, y, out=x)
    assert back is x and np.array_equal(x.get(), np.arange(5.0) + 1)
    wide = np.broadcast_to(dr.array(np.arange(4.0)), (3, 4))
    assert np.array_equal(wide.get(), np.broadcast_to(np.arange(4.0), (3, 4)))
    with pytest.raises(ValueError, match="read-only"):
        wide[0, 0] = 5.0
    with pytest.raises(ValueError, match="read-only"):
        wide[...] = dr.array(np.ones((3, 4))) * 2.0


def test_matrix_product_with_more_rows_than_one_launch_takes():
    """Points times a 3 x 3 matrix: 5 million rows are more 64-row tiles than the second
    grid dimension holds (65535), so the library multiplies slabs of rows."""
    rs = np.random.RandomState(20)
    pts = rs.standard_normal((5_000_000, 3)).astype(np.float32)
    rot = rs.standard_normal((3, 3)).astype(np.float32)
    import delayrepay_amd as dr
    got = (dr.array(pts) @ dr.array(rot)).get()
    ref = pts.astype(np.float64) @ rot.astype(np.float64)
    assert got.shape == ref.shape and got.dtype == np.float32
    np.testing.assert_allclose(got[::997], ref[::997], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[-3:], ref[-3:], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[65535 * 64 - 2:65535 * 64 + 2], ref[65535 * 64 - 2:65535 * 64 + 2],
                               rtol=1e-5, atol=1e-5)
