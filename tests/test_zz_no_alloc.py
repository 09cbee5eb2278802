"""drhip_launch_scratch (the entry point that allocates nothing) against drhip_launch
with pooled partial results: the same fused reduction kernels, called through the C ABI
twice in a row, the second time on a smaller input.  The reduction is deterministic
(no atomics), so the two routes must agree bit for bit."""
import ctypes
import struct

import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import codegen as cg, hip, hiprt
from delayrepay_amd.devarray import ndarray
from oracle import numpy_oracle as oracle

pytestmark = pytest.mark.gpu


def _reduction(n, seed):
    """Compiled kernels and argument pieces of s = sum((x - y)**2 * w) over n float64."""
    rs = np.random.RandomState(seed)
    x, y, w = rs.standard_normal(n), rs.standard_normal(n), rs.uniform(0, 1, n)
    dx, dy, dw = dr.array(x), dr.array(y), dr.array(w)
    ex = (dx - dy) ** 2 * dw
    tracer = hip.Tracer()
    root = tracer.visit(ex)
    plan = hip._make_plan(tracer, [root], reduce_op="add", axes=None)
    low = plan.low
    kern = hip._kernel_for(low, True)
    ptrs = [buf.ptr + off for buf, off in low.srcs]
    return dict(low=low, kern=kern, ptrs=ptrs, acc=plan.acc, host=(x, y, w),
                keep=(dx, dy, dw, ex))


def _by_launch(r, out):
    """Existing entry point: partial results in a block from the pool."""
    lib = hiprt.lib()
    low, kern = r["low"], r["kern"]
    nbytes = low.fin_count * cg.ITEMSIZE[r["acc"]]
    partial = hiprt.malloc(nbytes)
    args = kern.packer.pack(*r["ptrs"], partial, *low.scal, *low.tail)
    assert lib.drhip_launch(kern.func, low.grid, cg.BLOCK, 0, args, len(args)) == 0
    fin = struct.pack("@PPi", partial, out.ptr, low.fin_count)
    assert lib.drhip_launch(kern.finalize, 1, cg.BLOCK, 0, fin, len(fin)) == 0
    hiprt.sync()
    hiprt.free(partial)
    return out.get().copy()


def _by_launch_scratch(r, out):
    """The entry point under test: partial results in the static scratch array."""
    lib = hiprt.lib()
    low, kern = r["low"], r["kern"]
    nbytes = low.fin_count * cg.ITEMSIZE[r["acc"]]
    args = kern.packer.pack(*r["ptrs"], 0xDEAD0000, *low.scal, *low.tail)   # slot is overwritten
    rc = lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, args, len(args),
                                  8 * len(r["ptrs"]), nbytes)
    assert rc == 0, lib.drhip_last_error()
    fin = struct.pack("@PPi", 0, out.ptr, low.fin_count)
    rc = lib.drhip_launch_scratch(kern.finalize, 1, cg.BLOCK, 0, fin, len(fin), 0, nbytes)
    assert rc == 0, lib.drhip_last_error()
    hiprt.sync()
    return out.get().copy()


def test_launch_scratch_matches_launch_on_two_calls_in_a_row():
    hiprt.init()
    assert hiprt.scratch_bytes() == 4 << 20
    before = hiprt.pool_stats()["n_mallocs"]
    out = ndarray((), np.float64)
    big = _reduction((1 << 22) + 12345, 5)      # every block of the widest grid has work
    small = _reduction(70001, 6)                # fewer partial results than the call before
    assert small["low"].fin_count < big["low"].fin_count
    for r in (big, small):
        hiprt.fill64(out.ptr, 0x7FF8000000000000, 1)
        want = _by_launch(r, out)
        hiprt.fill64(out.ptr, 0x7FF8000000000000, 1)
        mallocs = hiprt.pool_stats()["n_mallocs"]
        got = _by_launch_scratch(r, out)
        assert hiprt.pool_stats()["n_mallocs"] == mallocs        # the pool was not asked
        assert got.tobytes() == want.tobytes()
        ref = float(oracle.sumsq(*r["host"]))
        assert abs(float(got) - ref) <= 1e-13 * abs(ref)
    assert hiprt.pool_stats()["n_mallocs"] > before


def test_launch_scratch_refuses_what_it_cannot_hold():
    hiprt.init()
    lib = hiprt.lib()
    r = _reduction(5000, 7)
    low, kern = r["low"], r["kern"]
    args = kern.packer.pack(*r["ptrs"], 0, *low.scal, *low.tail)
    slot = 8 * len(r["ptrs"])
    too_big = hiprt.scratch_bytes() + 1
    assert lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, args, len(args), slot,
                                    too_big) == 20002
    assert b"scratch" in lib.drhip_last_error()
    assert lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, args, len(args),
                                    len(args), 64) == 20002            # slot outside the block
    assert lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, args, len(args), slot + 4,
                                    64) == 20002                       # misaligned slot
    # an offset near the top of size_t must not wrap round the bound check (it is refused on
    # the host; nothing is launched)
    assert lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, args, len(args),
                                    ctypes.c_size_t(0xFFFFFFFFFFFFFFF8), 64) == 20002
    huge = ctypes.create_string_buffer(8192)
    assert lib.drhip_launch_scratch(kern.func, low.grid, cg.BLOCK, 0, huge, 8192, 0, 64) == 20002


def test_front_end_reductions_use_the_scratch_array_and_match_the_pooled_route():
    rs = np.random.RandomState(8)
    a = rs.standard_normal((3000, 700)).astype(np.float32)
    da = dr.array(a)
    results = {}
    for flag in (1, 0):
        hip.set_tune(static_scratch=flag)
        try:
            results[flag] = ((da * da).sum().get().copy(), (da + 1).sum(axis=0).get().copy(),
                             (da * 2).max(axis=1).get().copy())
        finally:
            hip.set_tune(static_scratch=1)
    for got, want in zip(results[1], results[0]):
        assert got.tobytes() == want.tobytes()
