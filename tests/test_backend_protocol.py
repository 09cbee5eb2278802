"""The HIP backend behind a front end that is not this repository's: nodes that
follow the reference's conventions (class names, `(0,)` scalars without a dtype,
sibling-copied dtypes) are traced, lowered and compiled like the repository's own."""
import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import hip
from delayrepay_amd.devarray import placeholder
from oracle import numpy_oracle as oracle

from . import refstyle_frontend as ref


def _own_and_foreign(build, *shapes_dtypes):
    arrays = [placeholder(shape, dt) for shape, dt in shapes_dtypes]
    own = build(*[dr.NPArray(a) for a in arrays])
    foreign = build(*[ref.NPArray(a) for a in arrays])
    assert type(foreign).__module__ != type(own).__module__
    return hip.lower_only(own), hip.lower_only(foreign)


def test_reference_style_saxpy_lowers_to_the_same_kernel():
    (low_a, src_a), (low_b, src_b) = _own_and_foreign(
        lambda x, y: 2.0 * x + y, ((1 << 20,), np.float32), ((1 << 20,), np.float32))
    assert low_b.kind == "flat"
    assert low_a.key == low_b.key and src_a == src_b
    assert "double" not in src_b.split("dr_")[-1]       # the weak scalar 2.0 is a float parameter
    hip.compile_source(src_b)


def test_reference_style_horner_lowers_to_the_same_kernel():
    c = [0.5, -0.25, 0.125, 1.5, -2.0, 0.75, 0.3, -0.1, 0.9]

    def horner(x):
        acc = c[8] * x + c[7]
        for k in range(6, -1, -1):
            acc = acc * x + c[k]
        return acc
    (low_a, src_a), (low_b, src_b) = _own_and_foreign(horner, ((1 << 22,), np.float32))
    assert low_a.key == low_b.key and src_a == src_b
    assert len(low_b.scal) == 9
    hip.compile_source(src_b)


def test_reference_style_functions_powers_and_mixed_types():
    def build(s, k, t):
        lib = dr if isinstance(s, dr.DelayArray) else None

        def f(fn, v):
            return fn(v) if lib else ref.unary(fn, v)
        d = (f(np.log, s / k) + 0.065 * t) / (0.3 * f(np.sqrt, t))
        return f(np.exp, -0.02 * t) * d ** 3 + (s - k) ** 2.5
    (low_a, src_a), (low_b, src_b) = _own_and_foreign(
        build, ((4096,), np.float64), ((4096,), np.float64), ((4096,), np.float32))
    assert low_a.key == low_b.key and src_a == src_b
    hip.compile_source(src_b)


def test_types_come_from_numpy_not_from_the_nodes():
    """The reference's dtype rule gives float32 for float32 * float64 (first child
    wins); the backend computes what NumPy computes."""
    a = ref.NPArray(placeholder((5000,), np.float32))
    b = ref.NPArray(placeholder((5000,), np.float64))
    ex = a * b + 1
    assert ex.dtype == np.float32                    # what the front end believes
    low, src = hip.lower_only(ex)
    tracer = hip.Tracer()
    assert tracer.visit(ex)[1] == "f8"
    assert ref.Scalar(1).dtype is None


def test_unknown_node_kinds_are_refused_clearly():
    class NPRef(ref.Node):
        shape = (8,)
    with pytest.raises(NotImplementedError, match="NPRef"):
        hip.lower_only(NPRef())
    with pytest.raises(NotImplementedError, match="logaddexp"):
        hip.lower_only(ref.BinaryFuncEx(np.logaddexp, ref.NPArray(placeholder((8,), np.float32)),
                                        ref.Scalar(1.0)))
    with pytest.raises(TypeError, match="device array"):
        hip.lower_only(ref.NPArray(np.zeros(8, np.float32)) * 2.0)


def test_own_nodes_advertise_the_dtype_the_backend_computes():
    rs = np.random.RandomState(3)
    leaves = [dr.NPArray(placeholder((4096,), dt))
              for dt in (np.float32, np.float64, np.int32, np.int64, np.bool_, np.uint8)]
    for _ in range(200):
        a, b = (leaves[i] for i in rs.randint(0, len(leaves), 2))
        op = [np.add, np.multiply, np.subtract, np.true_divide, np.maximum, np.greater,
              np.arctan2, np.hypot][rs.randint(0, 8)]
        other = [b, 2, 2.5, np.float32(2), True][rs.randint(0, 5)]
        try:
            node = op(a, other)
        except TypeError:
            continue                                   # NumPy refuses it, too
        try:
            code = hip.Tracer().visit(node)[1]
        except NotImplementedError:
            continue
        assert hip.code_dtype(code) == node.dtype, (op, a.dtype, other)


@pytest.mark.gpu
def test_reference_style_nodes_run_bit_exact_on_the_gpu():
    from delayrepay_amd.devarray import ndarray
    rs = np.random.RandomState(0)
    n = 1 << 20
    x = rs.uniform(-1, 1, n).astype(np.float32)
    y = rs.uniform(-1, 1, n).astype(np.float32)
    dx, dy = ref.NPArray(ndarray.from_host(x)), ref.NPArray(ndarray.from_host(y))
    z = (2.0 * dx + dy).evaluate(hip)
    assert z.get().tobytes() == oracle.saxpy(2.0, x, y).tobytes()

    c = rs.uniform(-1, 1, 9).astype(np.float32)
    xs = rs.uniform(-2, 2, n).astype(np.float32)
    node = ref.NPArray(ndarray.from_host(xs))
    acc = float(c[8]) * node + float(c[7])
    for k in range(6, -1, -1):
        acc = acc * node + float(c[k])
    assert acc.evaluate(hip).get().tobytes() == oracle.horner(c, xs).tobytes()

    s = rs.uniform(5, 30, n)
    t = rs.uniform(0.25, 10, n)
    ds, dt = ref.NPArray(ndarray.from_host(s)), ref.NPArray(ndarray.from_host(t))
    d = (ref.unary(np.log, ds) + 0.065 * dt) / (0.3 * ref.unary(np.sqrt, dt))
    got = (d * d - ref.unary(np.exp, -0.02 * dt)).evaluate(hip).get()
    want = (np.log(s) + 0.065 * t) / (0.3 * np.sqrt(t))
    want = want * want - np.exp(-0.02 * t)
    assert np.all(np.abs(got - want) <= 1e-13 * np.maximum(np.abs(want), 1.0))
    # an evaluated node is a leaf of a later expression, as in the reference
    again = (acc * 2.0).evaluate(hip).get()
    assert again.tobytes() == (oracle.horner(c, xs) * np.float32(2.0)).tobytes()
