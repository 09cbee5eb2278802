"""Random expressions over random view geometries are lowered and compiled for gfx950
(no GPU needed): every kernel shape and its variants (vector / element alignment,
broadcast kinds, merged outer dimensions, reduction tails, destinations with a pitch)
must produce source that hiprtc accepts."""
import numpy as np
import pytest

import delayrepay_amd as dr
from delayrepay_amd import hip
from delayrepay_amd.delayarray import NPArray, ReduceEx

DT = [np.float32, np.float64, np.int32, np.int64, np.uint8, np.bool_]
def rand_view(rs, shape, dt):
    """placeholder view with `shape`: random pitch, offset, broadcast dims, maybe transposed"""
    nd = len(shape)
    kind = rs.randint(7)
    if kind == 0:   # dense
        return hip.placeholder(shape, dt)
    if kind == 1:   # offset
        return hip.placeholder(shape, dt, offset=int(rs.randint(1, 9)))
    if kind == 2 and nd >= 2:  # padded rows
        pitch = shape[-1] + int(rs.randint(1, 9))
        strides = [1]
        for d in reversed(shape[1:]):
            strides.insert(0, strides[0] * (pitch if len(strides) == 1 else d))
        strides = tuple(strides)
        return hip.placeholder(shape, dt, strides=strides, offset=int(rs.randint(0, 5)))
    if kind == 3:   # broadcast along one dim
        k = int(rs.randint(nd))
        sub = tuple(1 if i == k else d for i, d in enumerate(shape))
        return hip.placeholder(sub, dt)
    if kind == 4 and nd >= 2:  # lower-rank
        return hip.placeholder(shape[1:], dt)
    if kind == 5 and nd == 2:  # transposed
        base = hip.placeholder((shape[1], shape[0]), dt)
        return base.transpose()
    if kind == 6:   # stepped
        big = tuple(d * 2 for d in shape)
        base = hip.placeholder(big, dt)
        return base[tuple(slice(None, None, 2) for _ in shape)]
    return hip.placeholder(shape, dt)
def rand_expr(rs, shape, depth):
    if depth == 0:
        dt = DT[rs.randint(len(DT))]
        return NPArray(rand_view(rs, shape, dt))
    op = rs.randint(8)
    a = rand_expr(rs, shape, depth - 1)
    if op == 0: return a * 2.5
    if op == 1: return np.sqrt(np.abs(a) + 1.0)
    if op == 2: return dr.where(a > 0, a, 1)
    if op == 3: return (a + 0).astype(np.float32)
    b = rand_expr(rs, shape, depth - 1)
    if op == 4: return a + b
    if op == 5: return a * b
    if op == 6: return np.maximum(a, b)
    return a - b


SEEN = {}


@pytest.mark.parametrize("seed", range(70))
def test_random_geometry_lowers_and_compiles(seed):
    rs = np.random.RandomState(seed)
    nd = int(rs.randint(1, 4))
    shape = tuple(int(rs.choice([1, 3, 16, 33, 64, 130, 4100])) for _ in range(nd))
    if np.prod(shape) > 1 << 22:
        shape = shape[:2]
    try:
        e = rand_expr(rs, shape, int(rs.randint(0, 4))) + NPArray(hip.placeholder(shape, np.float32))
    except TypeError as exc:          # NumPy's own refusal (boolean subtract), raised while building
        assert "boolean subtract" in str(exc)
        return
    mode = rs.randint(4)
    if mode == 0 or len(shape) < 2:
        low, src = hip.lower_only(e)
    elif mode == 1:
        low, src = hip.lower_only(ReduceEx(np.add, e))
    elif mode == 2:
        low, src = hip.lower_only(ReduceEx(np.maximum, e, (int(rs.randint(len(shape))),)))
    else:
        pad = tuple(d + 2 for d in shape)
        dst = hip.placeholder(pad, np.float64)[tuple(slice(1, 1 + d) for d in shape)]
        low, src = hip.lower_only(e, dst=dst)
    assert len(hip.compile_source(src)) > 0
    SEEN[low.key[0]] = SEEN.get(low.key[0], 0) + 1


def test_random_geometries_reached_the_kernel_shapes():
    for kind in ("flat", "nd", "tile2dv", "axis", "tile2dt"):
        assert SEEN.get(kind, 0) > 0, (kind, SEEN)
