"""DelayRepay for AMD Instinct MI355X: `import delayrepay_amd as np`.

A lazy NumPy look-alike (see `delayarray`) whose expressions are fused into
HIP kernels for gfx950 (see `hip`).  Surface as in the reference's package
root (delayrepay/__init__.py:4-17): everything from `delayarray`, the
`random` sub-module and `pi`.
"""
from . import backend as _be
from .delayarray import *  # noqa: F401,F403
from .delayarray import (DelayArray, NPArray, Scalar, NumpyEx, BinaryNumpyEx, BinaryFuncEx,  # noqa: F401
                         UnaryFuncEx, ReduceEx, CastEx, Memoiser, reset, evaluate, synchronize,
                         sum, max, min, abs, mean, var, average, where, clip, WhereEx,
                         std, count_nonzero, isclose, allclose, norm)
from .delayarray import any_ as any, all_ as all  # noqa: F401,A004
from . import random  # noqa: F401

backend = _be.backend
pi = _be.backend.np.pi
