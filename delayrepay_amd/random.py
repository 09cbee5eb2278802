"""`delayrepay.random`: backend random routines wrapped as lazy leaves
(cf. delayrepay/random.py:6-13).  Input generation only; nothing here is on
the fused hot path."""
from . import backend as be
from .delayarray import cast

_rnd = be.backend.np.random

rand = cast(_rnd.rand)
randn = cast(_rnd.randn)
random = cast(_rnd.random)
randint = cast(_rnd.randint)
choice = cast(_rnd.choice)
seed = _rnd.seed
