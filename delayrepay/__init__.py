"""`import delayrepay as np`: the reference's import name, served by
`delayrepay_amd` (the MI355X build).  Sub-modules a user of the reference may
import by path (`delayrepay.random`, `delayrepay.backend`, ...) resolve to the
same module objects."""
import sys as _sys

import delayrepay_amd as _impl
from delayrepay_amd import *  # noqa: F401,F403
from delayrepay_amd import (sum, max, min, abs, mean, var, average, evaluate,  # noqa: F401
                            synchronize, reset, pi, backend, random, std, count_nonzero, isclose,
                            allclose, norm, any, all)  # noqa: A004

for _name in ("backend", "delayarray", "visitor", "random", "cpu", "hip", "codegen", "devarray",
              "hiprt"):
    _mod = _sys.modules.get("delayrepay_amd." + _name)
    if _mod is not None:
        _sys.modules["delayrepay." + _name] = _mod
        if _name not in ("backend", "random"):
            globals()[_name] = _mod
del _name, _mod
