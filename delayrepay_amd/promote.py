"""Result types of ufuncs, decided by NumPy itself.

Both the lazy front end (for the `dtype` it shows on a node) and the HIP backend
(for the C type every statement is computed in) ask the same question here, so a
node's advertised dtype and the kernel's arithmetic cannot drift apart.  The
backend never relies on the dtype stored on a node: the reference's front end
stores `None` on scalars and copies a sibling's dtype onto interior nodes
(delayrepay/delayarray.py:462-467), metadata that neither of its backends
computes with.

An operand is described by a pair: ("a", dtype string) for anything array-valued,
("np", dtype string) for a NumPy scalar (it keeps its type), ("py", "b"|"i"|"f"|"c")
for a Python number (weak: it adopts the type of the array it meets).
"""
import numbers

import numpy as np

PY_DESCR = {bool: ("py", "b"), int: ("py", "i"), float: ("py", "f"), complex: ("py", "c")}
_PY_PROBE = {"b": True, "i": 1, "f": 1.0, "c": 1j}
_CACHE = {}


def scalar_descr(val):
    """Descriptor of a number used as an operand."""
    d = PY_DESCR.get(type(val))
    if d is not None:
        return d
    if isinstance(val, np.generic):
        return ("np", val.dtype.str)
    if isinstance(val, numbers.Integral):
        return ("py", "i")
    if isinstance(val, numbers.Real):
        return ("py", "f")
    return ("py", "c")


def result_dtype(func, descrs):
    """dtype NumPy gives `func` on operands described by `descrs`; found by calling
    `func` on empty arrays and unit scalars of those types, then remembered."""
    key = (func, descrs)
    try:
        return _CACHE[key]
    except KeyError:
        pass
    probes = []
    for kind, code in descrs:
        if kind == "a":
            probes.append(np.empty(0, dtype=code))
        elif kind == "np":
            probes.append(np.dtype(code).type(1))
        else:
            probes.append(_PY_PROBE[code])
    if all(kind != "a" for kind, _ in descrs):
        probes[0] = np.empty(0, dtype=np.asarray(probes[0]).dtype)
    with np.errstate(all="ignore"):
        dt = func(*probes).dtype
    _CACHE[key] = dt
    return dt
