"""`np` and `fallback` namespaces of the HIP backend (the backend-module protocol,
delayrepay/cuda.py:21-22): creation routines, eager reductions and the other
library calls the front end reaches through `backend.fallback.<name>`
(delayrepay/delayarray.py:85,511-568,588,596-644).  Everything runs on the device
through generated kernels or libdrhip; creation routines that need values build
them on the host and upload.
"""
import numpy

from . import hiprt
from .devarray import ndarray
from .hip import assign, materialise, run_reduce_product


def _upload(fn):
    def wrapper(*args, **kwargs):
        args = [a.get() if isinstance(a, ndarray) else a for a in args]
        return ndarray.from_host(fn(*args, **kwargs))
    wrapper.__name__ = fn.__name__
    return wrapper


def _filled(value_of):
    def make(shape, *args, dtype=None, **kwargs):
        value, default = value_of(args)
        if dtype is None:
            dtype = default
        if isinstance(shape, (int, numpy.integer)):
            shape = (int(shape),)
        out = ndarray(tuple(shape), dtype)
        if value is not None and out.size:
            assign(out, value)
        return out
    return make


def _like(maker):
    def make(proto, *args, dtype=None, **kwargs):
        proto = proto._force() if hasattr(proto, "_force") else proto
        return maker(proto.shape, *args, dtype=dtype or proto.dtype)
    return make


class _Random:
    """Host NumPy generators, uploaded (input generation; cf. delayrepay/random.py)."""

    def __getattr__(self, name):
        fn = getattr(numpy.random, name)
        if name in ("seed", "get_state", "set_state"):
            return fn
        return _upload(fn)


class _Fallback:
    """Eager routines on device arrays (the reference uses `cupy` here, cuda.py:22).
    Reductions and copies run as generated kernels; creation routines build on the
    host and upload; what has no device implementation raises."""

    newaxis = None
    pi = numpy.pi

    empty = staticmethod(_filled(lambda a: (None, numpy.float64)))
    zeros = staticmethod(_filled(lambda a: (0, numpy.float64)))
    ones = staticmethod(_filled(lambda a: (1, numpy.float64)))
    full = staticmethod(_filled(lambda a: (a[0], numpy.asarray(a[0]).dtype)))
    empty_like = staticmethod(_like(empty.__func__))
    zeros_like = staticmethod(_like(zeros.__func__))
    ones_like = staticmethod(_like(ones.__func__))
    full_like = staticmethod(_like(full.__func__))

    @staticmethod
    def asarray(obj, dtype=None, **kwargs):
        if hasattr(obj, "_force"):
            obj = obj._force()
        if isinstance(obj, ndarray):
            return obj if dtype is None or numpy.dtype(dtype) == obj.dtype else obj.astype(dtype)
        return ndarray.from_host(numpy.asarray(obj, dtype=dtype))

    array = asarray
    asanyarray = asarray

    @staticmethod
    def ascontiguousarray(obj, dtype=None):
        arr = _Fallback.asarray(obj, dtype)
        return arr if arr.is_contiguous else arr.copy()

    @staticmethod
    def copy(obj):
        return _Fallback.asarray(obj).copy()

    @staticmethod
    def transpose(arr, axes=None):
        return arr.transpose(axes) if axes is not None else arr.transpose()

    @staticmethod
    def broadcast_to(arr, shape):
        return _Fallback.asarray(arr).broadcast_to(shape)

    @staticmethod
    def _reduce(arr, name, axis, keepdims):
        from .delayarray import NPArray, _reduce
        return _reduce(getattr(numpy, name), NPArray(arr), axis=axis, keepdims=keepdims)

    @staticmethod
    def sum(arr, axis=None, keepdims=False):
        return _Fallback._reduce(arr, "add", axis, keepdims)

    @staticmethod
    def max(arr, axis=None, keepdims=False):
        return _Fallback._reduce(arr, "maximum", axis, keepdims)

    @staticmethod
    def min(arr, axis=None, keepdims=False):
        return _Fallback._reduce(arr, "minimum", axis, keepdims)

    @staticmethod
    def dot(a, b):
        """Matrix products on the device (vector.vector is fused by the front end)."""
        a, b = _Fallback.asarray(a), _Fallback.asarray(b)
        dt = numpy.result_type(a.dtype, b.dtype)
        if dt.kind != "f":
            dt = numpy.dtype(numpy.float64)
        a = _Fallback.ascontiguousarray(a, dt)
        b = _Fallback.ascontiguousarray(b, dt)
        if a.ndim == 1 and b.ndim == 1:
            return run_reduce_product(a, b)
        if (a.ndim, b.ndim) in ((2, 1), (1, 2)):
            # one pass over the matrix as a fused reduction
            from . import delayarray as fe
            return fe.NPArray(a)._dot([fe.NPArray(a), fe.NPArray(b)], {})._force()
        a2 = a.reshape(1, -1) if a.ndim == 1 else a
        b2 = b.reshape(-1, 1) if b.ndim == 1 else b
        if a2.ndim != 2 or b2.ndim != 2 or a2.shape[1] != b2.shape[0]:
            raise ValueError(f"shapes {a.shape} and {b.shape} not aligned")
        m, k = a2.shape
        n = b2.shape[1]
        out = ndarray((m, n), dt)
        hiprt.matmul(dt.itemsize == 8, a2.ptr, b2.ptr, out.ptr, m, n, k, k, n, n)
        if a.ndim == 1:
            return out.reshape(n)
        if b.ndim == 1:
            return out.reshape(m)
        return out

    matmul = dot

    # -- routines the front end reaches through `fallback.<name>` (delayarray.py:511-568,615):
    #    evaluated on the device through the lazy front end, returned as device arrays

    @staticmethod
    def _eager(fn, *args, **kwargs):
        from . import delayarray as fe
        wrapped = [fe.NPArray(a) if isinstance(a, ndarray) else a for a in args]
        res = fn(*wrapped, **kwargs)
        return res._force() if isinstance(res, fe.DelayArray) else res

    @staticmethod
    def mean(arr, axis=None, keepdims=False):
        from . import delayarray as fe
        return _Fallback._eager(fe.mean, arr, axis=axis, keepdims=keepdims)

    @staticmethod
    def var(arr, axis=None, ddof=0, keepdims=False):
        from . import delayarray as fe
        return _Fallback._eager(fe.var, arr, axis=axis, ddof=ddof, keepdims=keepdims)

    @staticmethod
    def average(arr, axis=None, weights=None):
        from . import delayarray as fe
        if weights is None:
            return _Fallback.mean(arr, axis=axis)
        a, w = fe.NPArray(_Fallback.asarray(arr)), fe.NPArray(_Fallback.asarray(weights))
        num = fe._reduce(numpy.add, a * w, axis=axis)
        den = fe._reduce(numpy.add, w if w.shape == a.shape else w + 0 * a, axis=axis)
        num = num if isinstance(num, fe.DelayArray) else fe.NPArray(num)
        den = den if isinstance(den, fe.DelayArray) else fe.NPArray(den)
        return (num / den)._force()

    @staticmethod
    def maximum(a, b):
        return _Fallback._eager(numpy.maximum, a, b)

    @staticmethod
    def minimum(a, b):
        return _Fallback._eager(numpy.minimum, a, b)

    @staticmethod
    def greater(a, b):
        return _Fallback._eager(numpy.greater, a, b)

    @staticmethod
    def less(a, b):
        return _Fallback._eager(numpy.less, a, b)

    @staticmethod
    def repeat(arr, repeats, axis=None):
        """Each element `repeats` times (an integer), as a broadcast view made dense."""
        arr = _Fallback.asarray(arr)
        if not isinstance(repeats, (int, numpy.integer)):
            raise NotImplementedError("repeat with per-element counts is not implemented on the device")
        if axis is None:
            arr, axis = arr.reshape(arr.size), 0
        axis %= max(arr.ndim, 1)
        shape = arr.shape[:axis + 1] + (int(repeats),) + arr.shape[axis + 1:]
        strides = arr._strides[:axis + 1] + (0,) + arr._strides[axis + 1:]
        dense = materialise(ndarray(shape, arr.dtype, arr.buf, arr.offset, strides))
        return dense.reshape(arr.shape[:axis] + (arr.shape[axis] * int(repeats),) + arr.shape[axis + 1:])

    @staticmethod
    def tile(arr, reps):
        """The array repeated `reps` times along each axis."""
        arr = _Fallback.asarray(arr)
        reps = (reps,) if isinstance(reps, (int, numpy.integer)) else tuple(reps)
        nd = max(arr.ndim, len(reps))
        reps = (1,) * (nd - len(reps)) + tuple(int(r) for r in reps)
        shape = (1,) * (nd - arr.ndim) + arr.shape
        strides = (0,) * (nd - arr.ndim) + arr._strides
        vshape, vstrides = [], []
        for r, d, s in zip(reps, shape, strides):
            vshape += [r, d]
            vstrides += [0, s]
        dense = materialise(ndarray(vshape, arr.dtype, arr.buf, arr.offset, vstrides))
        return dense.reshape(tuple(r * d for r, d in zip(reps, shape)))

    @staticmethod
    def cumsum(arr, axis=None):
        arr = _Fallback.asarray(arr)
        if axis is not None and arr.ndim > 1:
            raise NotImplementedError("cumsum along an axis of an N-d array is not implemented "
                                      "on the device")
        kinds = {"float32": 0, "float64": 1, "int32": 2, "int64": 3}
        if arr.dtype.name not in kinds:
            arr = arr.astype(numpy.int64 if arr.dtype.kind in "iub" else numpy.float64)
        elif arr.dtype == numpy.int32:
            arr = arr.astype(numpy.int64)           # NumPy accumulates small ints in int64
        flat = arr.reshape(arr.size) if arr.is_contiguous else arr.copy().reshape(arr.size)
        out = ndarray((arr.size,), flat.dtype)
        hiprt.cumsum(kinds[flat.dtype.name], flat.ptr, out.ptr, arr.size)
        return out

    @staticmethod
    def diag(arr, k=0):
        arr = _Fallback.asarray(arr)
        if arr.ndim == 2:
            rows, cols = arr.shape
            r0, c0 = (0, k) if k >= 0 else (-k, 0)
            n = max(0, min(rows - r0, cols - c0))
            view = ndarray((n,), arr.dtype, arr.buf,
                           arr.offset + r0 * arr._strides[0] + c0 * arr._strides[1],
                           (arr._strides[0] + arr._strides[1],))
            return materialise(view)
        if arr.ndim == 1:
            n = arr.shape[0] + abs(k)
            out = _Fallback.zeros((n, n), dtype=arr.dtype)
            r0, c0 = (0, k) if k >= 0 else (-k, 0)
            target = ndarray((arr.shape[0],), arr.dtype, out.buf, r0 * n + c0, (n + 1,))
            assign(target, arr)
            return out
        raise ValueError("Input must be 1- or 2-d.")

    @staticmethod
    def diagflat(arr, k=0):
        arr = _Fallback.asarray(arr)
        return _Fallback.diag(arr.reshape(arr.size), k)

    @staticmethod
    def roll(arr, shift, axis=None):
        if axis is None:
            flat = arr.reshape(arr.size)
            return _Fallback.roll(flat, shift, 0).reshape(arr.shape)
        n = arr.shape[axis]
        out = ndarray(arr.shape, arr.dtype)
        if n == 0:
            return out
        shift %= n
        head = [slice(None)] * arr.ndim
        tail = [slice(None)] * arr.ndim
        head[axis], tail[axis] = slice(shift, None), slice(0, n - shift)
        assign(out[tuple(head)], arr[tuple(tail)])
        if shift:
            head[axis], tail[axis] = slice(0, shift), slice(n - shift, None)
            assign(out[tuple(head)], arr[tuple(tail)])
        return out

    def __getattr__(self, name):
        fn = getattr(numpy, name, None)
        if name in ("eye", "identity", "arange", "linspace", "logspace", "geomspace", "tri",
                    "frombuffer", "fromfile", "fromfunction", "fromiter", "fromstring",
                    "loadtxt", "vander"):
            return _upload(fn)
        raise AttributeError(f"{name} has no device implementation in the HIP backend")


class _Np:
    """The slice of the array namespace the front end reads from `backend.np`
    (delayarray.py:188-194, __init__.py:17, random.py:6-13)."""

    pi = numpy.pi
    random = _Random()
    add = numpy.add
    subtract = numpy.subtract
    multiply = numpy.multiply
    true_divide = numpy.true_divide
    divide = numpy.divide
    matmul = numpy.matmul


np = _Np()
fallback = _Fallback()
