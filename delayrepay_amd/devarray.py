"""Device array of the HIP backend: what CuPy's `ndarray` is to the reference's
GPU backend (delayrepay/cuda.py:21-26).

The class is named `ndarray` on purpose: the front end recognises backend
arrays by that type name (delayrepay/delayarray.py:225).  An array is a
(buffer, element offset, shape, element strides, dtype) view; basic slicing
returns views of the same buffer, as the front end's `__getitem__` /
`__setitem__` expect (delayarray.py:114-128).  All data movement and compute
goes through libdrhip; nothing here computes on the host.
"""
import numbers
import warnings

import numpy as np
import numpy.lib.mixins

from . import hiprt

_CHECKED_DTYPES = set()
SUPPORTED_DTYPES = ("float32", "float64", "int32", "int64", "bool", "uint8", "uint32")
_WIDENED = set()        # types whose widening on upload has been announced


class Buffer:
    """One pooled device allocation shared by all views of an array.

    `version` counts writes, so results cached on expression nodes can tell when
    a leaf changed under them.  `shadow` is a second allocation of the same size
    used for ping-pong updates when a fused write would read what it
    overwrites (see hip.run_into); `shadow_region` names the part of the buffer
    that `shadow` does NOT mirror (everything outside it is identical)."""

    __slots__ = ("ptr", "nbytes", "version", "shadow", "shadow_region", "__weakref__")

    def __init__(self, nbytes, ptr=None):
        self.nbytes = int(nbytes)
        self.ptr = self.shadow = None
        if ptr is None:
            hiprt.init()
            ptr = hiprt.malloc(max(self.nbytes, 1))
        self.ptr = ptr
        self.version = 0
        self.shadow = None
        self.shadow_region = None

    def touch(self):
        """Record a write that did not go through the ping-pong path."""
        self.version += 1
        self.shadow_region = None

    def __del__(self, _free=hiprt.free):
        # `_free` is bound at definition time: module globals may already be gone
        # when buffers are finalised at interpreter exit
        if self.ptr:
            _free(self.ptr)
            self.ptr = None
        if self.shadow:
            _free(self.shadow)
            self.shadow = None


class _Placeholder(Buffer):
    """A buffer without device memory, for generating and compiling kernels on a
    machine with no GPU.  Kernels are never launched on it."""

    __slots__ = ()

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = 0
        self.version = 0
        self.shadow = None
        self.shadow_region = None


def _contiguous_strides(shape):
    strides = []
    acc = 1
    for d in reversed(shape):
        strides.append(acc)
        acc *= d
    return tuple(reversed(strides))


class ndarray(numpy.lib.mixins.NDArrayOperatorsMixin):
    """N-dimensional view of device memory."""

    __array_priority__ = 100

    def __init__(self, shape, dtype, buf=None, offset=0, strides=None):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = np.dtype(dtype)
        if self.dtype not in _CHECKED_DTYPES:        # `dtype.name` is slow: look once per dtype
            if self.dtype.name not in SUPPORTED_DTYPES:
                raise TypeError(f"dtype {self.dtype} is not supported on the device")
            _CHECKED_DTYPES.add(self.dtype)
        self._strides = _contiguous_strides(self.shape) if strides is None else tuple(strides)
        self.offset = int(offset)
        size = 1
        for d in self.shape:
            size *= d
        self.size = size
        self.buf = Buffer(size * self.dtype.itemsize) if buf is None else buf

    # ---- geometry --------------------------------------------------------

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def strides(self):
        """Byte strides, as NumPy reports them."""
        return tuple(s * self.dtype.itemsize for s in self._strides)

    @property
    def ptr(self):
        """Device address of element [0, 0, ...]."""
        return self.buf.ptr + self.offset * self.dtype.itemsize

    @property
    def is_contiguous(self):
        expect = 1
        for d, s in zip(reversed(self.shape), reversed(self._strides)):
            if d != 1 and s != expect:
                return False
            expect *= d
        return True

    def __len__(self):
        if not self.shape:
            raise TypeError("len() of unsized object")
        return self.shape[0]

    # ---- host <-> device -------------------------------------------------

    @classmethod
    def from_host(cls, host):
        host = np.asarray(host)
        if not host.flags.c_contiguous:       # (ascontiguousarray would make 0-d into 1-d)
            host = np.ascontiguousarray(host)
        if host.dtype.name not in SUPPORTED_DTYPES:
            # Types without a device form are widened to one that holds every value (said
            # once per type: the result's dtype, and with it the rounding or wrap-around
            # of later arithmetic, is then the wider type's, not NumPy's for the narrow one).
            if host.dtype.kind in "iu":
                if host.dtype == np.uint64 and host.size and int(host.max()) > np.iinfo(np.int64).max:
                    raise OverflowError("uint64 values of 2**63 and more have no device form "
                                        "(uint64 arrays are held as int64)")
                wide = np.int64
            elif host.dtype.kind == "f" and host.dtype.itemsize < 4:
                wide = np.float32
            else:
                raise TypeError(f"dtype {host.dtype} is not supported on the device")
            if host.dtype.name not in _WIDENED:
                _WIDENED.add(host.dtype.name)
                warnings.warn(f"delayrepay_amd: {host.dtype.name} arrays are held as "
                              f"{np.dtype(wide).name} on the device; results have that type",
                              RuntimeWarning, stacklevel=3)
            host = host.astype(wide)
        out = cls(host.shape, host.dtype)
        if host.nbytes:
            hiprt.memcpy_h2d(out.buf.ptr, host.ctypes.data, host.nbytes)
        return out

    def get(self):
        """Copy to a host `numpy.ndarray` (blocks)."""
        src = self if self.is_contiguous else self.copy()
        host = np.empty(self.shape, dtype=self.dtype)
        if host.nbytes:
            hiprt.memcpy_d2h(host.ctypes.data, src.ptr, host.nbytes)
        return host

    def __array__(self, dtype=None, copy=None):
        host = self.get()
        return host if dtype is None else host.astype(dtype, copy=False)

    def item(self):
        return self.get().item()

    def __float__(self):
        return float(self.get())

    def __int__(self):
        return int(self.get())

    def __bool__(self):
        return bool(self.get())

    def __index__(self):
        return self.get().__index__()

    def __repr__(self):
        return "device_" + repr(self.get())

    def __str__(self):
        return str(self.get())

    # ---- views -----------------------------------------------------------

    def _view(self, shape, strides, offset):
        view = ndarray.__new__(ndarray)     # same buffer and dtype: nothing to validate
        view.shape = tuple(shape)
        view.dtype = self.dtype
        view._strides = tuple(strides)
        view.offset = offset
        size = 1
        for d in view.shape:
            size *= d
        view.size = size
        view.buf = self.buf
        return view

    def __getitem__(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        # the same few slices of one array come back every pass of an iterative loop
        try:
            token = tuple((k.start, k.stop, k.step) if type(k) is slice else k for k in key)
            cache = self.__dict__.setdefault("_views", {})
            hit = cache.get(token)
            if hit is not None:
                return hit
        except TypeError:            # an unhashable index: no caching
            token = cache = None
        view = self._index(key)
        if cache is not None and len(cache) < 32:
            cache[token] = view
        return view

    def _index(self, key):
        n_specified = sum(1 for k in key if k is not None and k is not Ellipsis)
        if n_specified > self.ndim:
            raise IndexError("too many indices for array")
        if sum(1 for k in key if k is Ellipsis) > 1:
            raise IndexError("an index can only have a single ellipsis")
        shape, strides, offset = [], [], self.offset
        dim = 0
        for k in key:
            if k is None:
                shape.append(1)
                strides.append(0)
            elif k is Ellipsis:
                for _ in range(self.ndim - n_specified):
                    shape.append(self.shape[dim])
                    strides.append(self._strides[dim])
                    dim += 1
            elif isinstance(k, slice):
                start, stop, step = k.indices(self.shape[dim])
                length = len(range(start, stop, step))
                shape.append(length)
                strides.append(self._strides[dim] * step)
                offset += start * self._strides[dim]
                dim += 1
            elif isinstance(k, (numbers.Integral, np.integer)):
                idx = int(k)
                if idx < 0:
                    idx += self.shape[dim]
                if not 0 <= idx < self.shape[dim]:
                    raise IndexError(f"index {int(k)} is out of bounds for axis {dim} "
                                     f"with size {self.shape[dim]}")
                offset += idx * self._strides[dim]
                dim += 1
            else:
                raise NotImplementedError(
                    f"only basic indexing is supported on device arrays, not {type(k).__name__}")
        while dim < self.ndim:
            shape.append(self.shape[dim])
            strides.append(self._strides[dim])
            dim += 1
        return self._view(shape, strides, offset)

    def check_writable(self):
        """A view that repeats elements (a stride of zero along an axis longer than one, as
        `broadcast_to` makes them) is read-only, as in NumPy: one write would land on
        every repeat and on the source."""
        for d, s in zip(self.shape, self._strides):
            if d > 1 and s == 0:
                raise ValueError("assignment destination is read-only")

    def __setitem__(self, key, value):
        from . import hip
        self.check_writable()
        dst = self[key]
        hip.assign(dst, value)

    def broadcast_to(self, shape):
        """View with NumPy's broadcasting applied: new and stretched axes get stride 0."""
        shape = tuple(int(d) for d in shape)
        lead = len(shape) - self.ndim
        if lead < 0:
            raise ValueError(f"cannot broadcast shape {self.shape} to {shape}")
        strides = [0] * lead
        for have, want, stride in zip(self.shape, shape[lead:], self._strides):
            if have == want:
                strides.append(stride)
            elif have == 1:
                strides.append(0)
            else:
                raise ValueError(f"cannot broadcast shape {self.shape} to {shape}")
        return self._view(shape, strides, self.offset)

    def reshape(self, *shape, **kwargs):
        if len(shape) == 1 and not isinstance(shape[0], numbers.Integral):
            shape = tuple(shape[0])
        shape = list(int(d) for d in shape)
        if shape.count(-1) > 1:
            raise ValueError("can only specify one unknown dimension")
        if -1 in shape:
            known = 1
            for d in shape:
                if d != -1:
                    known *= d
            shape[shape.index(-1)] = self.size // known if known else 0
        total = 1
        for d in shape:
            total *= d
        if total != self.size:
            raise ValueError(f"cannot reshape array of size {self.size} into shape {tuple(shape)}")
        src = self if self.is_contiguous else self.copy()
        return ndarray(shape, self.dtype, src.buf, src.offset)

    def ravel(self):
        return self.reshape(self.size)

    def transpose(self, *axes):
        if not axes or axes == (None,):
            axes = tuple(reversed(range(self.ndim)))
        elif len(axes) == 1 and not isinstance(axes[0], numbers.Integral):
            axes = tuple(axes[0])
        if sorted(a % max(self.ndim, 1) for a in axes) != list(range(self.ndim)):
            raise ValueError("axes don't match array")
        axes = [a % self.ndim for a in axes]
        return self._view([self.shape[a] for a in axes], [self._strides[a] for a in axes],
                          self.offset)

    @property
    def T(self):
        return self.transpose()

    # ---- device-side operations -----------------------------------------

    def copy(self):
        """New contiguous array with the same contents."""
        from . import hip
        return hip.materialise(self)

    def astype(self, dtype, copy=True, **kwargs):
        from . import hip
        dtype = np.dtype(dtype)
        if dtype == self.dtype and not copy:
            return self
        return hip.materialise(self, dtype)

    def fill(self, value):
        from . import hip
        hip.assign(self, value)

    # arithmetic on a raw device array re-enters the lazy front end
    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        from .delayarray import NPArray
        wrapped = [NPArray(x) if isinstance(x, ndarray) else x for x in inputs]
        return getattr(ufunc, method)(*wrapped, **kwargs)

    def __array_function__(self, func, types, args, kwargs):
        from .delayarray import NPArray
        wrapped = [NPArray(x) if isinstance(x, ndarray) else x for x in args]
        return func(*wrapped, **kwargs)

    def sum(self, *args, **kwargs):
        return np.sum(self, *args, **kwargs)

    def max(self, *args, **kwargs):
        return np.max(self, *args, **kwargs)

    def min(self, *args, **kwargs):
        return np.min(self, *args, **kwargs)


def placeholder(shape, dtype, strides=None, offset=0, buf=None):
    """Array without device memory: lets kernels be generated and compiled (not
    launched) on a machine that has no GPU."""
    size = 1
    for d in shape:
        size *= d
    if buf is None:
        buf = _Placeholder((offset + size) * np.dtype(dtype).itemsize)
    return ndarray(shape, dtype, buf, offset, strides)
