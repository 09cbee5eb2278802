"""Lazy NumPy look-alike: arithmetic builds a hash-consed expression DAG.

Public names and protocol behaviour follow the reference's front end
(delayrepay/delayarray.py): `DelayArray` intercepts NumPy ufuncs through
`__array_ufunc__` (:46-61) and builds nodes instead of computing; a value is
produced only when one is asked for (`get`, `run`, `repr`, indexing; :35-44,
:101-128), by handing the whole DAG to the backend's `run` (:43).

Deliberate differences from the reference, each needed for NumPy-exact results
or bounded memory:
  * the hash-cons table is keyed on (class, function, child identities, exact
    scalar type and value) and holds nodes weakly; the reference keys on
    `hash(args)` (:224-231), under which `Scalar(-1)`/`Scalar(-2)` and `2`/`2.0`
    collide, and keeps every leaf alive for ever;
  * NumPy >= 2 names the division ufunc `divide`; both spellings are accepted
    (the reference's table knows only `true_divide`, :162-168);
  * shapes follow NumPy broadcasting and stay lazy (the reference computes
    unequal shapes eagerly, :47-55);
  * dtypes follow NumPy promotion with weak Python scalars instead of being
    copied between siblings (:462-467);
  * `astype` on a leaf returns a new leaf instead of converting in place (:401-408);
  * an evaluated node is reused as a leaf by later expressions, and a cached
    result is dropped when a leaf it was computed from has been written since;
  * `sum` builds a `ReduceEx` (a stub in the reference, :272-283) that the HIP
    backend fuses with the element-wise body;
  * `dst[key] = lazy_expression` is handed to the backend as one fused write;
  * `evaluate(a, b, ...)` computes several roots in one kernel.
"""
import builtins
import math
import numbers
import weakref

import numpy as np
import numpy.lib.mixins

from . import backend as be
from .promote import PY_DESCR, result_dtype, scalar_descr

_backend = be.backend
# A backend whose arrays carry no version of their own (NumPy's) cannot tell which results
# a write has made stale, so every write through `__setitem__` is counted and a result
# evaluated before the latest one is computed again when it is next asked for: on every
# backend an evaluated expression follows its leaves.
_COUNTS_WRITES = bool(getattr(_backend, "COUNTS_WRITES", False))
_WRITES = [0]


def cast(func):
    """Decorator: wrap a backend array returned by `func` as a lazy leaf
    (cf. delayarray.py:13-22)."""

    def wrapper(*args, **kwargs):
        res = func(*args, **kwargs)
        if isinstance(res, DelayArray):
            return res
        return NPArray(res)

    wrapper.__name__ = getattr(func, "__name__", "wrapped")
    wrapper.__doc__ = getattr(func, "__doc__", None)
    return wrapper


def _unwrap(obj):
    """Backend array (or plain object) behind a lazy array."""
    if isinstance(obj, DelayArray):
        return obj._force()
    return obj


class DelayArray(numpy.lib.mixins.NDArrayOperatorsMixin):
    """Base of every node; also the user-visible array type."""

    count = 0  # global creation serial (delayarray.py:27-32)

    def __init__(self, *args, **kwargs):
        self._count = DelayArray.count
        DelayArray.count += 1

    # ---- forcing ---------------------------------------------------------

    def _force(self):
        """Evaluate (once) and return the backend array."""
        d = self.__dict__
        arr = d.get("array")
        if arr is not None:
            deps = d.get("_deps")
            if deps is None:
                if d.get("_epoch", _WRITES[0]) == _WRITES[0]:
                    return arr
            elif all(buf.version == ver for buf, ver in deps):
                return arr
            del self.array  # a leaf was written to since: recompute
        self.array = _evaluate(_backend.run, self)
        self._depth = 0     # a leaf of whatever is built on it from now on
        if _COUNTS_WRITES and self.children:
            self._epoch = _WRITES[0]
        return self.array

    def __array__(self, dtype=None, copy=None):
        """Host `numpy.ndarray` holding the value (NumPy's conversion protocol)."""
        host = self.get()
        if dtype is not None and host.dtype != dtype:
            host = host.astype(dtype)
        return host

    def get(self):
        """Evaluate and copy to the host (delayarray.py:101-106)."""
        arr = self._force()
        getter = getattr(arr, "get", None)
        return getter() if getter is not None else arr

    def run(self):
        """Evaluate on the device without copying back (delayarray.py:108-109)."""
        self._force()

    def __repr__(self):
        return str(self.get())

    def __float__(self):
        return float(self.get())

    def __int__(self):
        return int(self.get())

    def __bool__(self):
        return bool(self.get())

    # ---- NumPy protocols -------------------------------------------------

    def __array_ufunc__(self, ufunc, method, *inputs, **kwargs):
        if method == "__call__" and not kwargs and len(inputs) == 1 and ufunc.__name__ != "square":
            return _unary(ufunc, self)          # `sqrt(x)`, `exp(x)`: the common, short way
        if method == "reduce" and ufunc.__name__ in ("add", "maximum", "minimum"):
            return _reduce(ufunc, inputs[0], **kwargs)
        if method != "__call__":
            return NotImplemented
        target = None
        if kwargs:
            out = kwargs.get("out")
            if isinstance(out, tuple) and len(out) == 1 and isinstance(out[0], DelayArray):
                # `np.multiply(a, b, out=c)`: the fused kernel writes straight into c
                target = out[0]
                kwargs = {k: v for k, v in kwargs.items() if k != "out"}
            bad = [k for k, v in kwargs.items() if v is not None]
            if bad:
                raise NotImplementedError(f"ufunc keyword(s) {bad} are not supported on lazy arrays")
        if ufunc.__name__ == "matmul":
            return self._dot(inputs, {})
        args = [arg_to_numpy_ex(arg) for arg in inputs]
        node = create_ex(ufunc, args)
        if target is not None:
            if tuple(node.shape) != tuple(target.shape):
                raise ValueError(f"non-broadcastable output operand with shape {tuple(target.shape)} "
                                 f"doesn't match the broadcast shape {tuple(node.shape)}")
            if not np.can_cast(node.dtype, target.dtype, casting="same_kind"):
                raise TypeError(f"Cannot cast ufunc '{ufunc.__name__}' output from {node.dtype} to "
                                f"{target.dtype} with casting rule 'same_kind'")
            target[...] = node
            return target
        return node

    def __array_function__(self, func, types, args, kwargs):
        if func.__name__ == "dot":
            return self._dot(args, kwargs)
        handler = HANDLED_FUNCTIONS.get(func)
        if handler is None:
            return NotImplemented
        return handler(*args, **kwargs)

    def __matmul__(self, other):
        return self._dot([self, other], {})

    def _dot(self, args, kwargs):
        left, right = (arg_to_numpy_ex(a) for a in args[:2])
        if len(left.shape) == 1 and len(right.shape) == 1:
            # vector . vector: fused multiply + reduction
            return _reduce(np.add, left * right)
        floats = left.dtype.kind == "f" and right.dtype.kind == "f"
        if floats and len(left.shape) == 2 and len(right.shape) == 1:
            # matrix . vector reads the matrix once: a fused row reduction streams it at
            # HBM speed, a matrix-matrix kernel with one output column does not
            if left.shape[1] != right.shape[0]:
                raise ValueError(f"shapes {left.shape} and {right.shape} not aligned")
            return _reduce(np.add, left * right, axis=1)
        if floats and len(left.shape) == 1 and len(right.shape) == 2:
            if left.shape[0] != right.shape[0]:
                raise ValueError(f"shapes {left.shape} and {right.shape} not aligned")
            return _reduce(np.add, left.reshape(left.shape[0], 1) * right, axis=0)
        return cast(_backend.fallback.dot)(left._force(), right._force())

    def dot(self, other, out=None):
        return self._dot([self, other], {})

    # The arithmetic operators build nodes directly; going through
    # NDArrayOperatorsMixin -> ufunc -> __array_ufunc__ gives the same node but
    # costs several times more host time per operation.
    def __add__(self, other):
        return _binary(np.add, self, other)

    def __radd__(self, other):
        return _binary(np.add, other, self)

    def __sub__(self, other):
        return _binary(np.subtract, self, other)

    def __rsub__(self, other):
        return _binary(np.subtract, other, self)

    def __mul__(self, other):
        return _binary(np.multiply, self, other)

    def __rmul__(self, other):
        return _binary(np.multiply, other, self)

    def __truediv__(self, other):
        return _binary(np.true_divide, self, other)

    def __rtruediv__(self, other):
        return _binary(np.true_divide, other, self)

    def __pow__(self, other):
        return create_ex(np.power, [self, arg_to_numpy_ex(other)])

    def __neg__(self):
        return UnaryFuncEx(np.negative, self)

    __iadd__, __isub__, __imul__, __itruediv__ = __add__, __sub__, __mul__, __truediv__

    def __gt__(self, other):
        return np.greater(self, other)

    def __lt__(self, other):
        return np.less(self, other)

    # ---- shape-like ------------------------------------------------------

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def __len__(self):
        if not self.shape:
            raise TypeError("len() of unsized object")
        return self.shape[0]

    @property
    def T(self):
        if len(self.shape) < 2:
            return self
        return np.transpose(self)

    def reshape(self, *args, **kwargs):
        if "array" not in self.__dict__ and not kwargs and self.ndim:
            want = args[0] if len(args) == 1 and not isinstance(args[0], (int, np.integer)) else args
            want = tuple(want) if isinstance(want, (tuple, list)) else None
            if want is not None and len(want) == self.ndim + 1 and want[-1] == 1 and \
                    builtins.all(w == d or w == -1 for w, d in zip(want, self.shape)) and want.count(-1) <= 1:
                res = _keep_last_axis(self)         # `a.sum(axis=1).reshape(-1, 1)`
                if res is not None:
                    return res
        return NPArray(self._force().reshape(*args, **kwargs))

    def copy(self):
        """Evaluated, contiguous copy as a new leaf."""
        return NPArray(_backend.fallback.copy(self._force()))

    def ravel(self):
        return self.reshape(self.size)

    def transpose(self, *axes):
        """Permuted view of the evaluated array, as a new leaf; of a small unevaluated
        element-wise expression: the expression over permuted views of its leaves."""
        if len(axes) == 1 and not isinstance(axes[0], (int, np.integer)):
            axes = tuple(axes[0]) if axes[0] is not None else ()
        return np.transpose(self, axes or None)

    flatten = ravel

    def astype(self, dtype, **kwargs):
        """Lazy cast, fused into whatever consumes it."""
        dtype = np.dtype(dtype)
        if dtype == self.dtype:
            return self
        return CastEx(dtype, self)

    # ---- indexing --------------------------------------------------------

    def __getitem__(self, key):
        """Force, then wrap the backend *view* as a new leaf (delayarray.py:123-128).
        A basic slice of a small unevaluated element-wise expression is instead the
        same expression over slices of its leaves: only the part asked for is ever
        computed, and shifted slices of one expression fuse into one stencil."""
        key = _unwrap(key)
        if "array" not in self.__dict__ and _adds_last_axis(key, self.ndim):
            res = _keep_last_axis(self)
            if res is not None:
                return res
        if "array" not in self.__dict__ and type(self) in _ELEMENTWISE and _basic_key(key):
            res = _over_views(self, lambda arr: arr[key], key)
            if res is not None:
                return res
        return NPArray(self._force()[key])

    def __setitem__(self, key, item):
        """Write into the materialised array.  A lazy right-hand side is handed
        to the backend as one fused kernel writing straight into the destination
        (the reference evaluates it to a temporary first, delayarray.py:114-121)."""
        arr = self._force()
        # written to by hand, the result is an array in its own right from now on: it
        # must not be recomputed (and the write lost) when one of its inputs changes,
        # the same expression built again must not find it (`b = a * 2; b[0] = 100;
        # c = a * 2`: c is a new node), and a backend that walks through evaluated nodes
        # stops here
        d = self.__dict__
        _WRITES[0] += 1
        if self.children:
            d.pop("_deps", None)
            d.pop("_plan", None)
            d.pop("_multi", None)
            d.pop("_epoch", None)
            d["_cut"] = True
            own = d.get("_key")
            if own is not None and Memoiser._cache.get(own) is self:
                Memoiser._cache.pop(own)
        key = _unwrap(key)
        check = getattr(arr, "check_writable", None)
        if check is not None:
            check()             # a stretched view is read-only as a whole, as in NumPy
        if isinstance(item, DelayArray) and "array" not in item.__dict__:
            _evaluate(_backend.run_into, item, arr[key])
        else:
            arr[key] = _unwrap(item)

    # ---- reductions and friends -----------------------------------------

    def sum(self, *args, **kwargs):
        node = _row_reduce(np.add, self, args, kwargs)
        return node if node is not None else np.sum(self, *args, **kwargs)

    def max(self, *args, **kwargs):
        node = _row_reduce(np.maximum, self, args, kwargs)
        return node if node is not None else np.max(self, *args, **kwargs)

    def min(self, *args, **kwargs):
        node = _row_reduce(np.minimum, self, args, kwargs)
        return node if node is not None else np.min(self, *args, **kwargs)

    def mean(self, *args, **kwargs):
        return np.mean(self, *args, **kwargs)

    def var(self, *args, **kwargs):
        return np.var(self, *args, **kwargs)

    def std(self, *args, **kwargs):
        return np.std(self, *args, **kwargs)

    def any(self, *args, **kwargs):
        return np.any(self, *args, **kwargs)

    def all(self, *args, **kwargs):
        return np.all(self, *args, **kwargs)

    def ptp(self, *args, **kwargs):
        return np.ptp(self, *args, **kwargs)

    def clip(self, a_min=None, a_max=None, **kwargs):
        return np.clip(self, a_min, a_max, **kwargs)

    def cumsum(self, *args, **kwargs):
        return np.cumsum(self, *args, **kwargs)

    def squeeze(self, axis=None):
        return np.squeeze(self, axis)

    def swapaxes(self, axis1, axis2):
        return np.swapaxes(self, axis1, axis2)

    def trace(self, *args, **kwargs):
        return np.trace(self, *args, **kwargs)

    def item(self, *args):
        """The element as a Python number (of a one-element array when no index is given)."""
        return self.get().item(*args)

    def tolist(self):
        return self.get().tolist()

    def fill(self, value):
        self[...] = value

    @property
    def itemsize(self):
        return np.dtype(self.dtype).itemsize

    @property
    def nbytes(self):
        return self.size * self.itemsize

    def repeat(self, *args, **kwargs):
        return repeat(self, *args, **kwargs)

    # ---- code-generation helpers ----------------------------------------

    @property
    def name(self):
        return f"arr{self._count}"

    @property
    def inputs(self):
        return {self.name: self}


# ufunc name -> C infix operator (delayarray.py:162-168, plus NumPy 2's `divide`)
OPS = {
    "matmul": "@",
    "add": "+",
    "multiply": "*",
    "subtract": "-",
    "true_divide": "/",
    "divide": "/",
}

# ufunc name -> C function spelling (delayarray.py:171-186, widened)
FUNCS = {
    "power": "pow",
    "arctan2": "atan2",
    "absolute": "abs",
    "sin": "sin",
    "cos": "cos",
    "tan": "tan",
    "sqrt": "sqrt",
    "log": "log",
    "negative": "-",
    "exp": "exp",
    "tanh": "tanh",
    "sinh": "sinh",
    "cosh": "cosh",
    "arcsin": "asin",
    "arccos": "acos",
    "arctan": "atan",
    "exp2": "exp2",
    "expm1": "expm1",
    "log2": "log2",
    "log10": "log10",
    "log1p": "log1p",
    "cbrt": "cbrt",
    "erf": "erf",
    "erfc": "erfc",
    "floor": "floor",
    "ceil": "ceil",
    "trunc": "trunc",
    "rint": "rint",
    "reciprocal": "1/",
    "positive": "+",
    "maximum": "max",
    "minimum": "min",
    "fmax": "fmax",
    "fmin": "fmin",
    "hypot": "hypot",
    "copysign": "copysign",
    "fmod": "fmod",
    "greater": ">",
    "less": "<",
    "greater_equal": ">=",
    "less_equal": "<=",
    "equal": "==",
    "not_equal": "!=",
}

ufunc_lookup = {
    "matmul": _backend.np.matmul,
    "add": _backend.np.add,
    "multiply": _backend.np.multiply,
    "subtract": _backend.np.subtract,
    "true_divide": _backend.np.true_divide,
    "divide": _backend.np.true_divide,
}


def calc_shape(left, right, op=None):
    """Result shape of a binary node: NumPy broadcasting (a scalar is `()`)."""
    if left == right or not right:
        return left
    if not left:
        return right
    return tuple(np.broadcast_shapes(left, right))


_PY_DESCR = PY_DESCR
_ARRAY_DESCR = {}


def _descr(node):
    """What NumPy's type resolution needs to know about an operand."""
    if type(node) is Scalar:
        return node._descr
    dt = node.dtype
    try:
        return _ARRAY_DESCR[dt]
    except KeyError:
        return _ARRAY_DESCR.setdefault(dt, ("a", dt.str))


_scalar_descr = scalar_descr


def calc_type(func, children):
    if len(children) == 2:
        return result_dtype(func, (_descr(children[0]), _descr(children[1])))
    return result_dtype(func, tuple(_descr(c) for c in children))


class _Ref(weakref.ref):
    """Weak reference that remembers its table key (`weakref.KeyedRef` does the same
    through a `__new__` and an `__init__` written in Python, two more frames per node)."""

    __slots__ = ("key",)


class _WeakTable:
    """key -> node, holding nodes weakly (a lean WeakValueDictionary: node
    construction is on the host's hot path)."""

    def __init__(self):
        self.data = data = {}

        def gone(ref):
            if data.get(ref.key) is ref:
                del data[ref.key]
        self._gone = gone

    def get(self, key):
        ref = self.data.get(key)
        return ref() if ref is not None else None

    def __setitem__(self, key, node):
        ref = self.data[key] = _Ref(node, self._gone)
        ref.key = key

    def pop(self, key, default=None):
        ref = self.data.pop(key, None)
        return ref() if ref is not None else default

    def __len__(self):
        return len(self.data)

    def clear(self):
        self.data.clear()


class Memoiser(type):
    """Metaclass that hash-conses node construction: building the same node
    twice yields the same object, so expressions form a DAG
    (cf. delayarray.py:216-231; tests/test.py:145-162)."""

    _cache = _WeakTable()

    def __call__(cls, *args, _table=_cache, _get=_cache.data.get, _ref=_Ref):
        key = cls._memo_key(*args)
        ref = _get(key)
        node = ref() if ref is not None else None
        if node is None:
            node = type.__call__(cls, *args)
            node._key = key
            ref = _table.data[key] = _ref(node, _table._gone)
            ref.key = key
        return node


def reset():
    """Forget every hash-consed node (delayarray.py:234-236) and every cached plan."""
    Memoiser._cache.clear()
    _NUMBERS.clear()
    forget = getattr(_backend, "forget", None)
    if forget is not None:
        forget()


# An expression this many operations deep has its deepest operand evaluated before it
# grows further (`x = f(x)` in a loop that never asks for a value): the walkers over
# the DAG recurse, and nobody wants a kernel of thousands of operations.
MAX_DEPTH = 128

class NumpyEx(DelayArray, metaclass=Memoiser):
    """Interior or leaf node of the expression DAG."""

    children = ()
    _depth = 0

    def __init__(self, children=()):
        super().__init__()
        self.children = children = list(children)
        if children:
            depth = 0
            for c in children:
                if c._depth > depth:
                    depth = c._depth
            if depth >= MAX_DEPTH:
                depth = 0
                for c in children:
                    if c._depth >= MAX_DEPTH:
                        c._force()
                        c._cut = True       # backends that re-walk evaluated nodes stop here
                    if c._depth > depth:
                        depth = c._depth
            self._depth = depth + 1

    def _seal(self):
        """Turn this evaluated node into a plain holder of its array: it forgets what it
        was computed from (and lets go of it), is never recomputed, and building the
        same expression again makes a new node."""
        d = self.__dict__
        d.pop("_deps", None)
        d.pop("_plan", None)
        d.pop("_multi", None)
        d.pop("_gen", None)
        key = d.get("_key")
        if key is not None and Memoiser._cache.get(key) is self:
            Memoiser._cache.pop(key)
        self.children = []
        self._depth = 0

    @classmethod
    def _memo_key(cls, func, *children):
        # children are kept alive by the node, so their ids stay unique while the
        # table entry exists
        if len(children) == 2:
            return (cls, func, id(children[0]), id(children[1]))
        return (cls, func) + tuple(id(c) for c in children)

    def __hash__(self):
        return id(self)

    @property
    def inputs(self):
        """Ordered, de-duplicated leaves (name -> node): kernel operand order."""
        found = {}
        stack = [self]
        seen = set()
        order = []
        while stack:
            node = stack.pop()
            if id(node) in seen:
                continue
            seen.add(id(node))
            if isinstance(node, NPArray) or "array" in node.__dict__:
                order.append(node)
            else:
                stack.extend(reversed(node.children))
        for node in order:
            found[node.name] = node
        return found


class Funcable:
    def to_op(self):
        return OPS[self.func.__name__]


class ReduceEx(NumpyEx, Funcable):
    """Reduction of an expression with a binary ufunc (`add`, `maximum`, `minimum`),
    over everything (`axis` None) or over a tuple of axes; evaluated as the tail of
    the fused element-wise kernel."""

    def __init__(self, func, arg, axis=None, keepdims=False):
        super().__init__(children=[arg])
        self.func = func
        self.axis = axis
        self.keepdims = keepdims
        if keepdims:
            self.shape = tuple(1 if (axis is None or k in axis) else d for k, d in enumerate(arg.shape))
        elif axis is None:
            self.shape = ()
        else:
            self.shape = tuple(d for k, d in enumerate(arg.shape) if k not in axis)
        self.dtype = arg.dtype

    @classmethod
    def _memo_key(cls, func, arg, axis=None, keepdims=False):
        return (cls, func, id(arg), axis, keepdims)

    @property
    def name(self):
        return f"redex{self._count}"


class UnaryFuncEx(NumpyEx, Funcable):
    def __init__(self, func, arg):
        super().__init__(children=[arg])
        self.func = func
        self.shape = arg.shape
        self.dtype = calc_type(func, [arg])

    def to_op(self):
        return FUNCS[self.func.__name__]

    @property
    def name(self):
        return f"unfunc{self._count}"


class CastEx(NumpyEx):
    """`astype` on a lazy expression: a conversion fused into the kernel."""

    def __init__(self, dtype, arg):
        super().__init__(children=[arg])
        self.shape = arg.shape
        self.dtype = np.dtype(dtype)

    @classmethod
    def _memo_key(cls, dtype, arg):
        return (cls, np.dtype(dtype).str, id(arg))

    @property
    def name(self):
        return f"cast{self._count}"


class BinaryFuncEx(NumpyEx):
    def __init__(self, func, left, right):
        super().__init__(children=[left, right])
        self.func = func
        self.shape = calc_shape(left.shape, right.shape, func)
        self.dtype = calc_type(func, [left, right])

    def to_op(self):
        return FUNCS[self.func.__name__]

    @property
    def name(self):
        return f"binfun{self._count}"


class BinaryNumpyEx(NumpyEx, Funcable):
    """`+ - * /` node."""

    def __init__(self, func, left, right):
        super().__init__(children=[left, right])
        self.func = func
        self.shape = calc_shape(left.shape, right.shape, func)
        self.dtype = calc_type(func, [left, right])

    @property
    def name(self):
        return f"binex{self._count}"


class WhereEx(NumpyEx):
    """`where(cond, x, y)`: element-wise selection, fused like any other node."""

    def __init__(self, func, cond, x, y):
        super().__init__(children=[cond, x, y])
        self.func = func
        self.shape = calc_shape(calc_shape(cond.shape, x.shape), y.shape)
        self.dtype = calc_type(np.add, [x, y])

    @property
    def name(self):
        return f"where{self._count}"


_ELEMENTWISE = (BinaryNumpyEx, BinaryFuncEx, UnaryFuncEx, WhereEx, CastEx)


def pow_ex(func, left, right):
    """`x ** k` with a Python-int k >= 2 becomes k-1 left-associated multiplies
    (delayarray.py:316-324), k == 1 is x itself.  The reference returns x for every
    k <= 1 as well; here k <= 0 gives what NumPy's `**` gives: `x**0` is ones,
    `x**-1` is `1/x` (correctly rounded, NumPy's own shortcut), other negative k go to
    `power`; an integer array to a negative power is an error, as in NumPy."""
    exponent = right.val if isinstance(right, Scalar) else None
    if not isinstance(exponent, int) or isinstance(exponent, bool):
        return BinaryFuncEx(func, left, right)
    if exponent < 1:
        integral = left.dtype.kind in "iu"
        if exponent < 0 and (integral or left.dtype.kind == "b"):
            raise ValueError("Integers to negative integer powers are not allowed.")
        if exponent == 0 and integral:
            return left * 0 + 1
        if exponent == -1 and left.dtype.kind == "f":
            return UnaryFuncEx(np.reciprocal, left)
        return BinaryFuncEx(func, left, right)
    ex = left
    for _ in range(exponent - 1):
        ex = BinaryNumpyEx(np.multiply, ex, left)
    return ex


def create_ex(func, args):
    """Node factory with the reference's rewrites (delayarray.py:327-336)."""
    name = func.__name__
    if name in OPS:
        return BinaryNumpyEx(func, *args)
    if name == "square":
        return BinaryNumpyEx(np.multiply, args[0], args[0])
    if len(args) == 1:
        return UnaryFuncEx(func, *args)
    if name == "power":
        return pow_ex(func, *args)
    return BinaryFuncEx(func, *args)


class NPArray(NumpyEx):
    """Leaf: a backend array."""

    def __init__(self, array):
        super().__init__()
        if not _backend.is_ndarray(array):
            array = _backend.fallback.asarray(array)
        self.array = array
        self.shape = tuple(array.shape)
        self.dtype = np.dtype(array.dtype)

    @classmethod
    def _memo_key(cls, array):
        # Device views with the same buffer and geometry are the same leaf, so the
        # slices an iterative loop re-creates every pass (`u[1:-1, 2:]`) map to the
        # same node, and the expression built on them to the same DAG.
        buf = getattr(array, "buf", None)
        if buf is not None:
            return (cls, id(buf), array.offset, array.shape, array._strides, array.dtype.str)
        return (cls, id(array))

    def _force(self):
        return self.array

    def astype(self, dtype, **kwargs):
        """Converted copy as a new leaf.  (The reference converts the leaf in place
        and returns the same wrapper, delayarray.py:401-408, which silently changes
        every expression already built on it; `arr = arr.astype(t)`, the form its
        tests use at tests/test.py:59-62,74-77, behaves the same either way.)"""
        dtype = np.dtype(dtype)
        if dtype == self.dtype:
            return self
        return NPArray(self.array.astype(dtype, **kwargs))

    @property
    def name(self):
        return f"arr{self._count}"

    @property
    def inputs(self):
        return {self.name: self}


class Scalar(NumpyEx):
    """A number.  Python numbers are weak (they take the dtype of the array
    they meet); NumPy scalars keep theirs."""

    def __init__(self, val):
        super().__init__()
        self.val = val
        self.shape = ()
        self._descr = _scalar_descr(val)

    @classmethod
    def _memo_key(cls, val):
        # 2 and 2.0 differ by type; 0.0 and -0.0 (equal, same type) by their text
        return (cls, type(val), val if val else repr(val))

    @property
    def dtype(self):
        return np.asarray(self.val).dtype

    def _force(self):
        return self.val

    @property
    def name(self):
        return str(self.val)

    @property
    def inputs(self):
        return {}


class _Generated(NumpyEx):
    """Base of leaves that are computed from the element index instead of read from
    memory.  Every call makes a new node (never hash-consed): like any new array it
    may be written to later, and two arrays must not share such a write."""

    _serial = 0

    @classmethod
    def _memo_key(cls, *args):
        _Generated._serial += 1
        return (cls, _Generated._serial)

    @property
    def version(self):
        """Results computed from this node while it was still lazy list it among their
        dependencies, like a buffer, with version 0; once it has become an array it
        may be written to, and those results are computed afresh."""
        return 1 if "array" in self.__dict__ else 0

    def _force(self):
        arr = self.__dict__.get("array")
        if arr is None:
            arr = self.array = _backend.run(self)
            self.__dict__.pop("_deps", None)     # from now on an array in its own right
        return arr

    @property
    def inputs(self):
        return {}


class FullEx(_Generated):
    """`full(shape, value)` (and `zeros`, `ones`) that has not been written to: inside
    an expression it is a scalar kernel parameter and costs no memory traffic;
    asked for on its own, or indexed, or assigned to, it becomes an ordinary array
    (delayarray.py:596-604 allocate and fill at once)."""

    def __init__(self, shape, val, dtype):
        super().__init__()
        self.shape = tuple(shape)
        self.dtype = np.dtype(dtype)
        self.val = self.dtype.type(val)

    @property
    def name(self):
        return f"full{self._count}"


class IotaEx(_Generated):
    """0, 1, 2, ... n-1 in `dtype`: the index sequence `arange` and `linspace` are
    built on.  Costs no memory traffic inside a 1-d expression of the same length."""

    def __init__(self, n, dtype):
        super().__init__()
        self.shape = (int(n),)
        self.dtype = np.dtype(dtype)

    @property
    def name(self):
        return f"iota{self._count}"


class RandEx(_Generated):
    """`n` consecutive outputs of a Philox-4x64-10 stream (`numpy.random.Philox` with
    the same key and counter), starting `pos` outputs into it: raw 64-bit words (dtype
    int64, the same bits as NumPy's uint64), doubles in [0, 1) made from their top 53
    bits as `numpy.random.Generator.random` makes them, or floats in [0, 1) made from the
    top 24 bits of each half of an output, low half first, as `random(dtype=float32)`
    makes them (`pos` then counts halves).  Every element is a function of its index
    alone, so inside a 1-d expression of the same length it is computed in the kernel
    and costs no memory traffic; made by `random.device(seed)`."""

    def __init__(self, n, key, counter, pos, dtype):
        super().__init__()
        self.shape = (int(n),)
        self.dtype = np.dtype(dtype)
        if self.dtype not in (np.int64, np.float64, np.float32):
            raise TypeError("a Philox stream yields int64 words, float64 or float32 numbers")
        self.key = int(key)
        self.counter = int(counter)        # counter of the block that holds output 0
        self.pos = int(pos)

    @property
    def name(self):
        return f"rand{self._count}"


PUSH_VIEWS_UP_TO = 48     # interior nodes; larger expressions are evaluated once, then viewed


def _basic_key(key):
    if not isinstance(key, tuple):
        key = (key,)
    return all(k is None or k is Ellipsis or isinstance(k, (slice, int, np.integer)) for k in key)


def _over_views(root, view, key=None):
    """The unevaluated element-wise expression `root` rebuilt over `view(leaf)` of each
    leaf, every leaf first broadcast to the root's shape (so one view function serves
    all of them); None when the expression is too large or holds something that has
    to be evaluated first."""
    shape = tuple(root.shape)
    fb = _backend.fallback
    if getattr(fb, "broadcast_to", None) is None:
        return None
    memo = {}
    budget = [PUSH_VIEWS_UP_TO]
    new_shape = tuple(view(np.broadcast_to(np.empty((), dtype=bool), shape)).shape)
    sl = key[0] if isinstance(key, tuple) and len(key) == 1 else key
    sl = sl if isinstance(sl, slice) and len(shape) == 1 else None

    def walk(node):
        hit = memo.get(id(node))
        if hit is not None:
            return hit
        kind = type(node)
        arr = node.__dict__.get("array")
        if kind is Scalar:
            res = node
        elif arr is not None and kind is not FullEx and kind is not IotaEx or kind is NPArray:
            res = NPArray(view(fb.broadcast_to(node._force(), shape)))
        elif kind is FullEx and arr is None:
            res = FullEx(new_shape, node.val, node.dtype)
        elif kind is IotaEx and arr is None and sl is not None and node.shape == shape \
                and shape[0] <= (1 << 24 if node.dtype == np.float32 else 1 << 53):
            # a slice of 0, 1, 2, ... is start + step * (0, 1, 2, ...): still no memory
            picked = range(shape[0])[sl]
            res = IotaEx(len(picked), node.dtype)
            if picked.step != 1:
                res = res * node.dtype.type(picked.step)
            if picked.start != 0:
                res = res + node.dtype.type(picked.start)
        elif kind in _ELEMENTWISE:
            budget[0] -= 1
            if budget[0] < 0:
                raise _TooLarge
            kids = [walk(c) for c in node.children]
            if kind is CastEx:
                res = CastEx(node.dtype, kids[0])
            else:
                res = kind(node.func, *kids)
        else:       # reductions, index arrays, written-to constants: evaluate, then view
            res = NPArray(view(fb.broadcast_to(node._force(), shape)))
        memo[id(node)] = res
        return res

    try:
        return walk(root)
    except _TooLarge:
        return None
    finally:
        # `walk` refers to itself through its closure, a reference cycle: empty what the
        # cycle holds (nodes and their arrays) rather than leave it to the cycle collector
        memo.clear()
        walk = view = fb = None


class _TooLarge(Exception):
    pass


def _adds_last_axis(key, ndim):
    """Whether indexing with `key` only appends an axis of one: `[:, None]`, `[..., None]`."""
    key = key if isinstance(key, tuple) else (key,)
    if len(key) < 2 or key[-1] is not None:
        return False
    head = key[:-1]
    if len(head) == 1 and head[0] is Ellipsis:
        return True
    return len(head) == ndim and builtins.all(isinstance(k, slice) and k == slice(None) for k in head)


def _keep_last_axis(root):
    """`root[..., None]` of an unevaluated expression over reductions along the last axis
    that are still lazy (`a.sum(axis=1)`, `a.max(axis=1) * 2`): the same expression over their
    `keepdims` twins, which the backend's row kernel takes as operands, so that
    `a / a.sum(axis=1)[:, None]` reads every row once.  None when the expression holds no
    such reduction (the caller then indexes as usual)."""
    memo = {}
    found = [False]
    budget = [PUSH_VIEWS_UP_TO]

    def walk(node):
        hit = memo.get(id(node))
        if hit is not None:
            return hit
        kind = type(node)
        arr = node.__dict__.get("array")
        if kind is Scalar:
            res = node
        elif kind is ReduceEx and arr is None and not node.keepdims and node.axis is not None \
                and node.axis == (node.children[0].ndim - 1,):
            found[0] = True
            res = ReduceEx(node.func, node.children[0], node.axis, True)
        elif arr is not None or kind is NPArray:
            res = NPArray(node._force()[..., None])
        elif kind in _ELEMENTWISE and kind is not CastEx:
            budget[0] -= 1
            if budget[0] < 0:
                raise _TooLarge
            res = kind(node.func, *[walk(c) for c in node.children])
        elif kind is CastEx:
            res = CastEx(node.dtype, walk(node.children[0]))
        else:
            raise _TooLarge
        memo[id(node)] = res
        return res

    try:
        res = walk(root)
        return res if found[0] else None
    except _TooLarge:
        return None
    finally:
        memo.clear()
        walk = None


_NODES = Memoiser._cache.data
_NODE_GONE = Memoiser._cache._gone
_new_node = object.__new__


def _binary(func, left, right):
    """`BinaryNumpyEx(func, left, right)` for the arithmetic operators, which are most of
    what a step that builds its expression anew spends on the host: the table lookup and
    the constructor's work in one frame."""
    if not isinstance(left, DelayArray):
        left = arg_to_numpy_ex(left)
    if not isinstance(right, DelayArray):
        right = arg_to_numpy_ex(right)
    key = (BinaryNumpyEx, func, id(left), id(right))
    ref = _NODES.get(key)
    if ref is not None:
        node = ref()
        if node is not None:
            return node
    depth = left._depth
    if right._depth > depth:
        depth = right._depth
    if depth >= MAX_DEPTH:
        return BinaryNumpyEx(func, left, right)     # evaluates the deep operand first
    shape = left.shape
    other = right.shape
    if shape != other and other:
        shape = other if not shape else _broadcast2(shape, other)
    node = _new_node(BinaryNumpyEx)
    node.__dict__ = {"_count": DelayArray.count, "children": [left, right], "_depth": depth + 1,
                     "func": func, "shape": shape,
                     "dtype": result_dtype(func, (_descr(left), _descr(right))), "_key": key}
    DelayArray.count += 1
    ref = _NODES[key] = _Ref(node, _NODE_GONE)
    ref.key = key
    return node


def _row_reduce(func, arr, args, kwargs):
    """`arr.sum(axis=-1)`, `arr.max(axis=1, keepdims=True)` ... of a float matrix as the lazy
    node `_reduce` would return, in one frame (a step that builds softmax anew calls this
    twice); None for every other call, which then goes the long way."""
    shape = arr.shape
    ndim = len(shape)
    if ndim < 2 or len(args) > 1 or arr.dtype.kind != "f" or shape[-1] < 2 \
            or not getattr(_backend, "LAZY_ROW_REDUCTIONS", False):
        return None
    axis = args[0] if args else kwargs.get("axis")
    if not isinstance(axis, int) or (axis != -1 and axis != ndim - 1):
        return None
    keep = False
    for name, value in kwargs.items():
        if name == "keepdims" and isinstance(value, bool):
            keep = value
        elif name != "axis":
            return None
    axis = (ndim - 1,)
    key = (ReduceEx, func, id(arr), axis, keep)
    ref = _NODES.get(key)
    if ref is not None:
        node = ref()
        if node is not None:
            return node
    if arr._depth >= MAX_DEPTH:
        return None
    node = _new_node(ReduceEx)
    node.__dict__ = {"_count": DelayArray.count, "children": [arr], "_depth": arr._depth + 1,
                     "func": func, "axis": axis, "keepdims": keep,
                     "shape": shape[:-1] + (1,) if keep else shape[:-1], "dtype": arr.dtype, "_key": key}
    DelayArray.count += 1
    ref = _NODES[key] = _Ref(node, _NODE_GONE)
    ref.key = key
    return node


def _broadcast2(a, b):
    """Broadcast shape of two shapes (NumPy's own routine takes several microseconds)."""
    if len(a) == len(b):
        out = []
        for x, y in zip(a, b):
            if x == y or y == 1:
                out.append(x)
            elif x == 1:
                out.append(y)
            else:
                break
        else:
            return tuple(out)
    return tuple(np.broadcast_shapes(a, b))       # other ranks, or NumPy's error message


def _unary(func, arg):
    """`UnaryFuncEx(func, arg)` in one frame, like `_binary`."""
    key = (UnaryFuncEx, func, id(arg))
    ref = _NODES.get(key)
    if ref is not None:
        node = ref()
        if node is not None:
            return node
    if arg._depth >= MAX_DEPTH:
        return UnaryFuncEx(func, arg)
    node = _new_node(UnaryFuncEx)
    node.__dict__ = {"_count": DelayArray.count, "children": [arg], "_depth": arg._depth + 1,
                     "func": func, "shape": arg.shape,
                     "dtype": result_dtype(func, (_descr(arg),)), "_key": key}
    DelayArray.count += 1
    ref = _NODES[key] = _Ref(node, _NODE_GONE)
    ref.key = key
    return node


# Numbers that expressions were built with lately, kept alive: a loop that builds its
# expression anew every pass then finds its constants instead of making them again (a
# node for a number holds nothing but the number).
_NUMBERS = {}


def _number(val):
    key = (type(val), val if val else repr(val))
    node = _NUMBERS.get(key)
    if node is None:
        if len(_NUMBERS) >= 512:
            _NUMBERS.clear()
        node = _NUMBERS[key] = Scalar(val)
    return node


def arg_to_numpy_ex(arg):
    """Operand -> node (delayarray.py:470-479)."""
    if isinstance(arg, DelayArray):
        return arg
    if type(arg) in _PY_DESCR:
        return _number(arg)
    if isinstance(arg, (numbers.Number, np.generic)):
        return Scalar(arg)
    if _backend.is_ndarray(arg) or isinstance(arg, np.ndarray):
        if arg.ndim == 0 and isinstance(arg, np.ndarray):
            return Scalar(arg[()])
        return NPArray(arg)
    raise NotImplementedError(f"cannot use a {type(arg).__name__} in a lazy expression")


def _reduce(func, arr, axis=None, dtype=None, out=None, keepdims=False, **other):
    """Full reduction -> 0-d backend array (what the reference's `sum` returns
    on its GPU backend, delayarray.py:516-518); a reduction over some axes -> a new leaf;
    a reduction along the last axis that keeps it (`keepdims=True`) stays lazy: inside a
    larger expression (`a - a.max(axis=-1, keepdims=True)`) the backend reduces each row and
    uses it again in one kernel."""
    arr = arg_to_numpy_ex(arr)
    if out is not None or dtype is not None:
        raise NotImplementedError("reductions with out= or dtype= are not supported")
    if not other and isinstance(axis, int) and isinstance(keepdims, bool):
        node = _row_reduce(func, arr, (axis,), {"keepdims": keepdims})      # the common case, in one frame
        if node is not None:
            return node
    for name, value in other.items():
        # `where=` and `initial=` change the result: say so instead of leaving them out
        if not (value is None or value is np._NoValue or (name == "where" and value is True)):
            raise NotImplementedError(f"reductions with {name}= are not supported on lazy arrays")
    ndim = arr.ndim
    if axis is not None:
        axes = (axis,) if isinstance(axis, (int, np.integer)) else tuple(axis)
        norm = []
        for a in axes:
            a = int(a)
            if not -ndim <= a < ndim:
                raise np.exceptions.AxisError(a, ndim)
            norm.append(a % ndim)
        if len(set(norm)) != len(norm):
            raise ValueError("duplicate value in 'axis'")
        axis = tuple(sorted(norm))
        if len(axis) == ndim:
            axis = None
    if axis == (ndim - 1,) and arr.dtype.kind == "f" and arr.shape[-1] > 1 \
            and getattr(_backend, "LAZY_ROW_REDUCTIONS", False):
        # with `keepdims` it is an operand of the row kernel as it is; without, it becomes
        # one when a last axis of one is put back (`a.sum(axis=1)[:, None]`,
        # `.reshape(-1, 1)`, `expand_dims(..., -1)`: `_keep_last_axis`), and is evaluated
        # on its own by whatever else reads it
        return ReduceEx(func, arr, axis, bool(keepdims))
    if 0 in arr.shape and func is not np.add and arr.dtype == np.bool_ and \
            (axis is None or 0 in [arr.shape[k] for k in axis]):
        # `any` / `all` of nothing: the identities of `or` and `and`
        shape = () if axis is None else tuple(d for k, d in enumerate(arr.shape) if k not in axis)
        if keepdims:
            shape = tuple(1 if (axis is None or k in axis) else d for k, d in enumerate(arr.shape))
        res = _backend.fallback.full(shape, func is np.minimum, dtype=np.bool_)
        return res if axis is None and not keepdims else NPArray(res)
    res = ReduceEx(func, arr, axis)._force() if axis is not None else ReduceEx(func, arr)._force()
    if keepdims:
        full = tuple(1 if (axis is None or k in axis) else d for k, d in enumerate(arr.shape))
        res = res.reshape(full)
    return res if axis is None and not keepdims else NPArray(res)


def _evaluate(entry, roots, *more):
    """`entry(roots, *more)` of the backend.  An expression is at most MAX_DEPTH operations
    deep, but evaluated operands whose leaves have been written to since are computed
    again as part of whatever reads them, and a chain of such operands (the iterates of a
    loop, each MAX_DEPTH deep, after a write to the array they all started from) can be
    deeper than the interpreter's stack allows.  Then the stale operands are brought up
    to date one by one, deepest first, and the evaluation is tried again."""
    try:
        return entry(roots, *more)
    except RecursionError:
        for root in (roots if isinstance(roots, (list, tuple)) else [roots]):
            _refresh_operands(root)
        return entry(roots, *more)


def _refresh_operands(root):
    """Evaluate again, children before parents and without recursion, every evaluated
    node below `root` whose leaves were written to after it was computed."""
    stack = [(root, False)]
    seen = set()
    while stack:
        node, after = stack.pop()
        if after:
            node._force()       # its operands are up to date: a walk of MAX_DEPTH at most
            continue
        if id(node) in seen:
            continue
        seen.add(id(node))
        d = node.__dict__
        if "array" in d and node is not root:
            deps = d.get("_deps")
            if deps is None or all(buf.version == ver for buf, ver in deps):
                continue        # a leaf, or a result that is up to date
            stack.append((node, True))
        for child in d.get("children", ()):
            if isinstance(child, DelayArray):
                stack.append((child, False))


def evaluate(*arrays):
    """Evaluate several lazy arrays together, in one fused kernel when their
    shapes agree, sharing common sub-expressions.  Returns the same objects."""
    todo = [a for a in arrays if isinstance(a, DelayArray) and "array" not in a.__dict__]
    if todo:
        results = _evaluate(_backend.run_multi, todo)
        for node, res in zip(todo, results):
            node.array = res
            node._depth = 0     # a leaf of whatever is built on it from now on
            if _COUNTS_WRITES and node.children:
                node._epoch = _WRITES[0]
    return arrays


def synchronize():
    """Wait until the device has finished everything queued so far."""
    _backend.synchronize()


HANDLED_FUNCTIONS = {}


def implements(np_function):
    """Register an `__array_function__` implementation (delayarray.py:485-490)."""

    def decorator(func):
        HANDLED_FUNCTIONS[np_function] = func
        return func

    return decorator


def _eager(name):
    def call(arr, *args, **kwargs):
        return getattr(_backend.fallback, name)(_unwrap(arr), *args, **kwargs)

    call.__name__ = name
    return call


@implements(np.sum)
def sum(arr, axis=None, **kwargs):
    return _reduce(np.add, arr, axis=axis, **kwargs)


@implements(np.max)
def max(arr, axis=None, **kwargs):
    return _reduce(np.maximum, arr, axis=axis, **kwargs)


@implements(np.min)
def min(arr, axis=None, **kwargs):
    return _reduce(np.minimum, arr, axis=axis, **kwargs)


@implements(np.where)
def where(cond, x=None, y=None):
    if x is None or y is None:
        raise NotImplementedError("where(cond) without values (nonzero) is not supported")
    return WhereEx(np.where, *(arg_to_numpy_ex(a) for a in (cond, x, y)))


@implements(np.clip)
def clip(arr, a_min=None, a_max=None, **kwargs):
    out = arg_to_numpy_ex(arr)
    if a_min is not None:
        out = np.maximum(out, a_min)
    if a_max is not None:
        out = np.minimum(out, a_max)
    return out


@implements(np.mean)
def mean(arr, axis=None, keepdims=False, **kwargs):
    arr = arg_to_numpy_ex(arr)
    if kwargs:
        return _backend.fallback.mean(arr._force(), axis=axis, keepdims=keepdims, **kwargs)
    total = _reduce(np.add, arr, axis=axis, keepdims=keepdims)
    total = total if isinstance(total, DelayArray) else NPArray(total)
    count = arr.size // total.size if total.size else 0
    if arr.dtype.kind in "iub":
        total = total.astype(np.float64)
    return total / count


@implements(np.average)
def average(arr, axis=None, weights=None, **kwargs):
    if weights is None:
        return mean(arr, axis=axis, **kwargs)
    return _backend.fallback.average(_unwrap(arr), axis=axis, weights=_unwrap(weights), **kwargs)


@implements(np.var)
def var(arr, axis=None, ddof=0, keepdims=False, **kwargs):
    """Two-pass variance: mean, then the fused mean of squared deviations."""
    arr = arg_to_numpy_ex(arr)
    if kwargs:
        return _backend.fallback.var(arr._force(), axis=axis, ddof=ddof, keepdims=keepdims,
                                     **kwargs)
    centre = mean(arr, axis=axis, keepdims=True)
    dev = arr - centre
    total = _reduce(np.add, dev * dev, axis=axis, keepdims=keepdims)
    total = total if isinstance(total, DelayArray) else NPArray(total)
    count = arr.size // total.size if total.size else 0
    return total / (count - ddof)


_eager_transpose = cast(_eager("transpose"))
_eager_roll = cast(_eager("roll"))


@implements(np.std)
def std(arr, axis=None, ddof=0, keepdims=False, **kwargs):
    return np.sqrt(var(arr, axis=axis, ddof=ddof, keepdims=keepdims, **kwargs))


def _truth(arr):
    arr = arg_to_numpy_ex(arr)
    return arr if arr.dtype == np.bool_ else np.not_equal(arr, 0)


@implements(np.any)
def any_(arr, axis=None, keepdims=False, **kwargs):
    """True where some element along `axis` is non-zero: the fused maximum of a mask."""
    return _reduce(np.maximum, _truth(arr), axis=axis, keepdims=keepdims, **kwargs)


@implements(np.all)
def all_(arr, axis=None, keepdims=False, **kwargs):
    return _reduce(np.minimum, _truth(arr), axis=axis, keepdims=keepdims, **kwargs)


@implements(np.count_nonzero)
def count_nonzero(arr, axis=None, keepdims=False):
    return _reduce(np.add, _truth(arr), axis=axis, keepdims=keepdims)


@implements(np.isclose)
def isclose(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """`numpy.isclose`, one fused mask: |a - b| <= atol + rtol |b| where b is finite, or a == b
    (equal infinities), or both NaN when asked for."""
    a, b = arg_to_numpy_ex(a), arg_to_numpy_ex(b)
    near = np.less_equal(np.absolute(a - b), atol + rtol * np.absolute(b))
    close = (near & np.isfinite(b)) | np.equal(a, b)
    if equal_nan:
        close = close | (np.isnan(a) & np.isnan(b))
    return close


@implements(np.allclose)
def allclose(a, b, rtol=1e-05, atol=1e-08, equal_nan=False):
    """`numpy.allclose`: the mask of `isclose` fused with its reduction; a Python bool."""
    return bool(all_(isclose(a, b, rtol=rtol, atol=atol, equal_nan=equal_nan)))


@implements(np.linalg.norm)
def norm(x, ord=None, axis=None, keepdims=False):           # noqa: A002
    """`numpy.linalg.norm` for the 2-norm of vectors and the Frobenius norm (the defaults):
    the square root of a fused sum of squares."""
    x = arg_to_numpy_ex(x)
    flat = axis is None or isinstance(axis, (int, np.integer)) or len(axis) == 1
    if not (ord is None or (ord == 2 and flat and (axis is not None or x.ndim == 1))
            or (ord == "fro" and (x.ndim == 2 or (axis is not None and not flat)))):
        raise NotImplementedError(f"norm(ord={ord!r}, axis={axis!r}) is not supported on lazy arrays")
    if x.dtype.kind in "iub":
        x = x.astype(np.float64)
    total = _reduce(np.add, x * x, axis=axis, keepdims=keepdims)
    total = total if isinstance(total, DelayArray) else NPArray(total)
    return np.sqrt(total)


# ---- views and compositions NumPy code reaches for (none is registered by the reference;
#      each is indexing, arithmetic or a fused write that the backend already has) -----------

def _axis(axis, ndim):
    axis = int(axis)
    if not -ndim <= axis < ndim:
        raise np.exceptions.AxisError(axis, ndim)
    return axis % ndim


@implements(np.flip)
def flip(m, axis=None):
    """Reversed along `axis` (all axes when None): a view with negative strides, read as
    reversed vectors by the tiled kernel."""
    m = arg_to_numpy_ex(m)
    axes = range(m.ndim) if axis is None else \
        [_axis(a, m.ndim) for a in ((axis,) if isinstance(axis, (int, np.integer)) else axis)]
    key = [slice(None)] * m.ndim
    for a in axes:
        key[a] = slice(None, None, -1)
    return m[tuple(key)]


@implements(np.flipud)
def flipud(m):
    return flip(m, 0)


@implements(np.fliplr)
def fliplr(m):
    if arg_to_numpy_ex(m).ndim < 2:
        raise ValueError("Input must be >= 2-d.")
    return flip(m, 1)


@implements(np.diff)
def diff(a, n=1, axis=-1, **kwargs):
    """n-th difference along `axis`: shifted views of one expression, one stencil kernel."""
    if kwargs:
        raise NotImplementedError(f"diff keyword(s) {sorted(kwargs)} are not supported on lazy arrays")
    a = arg_to_numpy_ex(a)
    axis = _axis(axis, a.ndim)
    hi, lo = [slice(None)] * a.ndim, [slice(None)] * a.ndim
    hi[axis], lo[axis] = slice(1, None), slice(None, -1)
    for _ in range(int(n)):
        a = a[tuple(hi)] ^ a[tuple(lo)] if a.dtype == np.bool_ else a[tuple(hi)] - a[tuple(lo)]
    return a


@implements(np.outer)
def outer(a, b):
    a, b = arg_to_numpy_ex(a), arg_to_numpy_ex(b)
    return a.reshape(a.size, 1) * b.reshape(1, b.size)


@implements(np.ptp)
def ptp(a, axis=None, keepdims=False):
    return max(a, axis=axis, keepdims=keepdims) - min(a, axis=axis, keepdims=keepdims)


@implements(np.expand_dims)
def expand_dims(a, axis):
    a = arg_to_numpy_ex(a)
    axes = (axis,) if isinstance(axis, (int, np.integer)) else tuple(axis)
    ndim = a.ndim + len(axes)
    axes = sorted(_axis(x, ndim) for x in axes)
    key = [slice(None)] * ndim
    for x in axes:
        key[x] = None
    return a[tuple(key)]


@implements(np.squeeze)
def squeeze(a, axis=None):
    a = arg_to_numpy_ex(a)
    if axis is None:
        drop = [k for k, d in enumerate(a.shape) if d == 1]
    else:
        drop = [_axis(x, a.ndim) for x in ((axis,) if isinstance(axis, (int, np.integer)) else axis)]
        if builtins.any(a.shape[k] != 1 for k in drop):
            raise ValueError("cannot select an axis to squeeze out which has size not equal to one")
    return a[tuple(0 if k in drop else slice(None) for k in range(a.ndim))]


@implements(np.swapaxes)
def swapaxes(a, axis1, axis2):
    a = arg_to_numpy_ex(a)
    order = list(range(a.ndim))
    i, j = _axis(axis1, a.ndim), _axis(axis2, a.ndim)
    order[i], order[j] = order[j], order[i]
    return transpose(a, order)


@implements(np.moveaxis)
def moveaxis(a, source, destination):
    a = arg_to_numpy_ex(a)
    src = [_axis(x, a.ndim) for x in ((source,) if isinstance(source, (int, np.integer)) else source)]
    dst = [_axis(x, a.ndim) for x in ((destination,) if isinstance(destination, (int, np.integer))
                                      else destination)]
    if len(src) != len(dst):
        raise ValueError("`source` and `destination` arguments must have the same number of elements")
    order = [k for k in range(a.ndim) if k not in src]
    for d, sx in sorted(zip(dst, src)):
        order.insert(d, sx)
    return transpose(a, order)


@implements(np.reshape)
def reshape(a, *args, **kwargs):
    return arg_to_numpy_ex(a).reshape(*args, **kwargs)


@implements(np.ravel)
def ravel(a):
    return arg_to_numpy_ex(a).ravel()


@implements(np.concatenate)
def concatenate(arrays, axis=0, **kwargs):
    """Every part is written straight into its slice of the result by its own fused kernel:
    lazy parts are never materialised on their own."""
    if kwargs:
        raise NotImplementedError(f"concatenate keyword(s) {sorted(kwargs)} are not supported on lazy arrays")
    parts = [arg_to_numpy_ex(a) for a in arrays]
    if not parts:
        raise ValueError("need at least one array to concatenate")
    if axis is None:
        parts, axis = [p.ravel() for p in parts], 0
    ndim = parts[0].ndim
    if ndim == 0:
        raise ValueError("zero-dimensional arrays cannot be concatenated")
    axis = _axis(axis, ndim)
    for p in parts:
        if p.ndim != ndim or builtins.any(p.shape[k] != parts[0].shape[k] for k in range(ndim) if k != axis):
            raise ValueError("all the input array dimensions except for the concatenation axis must match exactly")
    shape = list(parts[0].shape)
    shape[axis] = builtins.sum(p.shape[axis] for p in parts)
    dtype = np.result_type(*[p.dtype for p in parts])
    out = NPArray(_backend.fallback.empty(tuple(shape), dtype=dtype))
    at = 0
    for p in parts:
        key = [slice(None)] * ndim
        key[axis] = slice(at, at + p.shape[axis])
        if p.shape[axis]:
            out[tuple(key)] = p
        at += p.shape[axis]
    return out


_COLUMN_NUMBERS = {}        # (count, integer type) -> the leaf 0, 1, ... count - 1 that `stack` compares with


@implements(np.stack)
def stack(arrays, axis=0, **kwargs):
    parts = [arg_to_numpy_ex(a) for a in arrays]
    if not parts:
        raise ValueError("need at least one array to stack")
    if builtins.any(p.shape != parts[0].shape for p in parts):
        raise ValueError("all input arrays must have the same shape")
    axis = _axis(axis, parts[0].ndim + 1)
    if (axis == parts[0].ndim >= 1 and 2 <= len(parts) <= 8 and not kwargs
            and builtins.all(p.dtype.kind in "fiu" and p.dtype.itemsize in (4, 8) for p in parts)):
        # A few vectors side by side as the columns of a matrix (coordinates into points):
        # one expression, `where(column == 0, a, where(column == 1, b, c))`, that a single
        # kernel writes row by row (and that fuses with what reads it), instead of one
        # strided write per column.
        dtype = np.result_type(*[p.dtype for p in parts])
        kind = (len(parts), np.int32 if dtype.itemsize == 4 else np.int64)
        column = _COLUMN_NUMBERS.get(kind)
        if column is None:          # uploaded once: the same leaf every time, so plans are found again
            column = _COLUMN_NUMBERS[kind] = array(np.arange(kind[0], dtype=kind[1]))
        cols = [expand_dims(p if p.dtype == dtype else p.astype(dtype), axis) for p in parts]
        out = cols[-1]
        for k in range(len(parts) - 2, -1, -1):
            out = where(column == k, cols[k], out)
        return out
    return concatenate([expand_dims(p, axis) for p in parts], axis=axis, **kwargs)


@implements(np.vstack)
def vstack(tup):
    parts = [arg_to_numpy_ex(a) for a in tup]
    return concatenate([p.reshape(1, -1) if p.ndim < 2 else p for p in parts], axis=0)


@implements(np.hstack)
def hstack(tup):
    parts = [arg_to_numpy_ex(a) for a in tup]
    return concatenate(parts, axis=0 if parts and parts[0].ndim == 1 else 1)


@implements(np.broadcast_to)
def broadcast_to(a, shape, **kwargs):
    """Stretched view (no copy) of the evaluated array, as a leaf."""
    return NPArray(_backend.fallback.broadcast_to(arg_to_numpy_ex(a)._force(), _shape_of(shape)))


@implements(np.trace)
def trace(a, offset=0, axis1=0, axis2=1, **kwargs):
    a = arg_to_numpy_ex(a)
    if a.ndim != 2 or (axis1, axis2) != (0, 1) or kwargs:
        raise NotImplementedError("trace is supported for matrices (axis1=0, axis2=1) only")
    return _reduce(np.add, diag(a, offset))


@implements(np.inner)
def inner(a, b):
    a, b = arg_to_numpy_ex(a), arg_to_numpy_ex(b)
    if a.ndim != 1 or b.ndim != 1:
        raise NotImplementedError("inner is supported for vectors only")
    return a._dot([a, b], {})


@implements(np.vdot)
def vdot(a, b):
    a, b = arg_to_numpy_ex(a), arg_to_numpy_ex(b)
    return inner(a.ravel(), b.ravel())


@implements(np.transpose)
def transpose(arr, axes=None):
    """View of the evaluated array with permuted axes (delayarray.py:521-524); a small
    unevaluated element-wise expression is rebuilt over permuted views of its leaves."""
    if isinstance(arr, DelayArray) and "array" not in arr.__dict__ and type(arr) in _ELEMENTWISE:
        res = _over_views(arr, lambda a: a.transpose(axes) if axes is not None else a.transpose())
        if res is not None:
            return res
    return _eager_transpose(arr, axes) if axes is not None else _eager_transpose(arr)


@implements(np.roll)
def roll(arr, shift, axis=None):
    """`numpy.roll` (delayarray.py:527-530).  Along one axis of an unevaluated
    element-wise expression the two pieces are computed straight into their shifted
    places: two fused kernels, no unshifted temporary."""
    lazy = isinstance(arr, DelayArray) and "array" not in arr.__dict__ \
        and type(arr) in _ELEMENTWISE and isinstance(shift, (int, np.integer)) \
        and (isinstance(axis, (int, np.integer)) or (axis is None and arr.ndim == 1)) and arr.size
    if not lazy:
        return _eager_roll(arr, shift, axis)
    axis = 0 if axis is None else int(axis)
    if not -arr.ndim <= axis < arr.ndim:
        raise np.exceptions.AxisError(axis, arr.ndim)
    axis %= arr.ndim
    n = arr.shape[axis]
    shift = int(shift) % n
    out = empty(arr.shape, dtype=arr.dtype)

    def cut(lo, hi):
        return tuple(slice(lo, hi) if k == axis else slice(None) for k in range(arr.ndim))
    if shift == 0:
        out[...] = arr
    else:
        head, tail = arr[cut(0, n - shift)], arr[cut(n - shift, n)]
        if isinstance(head, NPArray):       # too large to rebuild: evaluated once, copied twice
            return _eager_roll(arr, shift, axis)
        out[cut(shift, n)] = head
        out[cut(0, shift)] = tail
    return out
repeat = implements(np.repeat)(cast(_eager("repeat")))
cumsum = implements(np.cumsum)(cast(_eager("cumsum")))
tile = implements(np.tile)(cast(_eager("tile")))
diagflat = implements(np.diagflat)(cast(_eager("diagflat")))
diag = implements(np.diag)(cast(_eager("diag")))


# ufuncs re-exported under their NumPy names (delayarray.py:571-587)
add = np.add
multiply = np.multiply
subtract = np.subtract
divide = np.divide
true_divide = np.true_divide
dot = np.dot
cos = np.cos
sin = np.sin
tan = np.tan
tanh = np.tanh
sinh = np.sinh
cosh = np.cosh
arcsin = np.arcsin
arccos = np.arccos
arctan = np.arctan
arctan2 = np.arctan2
exp = np.exp
exp2 = np.exp2
expm1 = np.expm1
log = np.log
log2 = np.log2
log10 = np.log10
log1p = np.log1p
power = np.power
sqrt = np.sqrt
cbrt = np.cbrt
square = np.square
abs = np.abs
absolute = np.absolute
negative = np.negative
maximum = np.maximum
minimum = np.minimum
greater = np.greater
less = np.less
floor = np.floor
ceil = np.ceil
hypot = np.hypot
sign = np.sign
isnan = np.isnan
isinf = np.isinf
isfinite = np.isfinite
logical_and = np.logical_and
logical_or = np.logical_or
logical_not = np.logical_not
newaxis = None

try:  # `erf` is a SciPy ufunc; the name is what the code generator keys on
    from scipy.special import erf, erfc  # noqa: F401
except ImportError:  # pragma: no cover
    pass

# dtypes
double = np.double
float64 = np.float64
float32 = np.float32
int32 = np.int32
int64 = np.int64
uint32 = np.uint32

# creation routines: evaluated by the backend, wrapped as leaves
# (delayarray.py:596-604, 620-625, 634-636, 641-643)
for _name in ("empty", "empty_like", "eye", "identity", "ones", "ones_like", "zeros",
              "zeros_like", "full", "full_like", "array", "asarray", "asanyarray",
              "ascontiguousarray", "copy", "arange", "linspace", "logspace", "tri", "tril",
              "triu", "asmatrix", "frombuffer", "fromfile", "fromfunction", "fromiter",
              "fromstring", "loadtxt", "geomspace", "vander"):
    _fn = getattr(_backend.fallback, _name, None)
    if _fn is not None:
        globals()[_name] = cast(_fn)
del _name, _fn

Shape = tuple          # (rows, columns), as annotated in delayarray.py:159


def is_matrix_matrix(left, right):
    """Shapes of a matrix-matrix product (delayarray.py:454-455)."""
    return len(left) > 1 and len(right) > 1


def is_matrix_vector(left, right):
    """Shapes of a matrix-vector product (delayarray.py:458-459)."""
    return len(left) > 1 and len(right) == 1


def _triangle(lower):
    def tri_part(m, k=0):
        """`numpy.tril` / `numpy.triu` (delayarray.py:642-643) as a lazy `where` over the
        row and column indices: fused with whatever produces `m`, no mask array."""
        m = arg_to_numpy_ex(m)
        if m.ndim < 2:
            raise ValueError("tril/triu need an array of at least two dimensions")
        rows, cols = m.shape[-2:]
        r = NPArray(_backend.fallback.asarray(np.arange(rows).reshape(rows, 1)))
        c = NPArray(_backend.fallback.asarray(np.arange(cols)))
        keep = (c - r <= int(k)) if lower else (c - r >= int(k))
        return where(keep, m, m.dtype.type(0))
    tri_part.__name__ = "tril" if lower else "triu"
    return tri_part


tril = _triangle(True)
triu = _triangle(False)
if "asmatrix" not in globals():
    def asmatrix(data, dtype=None):
        """2-d view of the data as a leaf (delayarray.py:624 wraps `numpy.asmatrix`; the
        matrix subclass itself has no device counterpart)."""
        arr = arg_to_numpy_ex(data if dtype is None else np.asarray(_unwrap_host(data), dtype=dtype))
        return arr if arr.ndim == 2 else arr.reshape((1, -1) if arr.ndim < 2 else arr.shape)


def _unwrap_host(obj):
    return obj.get() if isinstance(obj, DelayArray) else obj


# Generated leaves: constant and index-valued arrays stay lazy when the backend can
# compute them inside a kernel.  Arrays shorter than this are made at once, as before.
GENERATE_FROM = 4096
_eager_create = {k: globals()[k] for k in ("zeros", "ones", "full", "zeros_like", "ones_like",
                                           "full_like", "arange", "linspace") if k in globals()}
_GENERATES = bool(getattr(_backend, "GENERATED_LEAVES", False))


def _shape_of(shape):
    if isinstance(shape, (int, np.integer)):
        return (int(shape),)
    return tuple(int(d) for d in shape)


def _lazy_full(shape, val, dtype):
    """FullEx when that is worth it and the value fits the dtype; else None."""
    if not _GENERATES:
        return None
    try:
        shape = _shape_of(shape)
        dtype = np.dtype(dtype)
    except TypeError:
        return None
    size = 1
    for d in shape:
        size *= d
    if size < GENERATE_FROM or dtype.kind not in "fiub" or dtype.itemsize > 8 \
            or dtype == np.float16 or not isinstance(val, (numbers.Real, np.bool_)):
        return None
    return FullEx(shape, val, dtype)


def zeros(shape, dtype=float, **kwargs):
    node = None if kwargs.get("like") is not None else _lazy_full(shape, 0, dtype)
    return node if node is not None else _eager_create["zeros"](shape, dtype=dtype, **kwargs)


def ones(shape, dtype=float, **kwargs):
    node = None if kwargs.get("like") is not None else _lazy_full(shape, 1, dtype)
    return node if node is not None else _eager_create["ones"](shape, dtype=dtype, **kwargs)


def full(shape, fill_value, dtype=None, **kwargs):
    node = None
    if kwargs.get("like") is None and isinstance(fill_value, (numbers.Real, np.bool_)):
        node = _lazy_full(shape, fill_value, np.asarray(fill_value).dtype if dtype is None else dtype)
    return node if node is not None else _eager_create["full"](shape, fill_value, dtype=dtype, **kwargs)


def _like(name, val):
    def create(a, *args, dtype=None, shape=None, **kwargs):
        if name == "full_like":
            (fill,), args = args[:1], args[1:]
        else:
            fill = val
        if not args and hasattr(a, "shape") and hasattr(a, "dtype"):
            node = _lazy_full(a.shape if shape is None else shape, fill,
                              a.dtype if dtype is None else dtype)
            if node is not None:
                return node
        extra = (fill,) if name == "full_like" else ()
        return _eager_create[name](_unwrap(a), *extra, *args, dtype=dtype, shape=shape, **kwargs)

    create.__name__ = name
    return create


zeros_like = _like("zeros_like", 0)
ones_like = _like("ones_like", 1)
full_like = _like("full_like", None)


def arange(*args, **kwargs):
    """NumPy's `arange`; long ranges of Python numbers stay lazy.  NumPy fills element
    0 with `start`, element 1 with `start + step` (both computed in Python and then
    converted), and element i >= 2 with `start + i*delta` in the array's own type,
    where `delta` is the difference of the first two; so does this."""
    lazy = _GENERATES and 1 <= len(args) <= 3 and set(kwargs) <= {"dtype"} \
        and all(type(a) in (int, float) for a in args)
    if lazy:
        start, stop, step = (0, args[0], 1) if len(args) == 1 else (tuple(args) + (1,))[:3]
        dtype = kwargs.get("dtype")
        dtype = np.dtype(dtype) if dtype is not None else np.result_type(*args)
        lazy = step != 0 and dtype in (np.float32, np.float64, np.int32, np.int64) \
            and all(np.isfinite(a) for a in (start, stop, step))
    if lazy:
        n = math.ceil((stop - start) / step)
        lazy = n >= GENERATE_FROM
    if lazy and dtype.kind == "i":
        info = np.iinfo(dtype)
        lazy = all(type(a) is int for a in (start, stop, step)) \
            and all(info.min <= v <= info.max for v in (start, start + (n - 1) * step))
    if not lazy:
        return _eager_create["arange"](*args, **kwargs)
    first, second = dtype.type(start), dtype.type(start + step)
    idx = IotaEx(n, dtype)
    if dtype.kind == "i":
        return first + idx * dtype.type(step)
    with np.errstate(all="ignore"):
        delta = dtype.type(second - first)
    return where(idx == dtype.type(1), second, first + idx * delta)


def linspace(start, stop, num=50, endpoint=True, retstep=False, dtype=None, axis=0, **kwargs):
    """NumPy's `linspace`; long ones between Python numbers stay lazy: element i is
    `i*step + start` in float64 with `step = (stop - start)/div`, the last one is
    `stop` itself, then everything is converted to `dtype`."""
    lazy = _GENERATES and not retstep and axis == 0 and not kwargs \
        and type(start) in (int, float) and type(stop) in (int, float) \
        and isinstance(num, (int, np.integer)) and num >= GENERATE_FROM \
        and np.isfinite(start) and np.isfinite(stop) \
        and (dtype is None or np.dtype(dtype) in (np.float32, np.float64))
    if lazy:
        div = num - 1 if endpoint else num
        delta = np.float64(stop) - np.float64(start)
        step = delta / div
        lazy = step != 0 and np.isfinite(step)
    if not lazy:
        return _eager_create["linspace"](start, stop, num=num, endpoint=endpoint, retstep=retstep,
                                         dtype=dtype, axis=axis, **kwargs)
    idx = IotaEx(num, np.float64)
    y = idx * step + np.float64(start)
    if endpoint:
        y = where(idx == np.float64(num - 1), np.float64(stop), y)
    if dtype is not None and np.dtype(dtype) != np.float64:
        y = y.astype(dtype)
    return y
