"""A second, minimal front end that follows the *reference's* node conventions, to
prove that the HIP backend binds to any front end speaking the backend protocol
and not only to this repository's own classes.

Conventions restated from the reference (read, not imported):
  * a backend tells nodes apart by class name (delayrepay/visitor.py:18-21), so the
    classes here are named BinaryNumpyEx, UnaryFuncEx, BinaryFuncEx, NPArray, Scalar
    (delayrepay/delayarray.py:286-313,339-351,383-417,434-452) but are unrelated
    to delayrepay_amd's classes of the same names;
  * a node has `children`, interior nodes `func` (the NumPy ufunc), leaves `array`,
    scalars `val`; every node has `name` made from a global serial (:29-32,150-152);
  * a Scalar's shape is the sentinel `(0,)` and its dtype starts as None (:434-441);
  * a binary node takes the first non-None dtype of its children and writes it onto
    the other child (:462-467); shape is the non-scalar side (:197-213);
  * `x ** k` with an int k is a chain of multiplies, `square(x)` is `x*x` (:316-336);
  * evaluation stores the backend's result on the node as `array` (:38-44).
No hash-consing and no NumPy protocol hooks: the tests build nodes directly.
"""
import numpy as np

_serial = [0]


class Node:
    def __init__(self, children=()):
        self._count = _serial[0]
        _serial[0] += 1
        self.children = list(children)
        self.dtype = None

    def evaluate(self, backend):
        if "array" not in self.__dict__:
            self.array = backend.run(self)
        return self.array

    # arithmetic sugar for the tests
    def __add__(self, other):
        return BinaryNumpyEx(np.add, self, wrap(other))

    def __radd__(self, other):
        return BinaryNumpyEx(np.add, wrap(other), self)

    def __sub__(self, other):
        return BinaryNumpyEx(np.subtract, self, wrap(other))

    def __rsub__(self, other):
        return BinaryNumpyEx(np.subtract, wrap(other), self)

    def __mul__(self, other):
        return BinaryNumpyEx(np.multiply, self, wrap(other))

    def __rmul__(self, other):
        return BinaryNumpyEx(np.multiply, wrap(other), self)

    def __truediv__(self, other):
        return BinaryNumpyEx(np.true_divide, self, wrap(other))

    def __rtruediv__(self, other):
        return BinaryNumpyEx(np.true_divide, wrap(other), self)

    def __pow__(self, k):
        if isinstance(k, int):
            out = self
            for _ in range(k - 1):
                out = BinaryNumpyEx(np.multiply, out, self)
            return out
        return BinaryFuncEx(np.power, self, wrap(k))


def _shape(left, right):
    return right if left == (0,) else left


def _dtype(a, b):
    if a.dtype is not None:
        b.dtype = a.dtype
        return a.dtype
    a.dtype = b.dtype
    return b.dtype


class BinaryNumpyEx(Node):
    def __init__(self, func, left, right):
        super().__init__([left, right])
        self.func = func
        self.shape = _shape(left.shape, right.shape)
        self.dtype = _dtype(left, right)

    @property
    def name(self):
        return f"binex{self._count}"


class BinaryFuncEx(BinaryNumpyEx):
    @property
    def name(self):
        return f"binfun{self._count}"


class UnaryFuncEx(Node):
    def __init__(self, func, arg):
        super().__init__([arg])
        self.func = func
        self.shape = arg.shape
        self.dtype = arg.dtype

    @property
    def name(self):
        return f"unfunc{self._count}"


class NPArray(Node):
    def __init__(self, array):
        super().__init__()
        self.array = array
        self.shape = array.shape
        self.dtype = array.dtype

    @property
    def name(self):
        return f"arr{self._count}"


class Scalar(Node):
    def __init__(self, val):
        super().__init__()
        self.val = val
        self.shape = (0,)

    @property
    def name(self):
        return str(self.val)


def wrap(x):
    return x if isinstance(x, Node) else Scalar(x)


def unary(func, x):
    return UnaryFuncEx(func, x)
