"""`DELAY_CPU` backend: node-by-node NumPy evaluation on the host.

Mirrors the reference's CPU backend (delayrepay/cpu.py:12-31): every interior
node applies its stored NumPy ufunc to its evaluated children, leaves hand back
their array or Python scalar.  It is selected only by the `DELAY_CPU`
environment variable and is never used by the HIP backend.
"""
import numpy

from .visitor import Visitor

np = numpy
fallback = numpy
GENERATED_LEAVES = True     # FullEx / IotaEx nodes are understood


def is_ndarray(arr):
    return isinstance(arr, numpy.ndarray)


class CpuVisitor(Visitor):
    def visit_NPArray(self, node):
        return node.array

    def visit_Scalar(self, node):
        return node.val

    def _apply(self, node):
        return node.func(*[self.visit(child) for child in node.children])

    visit_UnaryFuncEx = _apply
    visit_BinaryFuncEx = _apply
    visit_BinaryNumpyEx = _apply
    visit_WhereEx = _apply

    def visit_FullEx(self, node):
        arr = node.__dict__.get("array")      # once forced it is an ordinary array
        return arr if arr is not None else numpy.full(node.shape, node.val, dtype=node.dtype)

    def visit_IotaEx(self, node):
        arr = node.__dict__.get("array")
        return arr if arr is not None else numpy.arange(node.shape[0]).astype(node.dtype)

    def visit_CastEx(self, node):
        return self.visit(node.children[0]).astype(node.dtype)

    def visit_ReduceEx(self, node):
        return node.func.reduce(self.visit(node.children[0]), axis=node.axis)


def run(ex):
    return CpuVisitor().visit(ex)


def run_multi(exs):
    visitor = CpuVisitor()
    return [visitor.visit(ex) for ex in exs]


def run_into(ex, dst_view):
    dst_view[...] = run(ex)


def synchronize():
    pass
