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
LAZY_ROW_REDUCTIONS = True  # reductions that keep their axis may stay lazy nodes


COUNTS_WRITES = True    # ndarrays have no version: the front end counts the writes instead


def is_ndarray(arr):
    return isinstance(arr, numpy.ndarray)


class CpuVisitor(Visitor):
    def visit_NPArray(self, node):
        return node.array

    def visit_Scalar(self, node):
        return node.val

    def _apply(self, node):
        if node.__dict__.get("_cut"):
            # where the front end evaluated an operand of a very deep expression the walk
            # ends (every other evaluated node is computed again, as in the reference)
            return node.array
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

    def visit_RandEx(self, node):
        arr = node.__dict__.get("array")
        if arr is not None:
            return arr
        # numpy.random.Philox steps its counter before it makes a block, so the block
        # that holds output `pos` is made from `counter + pos // 4`, entered one lower
        if node.dtype == numpy.float32:     # two numbers per output, its low half first
            start = (node.counter - 1) % (1 << 256)
            bits = numpy.random.Philox(key=node.key, counter=start)
            raw = bits.random_raw((node.pos + node.shape[0] + 1) // 2)
            halves = numpy.stack([raw & numpy.uint64(0xffffffff), raw >> numpy.uint64(32)], axis=1).ravel()
            halves = halves[node.pos:node.pos + node.shape[0]].astype(numpy.uint32)
            return (halves >> numpy.uint32(8)).astype(numpy.float32) * numpy.float32(1.0 / 16777216.0)
        first, skip = divmod(node.pos, 4)
        start = (node.counter + first - 1) % (1 << 256)
        bits = numpy.random.Philox(key=node.key, counter=start)
        raw = bits.random_raw(skip + node.shape[0])[skip:]
        if node.dtype == numpy.int64:
            return raw.view(numpy.int64)
        return (raw >> numpy.uint64(11)) * (1.0 / 9007199254740992.0)

    def visit_CastEx(self, node):
        return self.visit(node.children[0]).astype(node.dtype)

    def visit_ReduceEx(self, node):
        if node.__dict__.get("_cut"):
            return node.array
        return node.func.reduce(self.visit(node.children[0]), axis=node.axis,
                                keepdims=getattr(node, "keepdims", False))


def run(ex):
    return CpuVisitor().visit(ex)


def run_multi(exs):
    visitor = CpuVisitor()
    return [visitor.visit(ex) for ex in exs]


def run_into(ex, dst_view):
    dst_view[...] = run(ex)


def synchronize():
    pass
