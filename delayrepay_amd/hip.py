"""HIP fusion backend for MI355X (gfx950): the backend module the lazy front end
binds to when `DELAY_CPU` is not set.

Exports the duck-typed backend protocol of the reference's GPU backend
(delayrepay/cuda.py:21-26,91-96): `np`, `fallback`, `is_ndarray(arr)`,
`run(ex)`; plus `run_multi`, `run_into`, `synchronize` for the front end's
multi-root, fused-assignment and timing entry points.

`run` does what cuda.py:91-96 does with CuPy, without CuPy:
  trace    one memoised walk of the DAG into a straight-line `Program`;
  lower    choose a kernel shape from the operands' layouts, build the cache key
           (structure + dtypes + layout classes + tunables) and, on a miss, emit
           HIP C++ (`codegen`) and compile it with hiprtc through libdrhip
           (in-memory cache, then an on-disk cache of code objects);
  launch   pack the argument block and launch on the library stream; the output
           comes from libdrhip's pooled allocator.
Nothing is computed on the host, and there is no fall-back to NumPy: a missing
library or GPU raises.
"""
import collections
import hashlib
import os
import struct
import warnings

import numpy

from . import codegen as cg
from . import hiprt
from .devarray import Buffer, ndarray, placeholder  # noqa: F401
from .codegen import Program, dtype_code, code_dtype
from .promote import result_dtype, scalar_descr
from .visitor import Visitor
from .lowering import (TUNE, Lowered as _Lowered, broadcast_strides as _broadcast_strides,
                       lower as _lower, block_lanes as _block_lanes,
                       lower_axis_reduce as _lower_axis_reduce)

hiprt.lib()  # fail at import when libdrhip.so has not been built

COMPILE_OPTS = [
    "-O3",
    "-ffp-contract=off",                      # a*b+c stays two roundings, like NumPy
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no v_pk_*_f32
]

_FUSED = "DELAY_UNFUSED" not in os.environ
STATS = {"launches": 0, "compiles": 0, "disk_hits": 0, "mem_hits": 0, "plan_hits": 0,
         "lowering_hits": 0, "seen_hits": 0, "disk_write_failures": 0}

_ROW_OPS = {"add": "rowsum", "maximum": "rowmax", "minimum": "rowmin"}
_COMPARES = ("greater", "less", "greater_equal", "less_equal", "equal", "not_equal") \
    + tuple(cg._PREDICATES)


def set_fused(flag):
    """False: evaluate one kernel per DAG node with materialised temporaries (the
    un-fused baseline the fused kernels are measured against)."""
    global _FUSED, _STAMP
    _FUSED = bool(flag)
    _STAMP += 1


def set_tune(**kwargs):
    """Change tunables at run time (they are part of every cache key)."""
    global _STAMP
    for k, v in kwargs.items():
        if k not in TUNE:
            raise KeyError(k)
        TUNE[k] = int(v)
    _STAMP += 1


LAZY_ROW_REDUCTIONS = True  # a reduction along the last axis that keeps it may stay a lazy node
GENERATED_LEAVES = True     # FullEx / IotaEx nodes are computed inside kernels


def is_ndarray(arr):
    return isinstance(arr, ndarray)


def synchronize():
    hiprt.sync()


# ---------------------------------------------------------------------------
# tracing: DAG -> Program
# ---------------------------------------------------------------------------

def _scalar_value(value, code):
    """Python number to hand to struct.pack for a parameter of dtype `code`."""
    if code == "f8" or code == "f4":
        # native-mode struct packing of 'f' is a C cast: round to nearest, overflow to
        # infinity, which is what numpy.float32(value) gives
        return float(value)
    with numpy.errstate(all="ignore"):
        return code_dtype(code).type(value).item()


_CODES = {}
_M64 = (1 << 64) - 1


def _code_of(dtype):
    try:
        return _CODES[dtype]
    except KeyError:
        return _CODES.setdefault(dtype, dtype_code(dtype))


def _kind(node):
    """Node kind = its class name, the way the reference's backends tell nodes apart
    (delayrepay/visitor.py:18-21): any front end whose node classes carry these names
    and fields can hand its DAG to this backend."""
    return node.__class__.__name__


class Tracer(Visitor):
    """Walks the DAG of one or more roots once (memoised by node identity) and
    collects leaves, typed scalar parameters and SSA operations.

    Dispatch is by class name through `Visitor.visit_<ClassName>`, as in the
    reference's emitter (delayrepay/cuda.py:46-88): `BinaryNumpyEx`, `UnaryFuncEx`,
    `BinaryFuncEx`, `NPArray`, `Scalar`, plus this repository's `WhereEx`, `CastEx`,
    `ReduceEx`, `FullEx`, `IotaEx`.  Only `children`, `func`, `val` and `array` of a node
    are read; every statement's type is derived here with NumPy's promotion rules
    (`promote.result_dtype`) from the leaves' dtypes, so a front end that stores no
    dtype on a scalar, or a sibling's dtype on an interior node
    (delayrepay/delayarray.py:434-452,462-467), gets NumPy's result all the same.
    Each handler returns (operand reference, dtype code)."""

    def __init__(self, evaluated=None, reuse=False, rows=False):
        super().__init__()
        self._reuse = reuse       # evaluate deep operands met in an earlier evaluation first
        self._rows = rows         # reductions along the last axis become operations of the program
        self.row_len = None       # length of the rows those reductions run along
        self.leaves = []
        self.leaf_codes = []
        self._leaf_index = {}
        self.scalars = []
        self.scalar_codes = []
        self._scalar_index = {}
        self.scalar_uses = []     # the slot each use of a number took, in the order of use
        self.ops = []
        self._memo = {}
        self._evaluated = evaluated if evaluated is not None else {}
        self.leaf_nodes = []      # (node, its array, the deps it was computed from or None)
        self.gen_shapes = []      # shapes of generated leaves (they take part in broadcasting)
        self.iotas = []           # index-valued generated leaves

    def leaf(self, arr):
        if not isinstance(arr, ndarray):
            raise TypeError(f"a leaf of the expression holds a {type(arr).__name__}, not a device "
                            "array of this backend")
        code = _code_of(arr.dtype)
        key = (id(arr.buf), arr.offset, arr.shape, arr._strides, code)
        idx = self._leaf_index.get(key)
        if idx is None:
            idx = len(self.leaves)
            self._leaf_index[key] = idx
            self.leaves.append(arr)
            self.leaf_codes.append(code)
        return ("l", idx), code

    def scalar(self, value, code, ident=None):
        """Scalar kernel parameter of dtype `code`; the value is converted at pack
        time (struct packs Python numbers to float/double exactly as NumPy casts
        a weak scalar)."""
        key = (ident if ident is not None else ("v", repr(value)), code)
        idx = self._scalar_index.get(key)
        if idx is None:
            idx = len(self.scalars)
            self._scalar_index[key] = idx
            self.scalars.append(_scalar_value(value, code))
            self.scalar_codes.append(code)
        self.scalar_uses.append(idx)
        return ("s", idx), code

    def op(self, name, compute, result, refs):
        self.ops.append((name, compute, result, tuple(refs)))
        return ("v", len(self.ops) - 1), result

    def visit(self, node):
        memo = self._memo
        nid = id(node)
        hit = memo.get(nid)
        if hit is not None:
            return hit
        arr = self._evaluated.get(nid) if self._evaluated else None
        if arr is None:
            arr = node.__dict__.get("array")
            if arr is not None and _kind(node) != "NPArray":
                deps = node.__dict__.get("_deps")
                if deps is not None and any(buf.version != ver for buf, ver in deps):
                    arr = None  # stale: recompute inside this kernel
                elif node.__dict__.get("_gen", 0) >= MAX_GENERATIONS:
                    # the end of a long chain of results computed from results (`x = f(x)`
                    # in a loop): from here on this one is an array in its own right, and
                    # what it was computed from can be freed (a front end without `_seal`
                    # keeps its chain)
                    seal = getattr(node, "_seal", None)
                    if seal is not None:
                        seal()
        if arr is not None:
            res = self.leaf(arr)
            self.leaf_nodes.append((node, arr, node.__dict__.get("_deps")))
        else:
            res = Visitor.visit(self, node)
        memo[nid] = res
        return res

    def default_visit(self, node):
        raise NotImplementedError(f"{_kind(node)} nodes cannot be evaluated by the HIP backend")

    # -- operands of an interior node ---------------------------------------------

    def _operands(self, children):
        """[(child, reference-or-None, descriptor)]: array-valued children are traced,
        numbers are left for the consumer (a weak scalar takes the consumer's type)."""
        out = []
        reuse = self._reuse
        for child in children:
            if _kind(child) == "Scalar":
                out.append((child, None, scalar_descr(child.val)))
            else:
                if reuse:
                    d = child.__dict__
                    if "array" not in d and getattr(child, "_depth", 0) >= REUSE_DEPTH \
                            and id(child) not in self._memo:
                        seen = d.get("_seen", 0)
                        if seen < REUSE_AFTER:
                            d["_seen"] = seen + 1
                        else:
                            # A deep operand that earlier evaluations already computed
                            # inline (`x = f(x)` carried through a loop that only ever asks
                            # for `sum(g(x))`): computed once on its own now, it is a leaf
                            # here and in everything built on it later.
                            child._force()
                ref, code = self.visit(child)
                out.append((child, ref, ("a", code)))
        return out

    def _call(self, node):
        func = node.func
        name = func.__name__
        operands = self._operands(node.children)
        descrs = tuple(d for _, _, d in operands)
        if name not in cg.SUPPORTED_UFUNCS and name not in _COMPARES:
            raise NotImplementedError(f"ufunc {name!r} cannot be fused by the HIP backend")
        result = dtype_code(result_dtype(func, descrs))
        compute = result
        if name in _COMPARES:     # arithmetic in the operands' common type, bool out
            compute = dtype_code(result_dtype(numpy.add if len(descrs) == 2 else numpy.positive,
                                              descrs))
            if compute == "b1" and name not in cg._PREDICATES:
                compute = "u1"
        refs = [ref if ref is not None else self.scalar(child.val, compute, id(child))[0]
                for child, ref, _ in operands]
        self.ops.append((name, compute, result, tuple(refs)))
        return ("v", len(self.ops) - 1), result

    visit_BinaryNumpyEx = _call
    visit_BinaryFuncEx = _call
    visit_UnaryFuncEx = _call

    def visit_NPArray(self, node):
        res = self.leaf(node.array)
        self.leaf_nodes.append((node, node.array, None))
        return res

    def visit_Scalar(self, node):
        return self.scalar(node.val, dtype_code(numpy.asarray(node.val).dtype), id(node))

    def visit_WhereEx(self, node):
        operands = self._operands(node.children)
        result = dtype_code(result_dtype(numpy.add, (operands[1][2], operands[2][2])))
        refs = []
        for pos, (child, ref, _) in enumerate(operands):
            if ref is None:
                code = result if pos else dtype_code(numpy.asarray(child.val).dtype)
                ref = self.scalar(child.val, code, id(child))[0]
            refs.append(ref)
        return self.op("where", result, result, refs)

    def visit_CastEx(self, node):
        ref, code = self.visit(node.children[0])
        target = dtype_code(node.dtype)
        return self.op("cast", target, target, [ref]) if code != target else (ref, code)

    def visit_ReduceEx(self, node):
        """A reduction inside a larger expression.  Along the last axis, kept (`keepdims`),
        of a float expression: an operation of the program (`rowsum`, `rowmax`, `rowmin`;
        the row kernel reduces each row and uses it again, cf. the reference's `ReduceEx`
        as an interior node, delayarray.py:272-283, cuda.py:87-88).  Anything else is
        evaluated on its own first and read as a leaf."""
        child = node.children[0]
        name = _ROW_OPS.get(node.func.__name__)
        if self._rows and name and getattr(node, "keepdims", False) \
                and node.axis == (len(child.shape) - 1,) and child.shape[-1] > 1 \
                and (self.row_len is None or self.row_len == child.shape[-1]):
            ref, code = self.visit(child)
            if code in ("f4", "f8") and ref[0] != "s":
                self.row_len = child.shape[-1]
                return self.op(name, code, code, [ref])
            raise cg.RowFusionUnsupported("a reduction of integers or of a constant")
        res = self.leaf(node._force())
        self.leaf_nodes.append((node, node.array, node.__dict__.get("_deps")))
        return res

    def visit_FullEx(self, node):      # a constant array is a scalar parameter
        res = self.scalar(node.val, _code_of(node.dtype), id(node))
        self.gen_shapes.append(node.shape)
        self.leaf_nodes.append((node, None, None))   # the plan holds while it stays unwritten
        return res

    def visit_RandEx(self, node):      # a stretch of a Philox stream, from the element index
        words = [node.key & _M64, node.key >> 64] + [(node.counter >> (64 * k)) & _M64 for k in range(4)]
        refs = [self.scalar(w - (1 << 64) if w >> 63 else w, "i8")[0] for w in words]
        if node.pos:        # the draw starts inside a block
            refs.append(self.scalar(node.pos, "i8", ("pos", id(node)))[0])
        code = _code_of(node.dtype)
        res = self.op({"i8": "philox_raw", "f8": "philox_f8", "f4": "philox_f4"}[code], code, code, refs)
        self.gen_shapes.append(node.shape)
        self.iotas.append((res[0][1], node))
        self.leaf_nodes.append((node, None, None))
        return res

    def visit_IotaEx(self, node):      # the element index, converted
        code = _code_of(node.dtype)
        res = self.op("iota", code, code, [])
        self.gen_shapes.append(node.shape)
        self.iotas.append((res[0][1], node))
        self.leaf_nodes.append((node, None, None))
        return res

    def materialise_indices(self):
        """Turn every index-valued leaf into an array that is read like any other
        (for kernels that do not walk a 1-d array of exactly that length)."""
        for k, node in self.iotas:
            arr = node._force()
            ref, code = self.leaf(arr)
            self.ops[k] = ("positive", code, code, (ref,))
            self.leaf_nodes = [entry for entry in self.leaf_nodes if entry[0] is not node]
            self.leaf_nodes.append((node, arr, node.__dict__.get("_deps")))
        self.iotas = []

    def program(self, roots):
        return Program(self.leaf_codes, self.scalar_codes, self.ops, roots, TUNE["dmath"], TUNE["smath"],
                       TUNE["softdiv"])


# ---------------------------------------------------------------------------
# kernel cache
# ---------------------------------------------------------------------------

class Kernel:
    __slots__ = ("func", "finalize", "packer", "source")


_KERNELS = {}


def _cache_dir():
    d = os.environ.get("DELAYREPAY_CACHE_DIR")
    if d is None:
        d = os.path.join(os.path.expanduser("~"), ".cache", "delayrepay_amd")
    return d


def _load_or_compile(source):
    """Module handle for `source`: on-disk code-object cache, else hiprtc."""
    hiprt.init()
    use_disk = "DELAYREPAY_NO_DISK_CACHE" not in os.environ
    path = None
    if use_disk:
        info = hiprt.device_info()
        digest = hashlib.sha256("\0".join([source, info["arch"], str(info["hiprtc_version"])]
                                          + COMPILE_OPTS).encode()).hexdigest()
        path = os.path.join(_cache_dir(), digest + ".co")
        if os.path.exists(path):
            try:
                with open(path, "rb") as fh:
                    module = hiprt.load_code(fh.read())
                STATS["disk_hits"] += 1
                return module
            except (OSError, hiprt.DrhipError):
                pass
    module, code = hiprt.compile_module(source, "dr_kernel.hip", COMPILE_OPTS)
    STATS["compiles"] += 1
    if path is not None:
        try:
            os.makedirs(os.path.dirname(path), exist_ok=True)
            tmp = f"{path}.{os.getpid()}.tmp"
            with open(tmp, "wb") as fh:
                fh.write(code)
            os.replace(tmp, path)
        except OSError as exc:
            # not fatal, but every process would then recompile every kernel: say so once
            STATS["disk_write_failures"] += 1
            if STATS["disk_write_failures"] == 1:
                warnings.warn(f"delayrepay_amd: cannot write the kernel cache under "
                              f"{_cache_dir()!r} ({exc}); kernels will be recompiled by every "
                              "process.  Set DELAYREPAY_CACHE_DIR to a writable directory or "
                              "DELAYREPAY_NO_DISK_CACHE=1 to silence this.", RuntimeWarning,
                              stacklevel=2)
    return module


# Lanes per block of the kernels that are not launched with `codegen.BLOCK` of them (a row
# kernel whose block of 512 or 1024 lanes holds one long row), by function handle.
_BLOCK_OF = {}


def _kernel_name(low):
    """Symbol of the generated kernel: shape kind plus a digest of the cache key, so
    that profilers list structurally different kernels separately."""
    kind = low.kind + ("_reduce" if low.fin_count else "")
    return f"dr_{kind}_{hashlib.sha1(repr(low.key).encode()).hexdigest()[:10]}"


def _source(low):
    name = _kernel_name(low)
    return low.emit().replace("dr_finalize", name + "_fin").replace("dr_kernel", name), name


def _kernel_for(low, with_finalize):
    kern = _KERNELS.get(low.key)
    if kern is not None:
        STATS["mem_hits"] += 1
        return kern
    source, name = _source(low)
    module = _load_or_compile(source)
    kern = Kernel()
    kern.source = source
    kern.func = hiprt.get_function(module, name)
    kern.finalize = hiprt.get_function(module, name + "_fin") if with_finalize else None
    kern.packer = struct.Struct(low.fmt)
    block = _block_lanes(low)
    if block != cg.BLOCK:
        _BLOCK_OF[kern.func] = block
    _KERNELS[low.key] = kern
    return kern


class Replay:
    """Kernel launches recorded by `record()`: calling the object issues them again
    with the same arguments (same inputs, same outputs), without tracing, lowering
    or allocating.  Used to time kernels back to back and to re-run a fixed
    pipeline; it keeps the recorded outputs and scratch buffers alive.

    The recorded argument blocks hold device addresses.  Every replay bumps the write
    version of each buffer the recorded launches write, so results cached from those
    buffers are recomputed afterwards.  An update that reads what it overwrites goes
    through the buffer's second allocation and swaps the two addresses; a recording
    must therefore hold an even number of such updates per buffer (checked when the
    recording ends), and a replay refuses to run if a buffer's current address is not
    the one it was recorded with."""

    def __init__(self):
        self.launches = []      # (function, grid, lds bytes, packed arguments, scratch slot, bytes)
        self.keep = []
        self.written = []       # (buffer, whether the write swapped its two allocations)
        self._pinned = []       # (buffer, address it must have when a replay starts)
        self._scratch = []
        self._graph = None

    def _seal(self):
        swaps = {}
        for buf, swapped in self.written:
            if swapped:
                swaps[id(buf)] = (buf, swaps.get(id(buf), (buf, 0))[1] + 1)
        for buf, count in swaps.values():
            if count % 2:
                raise RuntimeError(
                    "hip.record(): an odd number of updates that read what they overwrite was "
                    "recorded for one array; record such sweeps in pairs, so that a replay "
                    "ends in the allocation it started in")
            self._pinned.append((buf, buf.ptr))

    def __call__(self):
        for buf, ptr in self._pinned:
            if buf.ptr != ptr:
                raise RuntimeError("replay refused: an array written by the recording has been "
                                   "swapped to its other allocation since it was recorded")
        if self._graph is not None:
            self._graph.launch()
        else:
            self._issue_all()
        for buf, swapped in self.written:
            if swapped:
                buf.version += 1
            else:
                buf.touch()

    def _issue_all(self):
        for func, grid, lds, args, slot, scratch in self.launches:
            if slot is None:
                hiprt.launch(func, grid, _BLOCK_OF.get(func, cg.BLOCK), lds, args, len(args))
            else:
                hiprt.launch_scratch(func, grid, _BLOCK_OF.get(func, cg.BLOCK), lds, args, len(args), slot, scratch)

    def as_graph(self):
        """Capture the recorded launches into a HIP graph; later calls replay the
        whole sequence with a single launch."""
        if self._graph is None and self.launches:
            hiprt.Graph.begin()
            try:
                self._issue_all()
            finally:
                graph = hiprt.Graph.end()
            self._graph = graph
        return self

    def __del__(self):
        for ptr in self._scratch:
            hiprt.free(ptr)
        self._scratch = []


_RECORDING = None


class record:
    """Context manager: `with hip.record() as plan: ...` runs the body normally
    and returns its kernel launches as a `Replay`."""

    def __enter__(self):
        global _RECORDING
        if _RECORDING is not None:
            raise RuntimeError("hip.record() does not nest")
        _RECORDING = Replay()
        return _RECORDING

    def __exit__(self, *exc):
        global _RECORDING
        rec, _RECORDING = _RECORDING, None
        if exc[0] is None:
            rec._seal()
        return False


# A result computed from results computed from results ...: past this many levels the
# older result is asked to become an array in its own right (`node._seal()`), so a loop of
# `x = f(x)` holds a bounded number of earlier iterates, and of their dependencies, alive.
MAX_GENERATIONS = 4
# An unevaluated operand at least this many operations deep that two earlier evaluations have
# already walked through is evaluated on its own when it is met a third time (shallower ones
# are cheaper to compute again than to write and read back; two roots that share a deep
# operand, a call and a put price, may well be asked for one after the other).
REUSE_DEPTH = 8
REUSE_AFTER = 2       # evaluations that computed it inline before it is computed on its own

_STAMP = 0            # bumped whenever tunables or the fusion mode change
_RECENT = collections.deque(maxlen=int(os.environ.get("DELAYREPAY_KEEP", "16")))
_RECENT_BYTES = int(os.environ.get("DELAYREPAY_KEEP_BYTES", str(8 << 30)))


_RECENT_SIZES = collections.deque()
_recent_held = 0


def _remember(node):
    """Keep `node` alive so that the same expression, built again, finds its nodes in
    the hash-cons table and its plan on the root.  A kept root also keeps its cached
    result, so the memory held this way is bounded as well as the count."""
    global _recent_held
    if not _RECENT.maxlen:
        return
    nbytes = numpy.dtype(node.dtype).itemsize
    for d in node.shape:
        nbytes *= d
    if len(_RECENT) == _RECENT.maxlen:
        _recent_held -= _RECENT_SIZES.popleft()
    _RECENT.append(node)
    _RECENT_SIZES.append(nbytes)
    _recent_held += nbytes
    while _recent_held > _RECENT_BYTES and len(_RECENT) > 1:
        _RECENT.popleft()
        _recent_held -= _RECENT_SIZES.popleft()


def forget():
    """Drop the recently evaluated roots kept alive for plan reuse."""
    global _recent_held
    _RECENT.clear()
    _RECENT_SIZES.clear()
    _recent_held = 0


class Plan:
    """Everything needed to launch an evaluated expression again: the lowered
    kernel choice, the leaves it reads, the shape and dtypes it produces.

    A plan is cached on the root node, and the last few evaluated roots are kept
    alive, so re-building the same expression over the same arrays (the body of an
    iterative loop) finds its nodes in the hash-cons table and its plan here: no
    tracing, no layout analysis, no cache-key hashing, only an argument pack and a
    launch.  `valid()` re-checks what could have changed underneath."""

    __slots__ = ("low", "kern", "checks", "stamp", "shape", "out_dtypes", "acc", "leaves",
                 "hazard", "region", "empty", "axes", "second", "kern2", "scratch", "out_shapes")

    def valid(self):
        if self.stamp != _STAMP:
            return False
        for node, arr, deps in self.checks:
            if node.__dict__.get("array") is not arr:
                return False
            if deps is not None:
                for buf, ver in deps:
                    if buf.version != ver:
                        return False
        return True

    def generation(self):
        """1 + the longest chain of cached results below this one."""
        gen = 0
        for node, _, _ in self.checks:
            g = node.__dict__.get("_gen", 0)
            if g > gen:
                gen = g
        return gen + 1

    def deps(self):
        """What the result just computed depends on, as (buffer, version) pairs: the
        buffers of the leaves and, for a leaf that is itself a cached result, what
        that result was computed from.  The cached leaf is refreshed in place when its
        own inputs change, which does not touch its buffer's version, so only the
        transitive closure tells a later reader that this result is stale too."""
        seen = {}
        for arr in self.leaves:
            seen[id(arr.buf)] = (arr.buf, arr.buf.version)
        for node, arr, deps in self.checks:
            if arr is None:                 # a generated leaf, still lazy
                seen[id(node)] = (node, 0)
            elif deps is not None:
                for dep in deps:
                    seen.setdefault(id(dep[0]), dep)
        return tuple(seen.values())


def _issue(func, grid, args, slot=None, scratch=0):
    """Launch (and record) one kernel.  `slot`: byte offset of the pointer parameter
    that takes the library's static scratch array, of which the kernel uses
    `scratch` bytes; None for a kernel without one."""
    if slot is None:
        hiprt.launch(func, grid, _BLOCK_OF.get(func, cg.BLOCK), 0, args, len(args))
    else:
        hiprt.launch_scratch(func, grid, _BLOCK_OF.get(func, cg.BLOCK), 0, args, len(args), slot, scratch)
    if _RECORDING is not None:
        _RECORDING.launches.append((func, grid, 0, args, slot, scratch))
    STATS["launches"] += 1


_SCRATCH_BYTES = hiprt.scratch_bytes()


def _partials(nbytes):
    """Where a reduction's partial results go: the library's static scratch array when
    they fit (nothing is allocated; launches on the one stream are ordered, so the
    finalising kernel has read them before the next reduction writes), else a pooled
    block.  Returns (pointer to pack, whether it is the static array)."""
    if nbytes <= _SCRATCH_BYTES and TUNE["static_scratch"]:
        return 0, True
    return hiprt.malloc(nbytes), False


_DEFER = None         # a list while launches are being collected (`_together`)


def _compile_together(entries):
    """Kernels that the collected launches need and that are not compiled yet, as ONE
    translation unit: the run-time compiler's fixed cost (120-190 ms here, whatever the
    kernel) is then paid once, not once per kernel.  The un-fused mode needs 46 kernels
    for Black-Scholes (cf. the reference's compile per evaluation, cuda.py:35-43)."""
    todo = {}
    for plan, _, reduce_out in entries:
        for low, kern, fin in ((plan.low, plan.kern, reduce_out is not None and plan.second is None),
                               (plan.second, plan.kern2, False)):
            if low is not None and kern is None and low.key not in _KERNELS:
                todo.setdefault(low.key, (low, fin))
    if len(todo) < 2:
        return
    parts, names = [], []
    for i, (low, fin) in enumerate(todo.values()):
        source, name = _source(low)
        # every kernel's source is complete in itself: its own namespace, and the macros
        # that differ from kernel to kernel start afresh
        parts.append("#undef DR_TAB_PTR\n#undef DR_LOG_TAB\n#undef DR_ERF_TAB\n#undef DR_STAGE_TABLES\n"
                     f"namespace dr_unit_{i} {{\n{source}\n}}\n")
        names.append((low, name, fin, source))
    module = _load_or_compile("".join(parts))
    for low, name, fin, source in names:
        kern = Kernel()
        kern.source = source
        kern.func = hiprt.get_function(module, name)
        kern.finalize = hiprt.get_function(module, name + "_fin") if fin else None
        kern.packer = struct.Struct(low.fmt)
        if _block_lanes(low) != cg.BLOCK:
            _BLOCK_OF[kern.func] = _block_lanes(low)
        _KERNELS[low.key] = kern


class _together:
    """Context: the launches inside are collected, their kernels compiled in one go, then
    issued in order."""

    def __enter__(self):
        global _DEFER
        self.outer = _DEFER
        if _DEFER is None:
            _DEFER = []
        return self

    def __exit__(self, exc_type, exc, tb):
        global _DEFER
        if self.outer is not None:       # nested: the outermost context issues everything
            return False
        entries, _DEFER = _DEFER, None
        if exc_type is None:
            _compile_together(entries)
            for plan, out_ptrs, reduce_out in entries:
                _fire(plan, out_ptrs, reduce_out)
        return False


def _fire(plan, out_ptrs, reduce_out=None):
    """Compile on first use, pack the argument block, launch."""
    if _DEFER is not None:
        _DEFER.append((plan, out_ptrs, reduce_out))
        return
    low = plan.low
    kern = plan.kern
    if kern is None:
        kern = plan.kern = _kernel_for(low, reduce_out is not None)
    ptrs = [buf.ptr + off for buf, off in low.srcs]
    slot = 8 * len(ptrs)         # the partials pointer follows the source pointers
    if plan.second is not None:
        # two-pass axis reduction: partials into scratch memory, then reduce those
        low2 = plan.second
        kern2 = plan.kern2
        if kern2 is None:
            kern2 = plan.kern2 = _kernel_for(low2, False)
        scratch, static = _partials(plan.scratch)
        args = kern.packer.pack(*ptrs, scratch, *low.scal, *low.tail)
        args2 = kern2.packer.pack(scratch, *out_ptrs, *low2.tail)
        if static:
            _issue(kern.func, low.grid, args, slot, plan.scratch)
            _issue(kern2.func, low2.grid, args2, 0, plan.scratch)
        else:
            _issue(kern.func, low.grid, args)
            _issue(kern2.func, low2.grid, args2)
            if _RECORDING is not None:
                _RECORDING._scratch.append(scratch)
            else:
                hiprt.free(scratch)  # stream-ordered: safe to recycle once queued
    elif reduce_out is not None:
        nbytes = low.fin_count * cg.ITEMSIZE[plan.acc]
        partial, static = _partials(nbytes)
        args = kern.packer.pack(*ptrs, partial, *low.scal, *low.tail)
        fin = struct.pack("@PPi", partial, reduce_out, low.fin_count)
        if static:
            _issue(kern.func, low.grid, args, slot, nbytes)
            _issue(kern.finalize, 1, fin, 0, nbytes)
        else:
            _issue(kern.func, low.grid, args)
            _issue(kern.finalize, 1, fin)
            if _RECORDING is not None:
                _RECORDING._scratch.append(partial)
            else:
                hiprt.free(partial)
    else:
        args = kern.packer.pack(*ptrs, *out_ptrs, *low.scal, *low.tail)
        _issue(kern.func, low.grid, args)


# ---------------------------------------------------------------------------
# evaluation entry points
# ---------------------------------------------------------------------------

_LOWERED = {}          # structure and geometry of an evaluation -> (Lowered, where its sources come from)
_LOWERED_MAX = 4096


def _lower_memo(prog, leaves, scalars, shape, out_codes, out_ptrs, out_strides, reduce_op,
                in_place=False):
    """`lowering.lower`, remembered by everything it looks at: the program, every operand's
    geometry, alignment, buffer size and which operands share a buffer, the destinations and
    the tunables.  The same expression over fresh arrays of the same layout (`x = f(x)` in a
    loop) then only has its buffers and scalar values filled in."""
    bufs = {}
    geo = []
    for a in leaves:
        buf = a.buf
        geo.append((a.shape, a._strides, a.offset, a.dtype.str, bufs.setdefault(id(buf), len(bufs)),
                    buf.nbytes, buf.ptr & 255))
    key = (prog.key(), tuple(geo), tuple(shape), tuple(out_codes), tuple(out_ptrs),
           tuple(tuple(st) for st in out_strides), reduce_op, in_place, tuple(TUNE.values()))
    hit = _LOWERED.get(key)
    if hit is not None:
        template, recipe = hit
        low = _Lowered()
        low.key, low.kind, low.emit, low.fmt = template.key, template.kind, template.emit, template.fmt
        low.tail, low.grid, low.fin_count, low.lds = template.tail, template.grid, template.fin_count, template.lds
        low.row_out = template.row_out
        low.srcs = [(leaves[i].buf, off) for i, off in recipe]
        low.scal = list(scalars)
        low.recipe = recipe
        STATS["lowering_hits"] += 1
        return low
    low = _lower(prog, leaves, scalars, shape, out_codes, out_ptrs, out_strides, reduce_op, in_place)
    low.recipe = None
    if low.kind != "rows":
        low.row_out = None
    recipe = []
    for buf, off in low.srcs:
        for i, a in enumerate(leaves):
            if a.buf is buf and a.offset * a.dtype.itemsize == off:
                recipe.append((i, off))
                break
        else:
            return low          # a source that is no operand's own view: not remembered
    if low.scal == list(scalars):
        if len(_LOWERED) >= _LOWERED_MAX:
            _LOWERED.clear()
        template = _Lowered()                     # holds no buffer alive
        template.key, template.kind, template.emit, template.fmt = low.key, low.kind, low.emit, low.fmt
        template.tail, template.grid, template.fin_count, template.lds = (low.tail, low.grid,
                                                                          low.fin_count, low.lds)
        template.row_out = low.row_out
        _LOWERED[key] = (template, recipe)
        low.recipe = recipe
    return low


# ---------------------------------------------------------------------------
# plans for structures seen before
# ---------------------------------------------------------------------------
# A step over fresh arrays (a new batch of data through the same expression) finds
# neither its nodes in the hash-cons table nor a plan on its root.  Tracing, type
# resolution, the program's key and the lowering's key then cost more host time than
# a SAXPY kernel of 2^24 elements runs.  `_scan` walks such a DAG once, in the tracer's
# order, and writes down everything the tracer and the lowering would look at: each
# node's function, which operand is which earlier node, each number's type, each leaf's
# geometry.  A structure met before has its plan in `_SEEN`; only buffers and numbers
# are filled in.

_SEEN = {}
_SEEN_MAX = 4096
_CALL_KINDS = frozenset(("BinaryNumpyEx", "BinaryFuncEx", "UnaryFuncEx"))


class _Unseen(Exception):
    """The expression has something in it that the tracer must look at itself."""


def _walk(node, key, leaves, uses, deep, index, bufs):
    """One ufunc node of `_scan`, operands first (a function of the module, not a closure:
    a closure that calls itself is a reference cycle, and what it holds would wait for the
    cycle collector)."""
    index[id(node)] = len(index)
    add = key.append
    add(node.func.__name__)
    children = node.children
    for child in children:
        n = index.get(id(child))
        if n is not None:
            add(n)
            continue
        kind = child.__class__.__name__
        if kind == "Scalar":
            index[id(child)] = len(index)
            add(scalar_descr(child.val))
        elif kind == "NPArray":
            index[id(child)] = len(index)
            arr = child.array
            buf = arr.buf
            add((arr.shape, arr._strides, arr.offset, arr.dtype.str,
                 bufs.setdefault(id(buf), len(bufs)), buf.nbytes, buf.ptr & 255))
            leaves.append(child)
        elif kind in _CALL_KINDS:
            d = child.__dict__
            if "array" in d:
                raise _Unseen
            if child._depth >= REUSE_DEPTH:
                if d.get("_seen", 0) >= REUSE_AFTER:
                    raise _Unseen
                deep.append(d)
            _walk(child, key, leaves, uses, deep, index, bufs)
        elif kind == "ReduceEx":
            # a reduction along the last axis that keeps it: an operation of the row kernel
            # (anything else the tracer evaluates on its own: not a structure to remember)
            if "array" in child.__dict__ or not getattr(child, "keepdims", False) \
                    or child.axis != (len(child.children[0].shape) - 1,):
                raise _Unseen
            add(("rows", child.children[0].shape[-1]))
            _walk(child, key, leaves, uses, deep, index, bufs)
        else:
            raise _Unseen
    for child in children:
        if child.__class__.__name__ == "Scalar":
            uses.append(child)


def _scan(roots, head):
    """(key, leaf nodes, uses of numbers, deep operands) of the DAG under `roots`, or None
    when it holds anything but ufunc nodes over arrays and numbers: an evaluated interior
    node, a generated leaf, a cast, a selection."""
    key = list(head)
    leaves, uses, deep = [], [], []
    index, bufs = {}, {}
    try:
        for root in roots:
            if root.__class__.__name__ not in _CALL_KINDS or "array" in root.__dict__:
                return None
            n = index.get(id(root))
            if n is not None:
                key.append(n)
            else:
                _walk(root, key, leaves, uses, deep, index, bufs)
            key.append(None)
    except (_Unseen, AttributeError):
        return None
    key.append(_STAMP)
    return tuple(key), leaves, uses, deep


def _seen_before(scan):
    """The plan of an earlier evaluation of this structure over these arrays and numbers,
    or None."""
    key, leaf_nodes, uses, deep = scan
    hit = _SEEN.get(key)
    if hit is None:
        return None
    model, slots, codes = hit
    mlow = model.low
    arrays = [node.array for node in leaf_nodes]
    scal = [None] * len(codes)
    for node, slot in zip(uses, slots):
        scal[slot] = _scalar_value(node.val, codes[slot])
    low = _Lowered()
    low.key, low.kind, low.emit, low.fmt = mlow.key, mlow.kind, mlow.emit, mlow.fmt
    low.tail, low.grid, low.fin_count, low.lds = mlow.tail, mlow.grid, mlow.fin_count, mlow.lds
    low.recipe = mlow.recipe
    low.srcs = [(arrays[i].buf, off) for i, off in mlow.recipe]
    low.scal = scal
    if model.kern is None:
        model.kern = _kernel_for(low, model.acc is not None)
    plan = Plan()
    plan.low = low
    plan.kern = model.kern
    plan.stamp = _STAMP
    plan.checks = [(node, arr, None) for node, arr in zip(leaf_nodes, arrays)]
    plan.leaves = arrays
    plan.shape, plan.out_dtypes, plan.acc = model.shape, model.out_dtypes, model.acc
    plan.hazard = False
    plan.region = None
    plan.empty = False
    plan.axes = False
    plan.second = None
    plan.kern2 = None
    plan.scratch = 0
    plan.out_shapes = model.out_shapes
    low.row_out = mlow.row_out
    for d in deep:
        d["_seen"] = d.get("_seen", 0) + 1
    STATS["seen_hits"] += 1
    return plan


def _remember_structure(scan, tracer, plan):
    """Keep `plan` as the model for this structure, if the tracer saw what `_scan` saw
    (it may have evaluated a deep operand on its own, or met a leaf twice under two
    nodes) and the lowering can be filled in again from the leaves alone."""
    key, leaf_nodes, uses, _ = scan
    low = plan.low
    if low is None or plan.second is not None or plan.axes or low.recipe is None:
        return
    seen_nodes = tracer.leaf_nodes
    if len(seen_nodes) != len(leaf_nodes) or len(tracer.leaves) != len(leaf_nodes) \
            or len(tracer.scalar_uses) != len(uses):
        return
    for (node, arr, deps), mine in zip(seen_nodes, leaf_nodes):
        if node is not mine or deps is not None:
            return
    if len(_SEEN) >= _SEEN_MAX:
        _SEEN.clear()
    model = Plan()
    mlow = _Lowered()         # holds no buffer alive
    mlow.key, mlow.kind, mlow.emit, mlow.fmt = low.key, low.kind, low.emit, low.fmt
    mlow.tail, mlow.grid, mlow.fin_count, mlow.lds = low.tail, low.grid, low.fin_count, low.lds
    mlow.recipe = low.recipe
    mlow.row_out = low.row_out
    model.low = mlow
    model.kern = plan.kern
    model.out_shapes = plan.out_shapes
    model.shape, model.out_dtypes, model.acc = plan.shape, plan.out_dtypes, plan.acc
    _SEEN[key] = (model, tuple(tracer.scalar_uses), tuple(tracer.scalar_codes))


def _common_shape(leaves, gen_shapes):
    """Broadcast shape of the operands (most often they all have the same one)."""
    if leaves and not gen_shapes:
        first = leaves[0].shape
        for a in leaves:
            if a.shape != first:
                break
        else:
            return first
    return tuple(numpy.broadcast_shapes(*[a.shape for a in leaves], *gen_shapes))


def _make_plan(tracer, roots, dst=None, reduce_op=None, axes=None):
    """Lower traced `roots` (list of (ref, code)) into a Plan.  `dst`: existing
    destination view (single root); `reduce_op`/`axes`: reduce the single root with
    that ufunc over everything (axes None) or over those axes."""
    if tracer.iotas:
        # the element index is at hand only in the flat kernel, over a 1-d array
        shape = dst.shape if dst is not None else tuple(numpy.broadcast_shapes(
            *[a.shape for a in tracer.leaves], *tracer.gen_shapes))
        if axes is not None or len(shape) != 1 or (dst is not None and dst._strides != (1,)) \
                or any(node.shape != shape for _, node in tracer.iotas):
            tracer.materialise_indices()
    prog = tracer.program(roots)
    leaves = tracer.leaves
    plan = Plan()
    plan.kern = None
    plan.stamp = _STAMP
    plan.checks = tracer.leaf_nodes
    plan.leaves = list(leaves)
    plan.hazard = False
    plan.region = None
    plan.acc = None
    plan.empty = False
    plan.axes = False
    plan.second = None
    plan.kern2 = None
    plan.scratch = 0
    plan.out_shapes = None
    if tracer.row_len is not None:
        # reductions along the last axis inside the expression: rows are reduced and used
        # again in one kernel, or the caller evaluates those reductions on their own
        if dst is not None:
            raise cg.RowFusionUnsupported("row reductions inside a write")
        shape = _common_shape(leaves, tracer.gen_shapes)
        if not shape or shape[-1] != tracer.row_len or 0 in shape:
            raise cg.RowFusionUnsupported("the rows of the reductions are not the rows of the result")
        if reduce_op:
            # the root itself is reduced along the rows: one more operation, one value per row
            if axes != (len(shape) - 1,) or reduce_op not in _ROW_OPS or roots[0][1] not in ("f4", "f8"):
                raise cg.RowFusionUnsupported("a reduction along other axes than the rows")
            roots = [tracer.op(_ROW_OPS[reduce_op], roots[0][1], roots[0][1], [roots[0][0]])]
            prog = tracer.program(roots)
        out_codes = [code for _, code in roots]
        plan.out_dtypes = [code_dtype(code) for code in out_codes]
        plan.shape = shape
        plan.low = _lower_memo(prog, leaves, tracer.scalars, shape, out_codes, [0] * len(roots), [], None)
        plan.out_shapes = [shape[:-1] + (1,) if u else shape for u in plan.low.row_out]
        return plan
    if reduce_op:
        shape = _common_shape(leaves, tracer.gen_shapes)
        code = roots[0][1]
        plan.acc = "i8" if (reduce_op == "add" and code in ("i4", "u4", "u1", "b1")) else code
        plan.out_dtypes = [code_dtype(plan.acc)]
        if axes is not None:
            plan.shape = tuple(d for k, d in enumerate(shape) if k not in axes)
            plan.axes = True
            if 0 in shape:
                if reduce_op != "add" and 0 in [shape[k] for k in axes]:
                    raise ValueError(f"zero-size array to reduction operation {reduce_op} "
                                     "which has no identity")
                plan.empty = True
                plan.low = None
                return plan
            plan.low, S, K, strategy = _lower_axis_reduce(prog, leaves, tracer.scalars, shape,
                                                          axes, plan.acc, reduce_op)
            if S > 1:
                # second pass over the S partials of every output: an identity program on
                # a stand-in array with the partials' layout (pointer filled in at launch)
                acc_dt = code_dtype(plan.acc)
                pshape, paxis = ((S, K), (0,)) if strategy == "col" else ((K, S), (1,))
                stand_in = ndarray(pshape, acc_dt, _Elsewhere(S * K * acc_dt.itemsize))
                prog2 = Program([plan.acc], [], [], [(("l", 0), plan.acc)])
                plan.second = _lower_axis_reduce(prog2, [stand_in], [], pshape, paxis, plan.acc,
                                                 reduce_op, slices=1)[0]
                plan.scratch = S * K * acc_dt.itemsize
            return plan
        plan.shape = ()
        if 0 in shape:
            if reduce_op != "add":
                raise ValueError(f"zero-size array to reduction operation {reduce_op} "
                                 "which has no identity")
            plan.empty = True
            plan.low = None
            return plan
        plan.low = _lower_memo(prog, leaves, tracer.scalars, shape, [plan.acc], [], [], reduce_op)
        if tracer.iotas and plan.low.kind != "flat":
            tracer.materialise_indices()
            return _make_plan(tracer, roots, None, reduce_op)
        return plan
    if dst is None:
        shape = _common_shape(leaves, tracer.gen_shapes)
        plan.out_dtypes = [code_dtype(code) for _, code in roots]
        out_codes = [code for _, code in roots]
        out_ptrs = [0] * len(roots)          # pool blocks are 256-byte aligned
        out_strides = [list(_contiguous(shape))] * len(roots)
        in_place = False
    else:
        shape = dst.shape
        plan.out_dtypes = [dst.dtype]
        out_codes = [dtype_code(dst.dtype)]
        out_ptrs = [dst.offset * dst.dtype.itemsize]   # alignment relative to the buffer start
        out_strides = [_broadcast_strides(dst, shape)]
        in_place = any(a.buf is dst.buf for a in leaves)
    plan.shape = shape
    n = 1
    for d in shape:
        n *= d
    if n == 0:
        plan.empty = True
        plan.low = None
        return plan
    plan.low = _lower_memo(prog, leaves, tracer.scalars, shape, out_codes, out_ptrs, out_strides, None,
                      in_place)
    if tracer.iotas and plan.low.kind != "flat":
        tracer.materialise_indices()
        return _make_plan(tracer, roots, dst)
    return plan


def _contiguous(shape):
    strides, acc = [], 1
    for d in reversed(shape):
        strides.append(acc if d != 1 else 0)
        acc *= d
    return tuple(reversed(strides))


def _launch_fresh(plan):
    """Allocate outputs for `plan` and launch it; returns the output arrays."""
    if plan.axes:
        out = ndarray(plan.shape, plan.out_dtypes[0])
        if plan.empty:
            if out.size:
                assign(out, 0)
        else:
            _fire(plan, [out.ptr])
        outs = [out]
    elif plan.acc is not None:
        out = ndarray((), plan.out_dtypes[0])
        if plan.empty:       # sum over nothing
            (hiprt.fill64 if out.itemsize == 8 else hiprt.fill32)(out.ptr, 0, 1)
        else:
            _fire(plan, [], out.ptr)
        outs = [out]
    else:
        if plan.out_shapes is not None:
            outs = [ndarray(shape, dt) for shape, dt in zip(plan.out_shapes, plan.out_dtypes)]
        else:
            outs = [ndarray(plan.shape, dt) for dt in plan.out_dtypes]
        if not plan.empty:
            _fire(plan, [o.ptr for o in outs])
    if _RECORDING is not None:
        _RECORDING.keep += outs + plan.leaves
    return outs


def _trace_root(tracer, node):
    return tracer.visit(node)


def _run_unfused(ex, evaluated):
    """One kernel per interior node, children first."""
    nid = id(ex)
    if nid in evaluated:
        return evaluated[nid]
    if _kind(ex) == "NPArray":
        return ex.array
    for child in ex.children:
        if _kind(child) not in ("Scalar", "NPArray"):
            _run_unfused(child, evaluated)
    tracer = Tracer(evaluated)
    if _kind(ex) == "ReduceEx":
        root = tracer.visit(ex.children[0])
        out = _launch_fresh(_make_plan(tracer, [root], reduce_op=ex.func.__name__,
                                       axes=getattr(ex, "axis", None)))[0]
        if out.shape != tuple(ex.shape):
            out = out.reshape(tuple(ex.shape))
    else:
        root = tracer.visit(ex)
        out = _launch_fresh(_make_plan(tracer, [root]))[0]
    evaluated[nid] = out
    return out


def run(ex):
    """Evaluate one DAG root; returns a new device array owned by the caller
    (cf. cuda.py:91-96)."""
    if not _FUSED:
        with _together():
            return _run_unfused(ex, {})
    d = ex.__dict__
    plan = d.get("_plan")
    if plan is None or not plan.valid():
        reduction = _kind(ex) == "ReduceEx"
        if reduction:
            axis = getattr(ex, "axis", None)
            scan = None if axis is not None else _scan(ex.children[:1], ("reduce", ex.func.__name__))
        else:
            scan = _scan((ex,), ("run",))
        plan = _seen_before(scan) if scan is not None else None
        if plan is None:
            for rows in (True, False):
                # first with reductions along the last axis as operations of the program;
                # when the row kernel does not take the result, with those evaluated first
                tracer = Tracer(reuse=True, rows=rows)
                try:
                    if reduction:
                        root = tracer.visit(ex.children[0])
                        plan = _make_plan(tracer, [root], reduce_op=ex.func.__name__, axes=axis)
                    else:
                        root = _trace_root(tracer, ex)
                        plan = _make_plan(tracer, [root])
                    break
                except cg.RowFusionUnsupported:
                    if not rows:
                        raise
            if scan is not None:
                _remember_structure(scan, tracer, plan)
        d["_plan"] = plan
        _remember(ex)
    else:
        STATS["plan_hits"] += 1
    out = _launch_fresh(plan)[0]
    if out.shape != tuple(ex.shape) and _kind(ex) == "ReduceEx":
        out = out.reshape(tuple(ex.shape))      # the reduced axes kept, or a row kernel's column
    d["_deps"] = plan.deps()
    d["_gen"] = plan.generation()
    return out


def run_multi(exs):
    """Evaluate several roots; roots of equal shape share one kernel (and their
    common sub-expressions)."""
    if not _FUSED:
        with _together():       # one kernel per node, a node shared by two roots once
            evaluated = {}
            return [_run_unfused(ex, evaluated) for ex in exs]
    by_shape = {}
    for i, ex in enumerate(exs):
        by_shape.setdefault(tuple(ex.shape), []).append(i)
    results = [None] * len(exs)
    for shape, idxs in by_shape.items():
        first = exs[idxs[0]].__dict__
        key = tuple(id(exs[i]) for i in idxs)
        cached = first.get("_multi")
        if cached is not None and cached[0] == key and cached[1].valid():
            plan = cached[1]
            STATS["plan_hits"] += 1
        else:
            scan = _scan([exs[i] for i in idxs], ("multi",))
            plan = _seen_before(scan) if scan is not None else None
            if plan is None:
                for rows in (True, False):
                    tracer = Tracer(reuse=True, rows=rows)
                    try:
                        roots = [_trace_root(tracer, exs[i]) for i in idxs]
                        plan = _make_plan(tracer, roots)
                        break
                    except cg.RowFusionUnsupported:
                        if not rows:
                            raise
                if scan is not None:
                    _remember_structure(scan, tracer, plan)
            # the other roots are kept alive with the entry (the key holds their ids, which
            # are only theirs while they live); not the first root itself: on its own
            # attribute that would be a reference cycle, and every result would wait for
            # the cycle collector
            first["_multi"] = (key, plan, [exs[i] for i in idxs[1:]])
            _remember(exs[idxs[0]])
        outs = _launch_fresh(plan)
        deps = plan.deps()
        gen = plan.generation()
        for i, out in zip(idxs, outs):
            if out.shape != shape:   # every leaf of this root was a broadcast scalar
                out = materialise(out, shape=shape)
            results[i] = out
            exs[i].__dict__["_deps"] = deps
            exs[i].__dict__["_gen"] = gen
    return results


def _extent(arr):
    """[lo, hi) element range of the buffer that `arr` can touch."""
    lo = hi = arr.offset
    for d, s in zip(arr.shape, arr._strides):
        if d == 0:
            return (arr.offset, arr.offset)
        if s >= 0:
            hi += (d - 1) * s
        else:
            lo += (d - 1) * s
    return lo, hi + 1


def _same_view(a, b):
    return (a.offset == b.offset and a.shape == b.shape and a._strides == b._strides
            and a.dtype == b.dtype)


def _plan_write(tracer, root, dst):
    """Plan for launching traced `root` into the existing view `dst`; decides
    whether the kernel would read what it overwrites."""
    shape = dst.shape
    for a in tracer.leaves:
        _broadcast_strides(a, shape)  # raises when the value does not fit the destination
    for gen in tracer.gen_shapes:     # generated leaves have a shape too
        if tuple(numpy.broadcast_shapes(gen, shape)) != tuple(shape):
            raise ValueError(f"could not broadcast input array from shape {tuple(gen)} "
                             f"into shape {tuple(shape)}")
    hazard = False
    d_lo, d_hi = _extent(dst)
    for a in tracer.leaves:
        if a.buf is dst.buf and not _same_view(a, dst):
            a_lo, a_hi = _extent(a)
            it = dst.dtype.itemsize
            if a_lo * a.dtype.itemsize < d_hi * it and d_lo * it < a_hi * a.dtype.itemsize:
                hazard = True
    if hazard:
        # the kernel will write a different allocation: lower it as not-in-place
        stand_in = ndarray(dst.shape, dst.dtype, _Elsewhere(dst.buf.nbytes), dst.offset,
                           dst._strides)
        plan = _make_plan(tracer, [root], dst=stand_in)
    else:
        plan = _make_plan(tracer, [root], dst=dst)
    plan.hazard = hazard
    plan.region = (dst.offset, dst.shape, dst._strides, dst.dtype.str)
    return plan


class _Elsewhere(Buffer):
    """Stands for "an allocation other than the source buffer, same layout" while
    lowering a ping-pong write; owns no memory."""

    __slots__ = ()

    def __init__(self, nbytes):
        self.nbytes = nbytes
        self.ptr = 0
        self.version = 0
        self.shadow = None
        self.shadow_region = None


def _write(plan, dst):
    """Launch `plan` into `dst`."""
    buf = dst.buf
    if plan.empty:
        return
    off = dst.offset * dst.dtype.itemsize
    if not plan.hazard:
        _fire(plan, [buf.ptr + off])
        buf.touch()
    else:
        # Ping-pong: write into the shadow allocation, which mirrors the buffer
        # everywhere outside `region`, then swap the two device pointers.  Every view
        # of the buffer (they share the Buffer object) sees the update at once.
        if buf.shadow is None:
            buf.shadow = hiprt.malloc(max(buf.nbytes, 1))
            buf.shadow_region = None
        if buf.shadow_region != plan.region:
            hiprt.memcpy_d2d(buf.shadow, buf.ptr, buf.nbytes)
        _fire(plan, [buf.shadow + off])
        buf.ptr, buf.shadow = buf.shadow, buf.ptr
        buf.shadow_region = plan.region
        buf.version += 1
    if _RECORDING is not None:
        _RECORDING.keep += [dst] + plan.leaves
        _RECORDING.written.append((buf, plan.hazard))


def run_into(ex, dst):
    """`dst[...] = ex` as one fused kernel writing the destination view directly."""
    dst.check_writable()
    if not _FUSED:
        assign(dst, run(ex))
        return
    d = ex.__dict__
    key = (id(dst.buf), dst.offset, dst.shape, dst._strides, dst.dtype.str)
    cached = d.get("_into")
    if cached is not None and cached[0] == key and cached[1].valid():
        plan = cached[1]
        STATS["plan_hits"] += 1
    else:
        tracer = Tracer(reuse=True)
        root = _trace_root(tracer, ex)
        plan = _plan_write(tracer, root, dst)
        d["_into"] = (key, plan, dst.buf)     # holding the buffer keeps its id unique
        _remember(ex)
    _write(plan, dst)


def assign(dst, value):
    """`dst[...] = value` for a number, a host array or a device array."""
    from .delayarray import DelayArray
    if isinstance(value, DelayArray):
        if "array" in value.__dict__:
            value = value._force()
        else:
            return run_into(value, dst)
    tracer = Tracer()
    if isinstance(value, ndarray):
        root = tracer.leaf(value)
    elif isinstance(value, (int, float, bool, numpy.generic)):
        root = tracer.scalar(value, dtype_code(dst.dtype))
    else:
        host = numpy.asarray(value)
        if host.ndim == 0:
            root = tracer.scalar(host[()], dtype_code(dst.dtype))
        else:
            root = tracer.leaf(ndarray.from_host(host))
    _write(_plan_write(tracer, root, dst), dst)


def materialise(arr, dtype=None, shape=None):
    """Contiguous copy of a device array, optionally converted / broadcast."""
    tracer = Tracer()
    root = tracer.leaf(arr)
    if dtype is not None and numpy.dtype(dtype) != arr.dtype:
        code = dtype_code(dtype)
        root = tracer.op("cast", code, code, [root[0]])
    if shape is not None and tuple(shape) != arr.shape:
        out = ndarray(shape, code_dtype(root[1]))
        _write(_plan_write(tracer, root, out), out)
        return out
    return _launch_fresh(_make_plan(tracer, [root]))[0]


def run_reduce_product(a, b):
    from .delayarray import NPArray, ReduceEx
    return run(ReduceEx(numpy.add, NPArray(a) * NPArray(b)))


def lower_only(exs, dst=None):
    """Trace and lower without touching the device: returns (Lowered, source).
    Works with placeholder arrays on a machine that has no GPU."""
    if not isinstance(exs, (list, tuple)):
        exs = [exs]
    tracer = Tracer(rows=True)
    if _kind(exs[0]) == "ReduceEx":
        root = tracer.visit(exs[0].children[0])
        low = _make_plan(tracer, [root], reduce_op=exs[0].func.__name__,
                         axes=getattr(exs[0], "axis", None)).low
    elif dst is not None:
        low = _plan_write(tracer, tracer.visit(exs[0]), dst).low
    else:
        low = _make_plan(tracer, [tracer.visit(ex) for ex in exs]).low
    return low, _source(low)[0]


def compile_source(source):
    """hiprtc-compile generated source without loading it (no GPU needed)."""
    return hiprt.compile_only(source, "dr_kernel.hip", COMPILE_OPTS)


# the `np` and `fallback` namespaces of the backend protocol live in arrayns.py (it
# imports this module, hence the late import)
from .arrayns import fallback, np  # noqa: E402,F401
