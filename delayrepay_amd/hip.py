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
import sys

import numpy

from . import codegen as cg
from . import hiprt
from .devarray import Buffer, ndarray, placeholder  # noqa: F401
from .codegen import Program, dtype_code, code_dtype

hiprt.lib()  # fail at import when libdrhip.so has not been built

COMPILE_OPTS = [
    "-O3",
    "-ffp-contract=off",                      # a*b+c stays two roundings, like NumPy
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",  # no v_pk_*_f32
]

# Tunables; part of every cache key.  DELAYREPAY_TUNE="unroll=2,bpc=16" overrides.
TUNE = {
    "unroll": 1,      # 16-byte vectors per thread and chunk in flat element-wise kernels
    "red_unroll": 4,  # the same for flat kernels with a reduction tail
    "red_blocks": 4096,  # most blocks (= partial results) of a reduction kernel
    "flat_cap": 0,    # most blocks of a flat element-wise kernel (0: one chunk per block)
    "bpc": 8,         # resident blocks per CU that bound the grid of `nd` kernels
    "ntl": 1,         # non-temporal loads  } for working sets beyond `cache_mib`;
    "nts": 1,         # non-temporal stores } smaller ones stay cacheable
    "cache_mib": 200,  # working sets up to this size are left to the 256 MB Infinity Cache
    "tw": 128,        # stencil tile width (elements)
    "th": 16,         # stencil tile height (rows)
    "lds": 1,         # stage shifted views through LDS (0: read them directly)
    "svec": 1,        # aligned stencils: 16-byte loads into LDS and 16-byte stores
    "gpr": 64,        # vectorised stencil: 16-byte column groups per tile row
    "rpt": 2,         # vectorised stencil: consecutive rows per thread
    "xcd": 1,         # vectorised stencil: give each XCD a contiguous band of tiles
    "sntl": 0,        # vectorised stencil: non-temporal loads / stores
    "snts": 1,
}
for _kv in filter(None, os.environ.get("DELAYREPAY_TUNE", "").split(",")):
    _k, _v = _kv.split("=")
    TUNE[_k.strip()] = int(_v)

_FUSED = "DELAY_UNFUSED" not in os.environ
STATS = {"launches": 0, "compiles": 0, "disk_hits": 0, "mem_hits": 0, "plan_hits": 0}

_SCALAR_FMT = {"f4": "f", "f8": "d", "i4": "i", "i8": "q", "u4": "I", "u1": "B", "b1": "B"}
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


_FE = None          # the front-end module, bound on first use (it imports this one)
_CODES = {}


def _bind_frontend():
    global _FE
    from . import delayarray
    _FE = delayarray


def _code_of(dtype):
    try:
        return _CODES[dtype]
    except KeyError:
        return _CODES.setdefault(dtype, dtype_code(dtype))


class Tracer:
    """Collects leaves, scalar parameters and SSA operations of one or more roots."""

    def __init__(self, evaluated=None):
        self.leaves = []
        self.leaf_codes = []
        self._leaf_index = {}
        self.scalars = []
        self.scalar_codes = []
        self._scalar_index = {}
        self.ops = []
        self._memo = {}
        self._evaluated = evaluated if evaluated is not None else {}
        self.leaf_nodes = []      # (node, its array, the deps it was computed from or None)

    def leaf(self, arr):
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
        if _FE is None:
            _bind_frontend()
        kind = type(node)
        arr = self._evaluated.get(nid) if self._evaluated else None
        if arr is None:
            arr = node.__dict__.get("array")
            if arr is not None and kind is not _FE.NPArray:
                deps = node.__dict__.get("_deps")
                if deps is not None and any(buf.version != ver for buf, ver in deps):
                    arr = None  # stale: recompute inside this kernel
        if arr is not None:
            res = self.leaf(arr)
            self.leaf_nodes.append((node, arr, node.__dict__.get("_deps")))
        elif kind is _FE.BinaryNumpyEx or kind is _FE.BinaryFuncEx or kind is _FE.UnaryFuncEx:
            func = node.func
            name = func.__name__
            result = _code_of(node.dtype)
            compute = result
            if name in _COMPARES:     # arithmetic in the operands' common type, bool out
                descrs = tuple(_FE._descr(c) for c in node.children)
                compute = dtype_code(_FE.result_dtype(
                    numpy.add if len(descrs) == 2 else numpy.positive, descrs))
                if compute == "b1" and name not in cg._PREDICATES:
                    compute = "u1"
            elif name not in cg.SUPPORTED_UFUNCS:
                raise NotImplementedError(f"ufunc {name!r} cannot be fused by the HIP backend")
            refs = []
            for child in node.children:
                if type(child) is _FE.Scalar:
                    refs.append(self.scalar(child.val, compute, id(child))[0])
                else:
                    refs.append(self.visit(child)[0])
            self.ops.append((name, compute, result, tuple(refs)))
            res = (("v", len(self.ops) - 1), result)
        elif kind is _FE.WhereEx:
            result = _code_of(node.dtype)
            refs = []
            for pos, child in enumerate(node.children):
                if type(child) is _FE.Scalar:
                    code = result if pos else dtype_code(numpy.asarray(child.val).dtype)
                    refs.append(self.scalar(child.val, code, id(child))[0])
                else:
                    refs.append(self.visit(child)[0])
            self.ops.append(("where", result, result, tuple(refs)))
            res = (("v", len(self.ops) - 1), result)
        elif kind is _FE.Scalar:
            res = self.scalar(node.val, dtype_code(numpy.asarray(node.val).dtype), nid)
        elif kind is _FE.CastEx:
            ref, code = self.visit(node.children[0])
            target = dtype_code(node.dtype)
            res = self.op("cast", target, target, [ref]) if code != target else (ref, code)
        elif kind is _FE.ReduceEx:
            res = self.leaf(node._force())
        else:
            raise NotImplementedError(f"{kind.__name__} nodes cannot be evaluated by the HIP backend")
        memo[nid] = res
        return res

    def program(self, roots):
        return Program(self.leaf_codes, self.scalar_codes, self.ops, roots)

    def deps(self):
        seen = {}
        for arr in self.leaves:
            seen[id(arr.buf)] = arr.buf
        return tuple((buf, buf.version) for buf in seen.values())


# ---------------------------------------------------------------------------
# layout analysis
# ---------------------------------------------------------------------------

def _broadcast_strides(arr, shape):
    """Element strides of `arr` viewed at `shape` (NumPy broadcasting)."""
    nd = len(shape)
    pad = nd - len(arr.shape)
    if pad < 0:
        raise ValueError(f"operand of shape {arr.shape} does not broadcast to {shape}")
    out = [0] * nd
    for k in range(len(arr.shape)):
        d = arr.shape[k]
        if d == shape[pad + k]:
            out[pad + k] = arr._strides[k] if d != 1 else 0
        elif d == 1:
            out[pad + k] = 0
        else:
            raise ValueError(f"operand of shape {arr.shape} does not broadcast to {shape}")
    return out


def _merge_dims(shape, stride_sets):
    """Drop unit dims and merge neighbours that every operand walks contiguously."""
    dims = [(d, [s[k] for s in stride_sets]) for k, d in enumerate(shape) if d != 1]
    if not dims:
        return [], [[] for _ in stride_sets]
    merged = [dims[0]]
    for d, strides in dims[1:]:
        pd, ps = merged[-1]
        if all(p == s * d for p, s in zip(ps, strides)):
            merged[-1] = (pd * d, strides)
        else:
            merged.append((d, strides))
    mshape = [d for d, _ in merged]
    msets = [[st[i] for _, st in merged] for i in range(len(stride_sets))]
    return mshape, msets


class Lowered:
    """A kernel choice for one evaluation: cache key, source builder, launch recipe."""

    __slots__ = ("key", "kind", "emit", "fmt", "srcs", "scal", "tail", "grid", "fin_count", "lds")


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
        arch = hiprt.device_info()["arch"]
        digest = hashlib.sha256("\0".join([source, arch] + COMPILE_OPTS).encode()).hexdigest()
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
        except OSError:
            pass
    return module


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
    _KERNELS[low.key] = kern
    return kern


# ---------------------------------------------------------------------------
# lowering
# ---------------------------------------------------------------------------

_CUS = None


def _grid_cap():
    """Blocks that fill the device `bpc` deep (256 CUs assumed until a device is open)."""
    global _CUS
    if _CUS is None:
        if not hiprt._initialised:
            return 256 * TUNE["bpc"]
        _CUS = hiprt.device_info()["compute_units"]
    return _CUS * TUNE["bpc"]


def _lower(prog, leaves, scalars, out_shape, out_codes, out_ptrs, out_strides, reduce_op,
           in_place=False):
    """Pick the kernel shape.  `out_ptrs`/`out_strides` describe the destinations
    (element strides at `out_shape`); for a reduction they are empty and the
    partial-sums pointer is appended at launch."""
    n = 1
    for d in out_shape:
        n *= d
    leaf_strides = [_broadcast_strides(a, out_shape) for a in leaves]
    mshape, msets = _merge_dims(out_shape, leaf_strides + list(out_strides))
    m_leaf, m_out = msets[:len(leaves)], msets[len(leaves):]
    ndim = len(mshape)
    low = Lowered()
    low.lds = 0
    low.fin_count = 0
    scal_fmt = "".join(_SCALAR_FMT[c] for c in prog.scalars)
    scal_vals = list(scalars)
    tune = tuple(sorted(TUNE.items()))

    flat = ndim <= 1 and all(s == [1] or s == [0] or s == [] for s in m_leaf) \
        and all(s == [1] or s == [] for s in m_out)
    if flat:
        leaf_class = tuple("b" if (s == [0] and n > 1) else "c" for s in m_leaf)
        ptrs = [a.ptr for a in leaves]
        widths_ok = all(cg.ITEMSIZE[c] in (4, 8) for c, k in zip(prog.leaves, leaf_class) if k == "c")
        align_ok = all(p % 16 == 0 for p, k in zip(ptrs, leaf_class) if k == "c")
        if not reduce_op:
            widths_ok = widths_ok and all(cg.ITEMSIZE[c] in (4, 8) for c in out_codes)
            align_ok = align_ok and all(p % 16 == 0 for p in out_ptrs)
        vec = widths_ok and align_ok and n >= 64
        unroll = TUNE["red_unroll"] if reduce_op else TUNE["unroll"]
        footprint = sum(a.nbytes for a, k in zip(leaves, leaf_class) if k == "c")
        if not reduce_op:
            footprint += sum(n * cg.ITEMSIZE[c] for c in out_codes)
        streaming = footprint > TUNE["cache_mib"] << 20
        ntl = bool(TUNE["ntl"]) and streaming
        nts = bool(TUNE["nts"]) and streaming
        low.kind = "flat"
        low.key = ("flat", prog.key(), leaf_class, tuple(out_codes), vec, reduce_op, in_place,
                   unroll, ntl, nts)

        def emit():
            src, _ = cg.emit_flat(prog, leaf_class, out_codes, vec, unroll, ntl, nts,
                                  restrict=not in_place, reduce_op=reduce_op)
            return src
        low.emit = emit
        if vec:
            widths = [cg.ITEMSIZE[c] for c, k in zip(prog.leaves, leaf_class) if k == "c"]
            if not reduce_op:
                widths += [cg.ITEMSIZE[c] for c in out_codes]
            E = 16 // min(widths) if widths else 4
        else:
            E = 1
        chunks = max(1, (n // E) // (cg.BLOCK * unroll))   # one chunk per block ...
        cap = TUNE["red_blocks"] if reduce_op else (TUNE["flat_cap"] or (1 << 24) - 1)
        low.grid = min(chunks, cap)
        n_out_ptr = 1 if reduce_op else len(out_ptrs)
        low.fmt = "@" + "P" * (len(ptrs) + n_out_ptr) + scal_fmt + "q"
        low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
        low.scal, low.tail = scal_vals, [n]
        if reduce_op:
            low.fin_count = low.grid
        return low

    tiled = (not reduce_op and ndim == 2 and all(s[1] == 1 for s in m_out)
             and all(s[1] == 1 or s == [0, 0] for s in m_leaf))
    if tiled:
        H, W = mshape
        tw, th = TUNE["tw"], TUNE["th"]
        # halo group: >= 2 leaves that are shifted views of one buffer
        groups = {}
        for i, (a, s) in enumerate(zip(leaves, m_leaf)):
            if s[1] == 1 and s[0] > 0:
                groups.setdefault((id(a.buf), s[0], prog.leaves[i]), []).append(i)
        best = max(groups.values(), key=len) if groups else []
        kinds = [None] * len(leaves)
        group = None
        if len(best) >= 2 and TUNE["lds"]:
            rs = m_leaf[best[0]][0]
            ref_off = min(leaves[i].offset for i in best)
            shifts = {}
            for i in best:
                d = leaves[i].offset - ref_off
                dy, dx = divmod(d, rs)
                if dx > rs // 2:
                    dy, dx = dy + 1, dx - rs
                shifts[i] = (dy, dx)
            dy_max = max(dy for dy, _ in shifts.values())
            dx_min = min(dx for _, dx in shifts.values())
            dx_max = max(dx for _, dx in shifts.values())
            itemsize = cg.ITEMSIZE[prog.leaves[best[0]]]
            lds_bytes = (th + dy_max) * (tw + dx_max - dx_min) * itemsize
            if dy_max <= 16 and dx_max - dx_min <= 32 and lds_bytes <= 48 * 1024:
                group = (prog.leaves[best[0]], dy_max, dx_min, dx_max)
                for i in best:
                    kinds[i] = ("g",) + shifts[i]
                g_buf = leaves[best[0]].buf
                g_ptr = g_buf.ptr + ref_off * itemsize
                g_src = (g_buf, ref_off * itemsize)
                g_args = [rs, -ref_off, g_buf.nbytes // itemsize - ref_off]
        for i, s in enumerate(m_leaf):
            if kinds[i] is None:
                kinds[i] = ("b",) if s == [0, 0] else ("d",)
        kinds = tuple(kinds)
        low.kind = "tile2d"
        vec_ok = False
        if group is not None and TUNE["svec"]:
            gsize = cg.ITEMSIZE[group[0]]
            vw = 16 // gsize
            vec_ok = (gsize in (4, 8) and all(cg.ITEMSIZE[c] == gsize for c in out_codes)
                      and g_args[0] % vw == 0 and all(s[0] % vw == 0 for s in m_out)
                      and len({(p // gsize) % vw for p in out_ptrs}) == 1)
        if vec_ok:
            ph_g = (g_ptr // gsize) % vw
            ph_o = (out_ptrs[0] // gsize) % vw
            gpr, rpt = TUNE["gpr"], TUNE["rpt"]
            sntl, snts = bool(TUNE["sntl"]), bool(TUNE["snts"])
            bands = bool(TUNE["xcd"])
            low.key = ("tile2dv", prog.key(), kinds, group, tuple(out_codes), in_place, ph_g, ph_o,
                       gpr, rpt, sntl, snts, bands)
            tw, th = gpr * vw, (cg.BLOCK // gpr) * rpt

            def emit():
                return cg.emit_stencil_vec(prog, kinds, group, out_codes, gpr, rpt, ph_g, ph_o,
                                           restrict=not in_place, nt_load=sntl, nt_store=snts,
                                           xcd_bands=bands)[0]
            W = W + ph_o          # tiles start `ph_o` columns left of the view
        else:
            low.key = ("tile2d", prog.key(), kinds, group, tuple(out_codes), in_place, tune)

            def emit():
                return cg.emit_stencil(prog, kinds, group, out_codes, tw, th,
                                       restrict=not in_place)
        low.emit = emit
        tiles_x = -(-W // tw)
        tiles_y = -(-H // th)
        low.grid = tiles_x * tiles_y
        srcs = [(a.buf, a.offset * a.dtype.itemsize) for a, k in zip(leaves, kinds) if k[0] != "g"]
        fmt = "@" + "P" * len(srcs)
        tail_vals = []
        if group is not None:
            fmt += "P"
            srcs.append(g_src)
        fmt += "P" * len(out_ptrs) + scal_fmt + "ii"
        tail_vals += [mshape[0], mshape[1]]
        if group is not None:
            fmt += "qqq"
            tail_vals += g_args
        fmt += "i"
        tail_vals.append(tiles_x)
        for k, s in zip(kinds, m_leaf):
            if k[0] == "d":
                fmt += "q"
                tail_vals.append(s[0])
        for s in m_out:
            fmt += "q"
            tail_vals.append(s[0])
        low.fmt = fmt
        low.srcs, low.scal, low.tail = srcs, scal_vals, tail_vals
        return low

    # general strided kernel
    if ndim == 0:
        mshape, m_leaf, m_out, ndim = [1], [[0] for _ in m_leaf], [[0] for _ in m_out], 1
    index32 = n < 2 ** 31
    low.kind = "nd"
    low.key = ("nd", prog.key(), ndim, tuple(out_codes), index32, reduce_op, tune)

    def emit():
        return cg.emit_nd(prog, ndim, out_codes, index32, reduce_op)
    low.emit = emit
    blocks = -(-n // cg.BLOCK)
    low.grid = max(1, min(blocks, _grid_cap()))
    n_out_ptr = 1 if reduce_op else len(out_ptrs)
    fmt = "@" + "P" * (len(leaves) + n_out_ptr) + scal_fmt + "q" + ("I" if index32 else "q") * ndim
    tail = [n] + list(mshape)
    for s in m_leaf:
        fmt += "q" * ndim
        tail += s
    if not reduce_op:
        for s in m_out:
            fmt += "q" * ndim
            tail += s
    low.fmt = fmt
    low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
    low.scal, low.tail = scal_vals, tail
    if reduce_op:
        low.fin_count = low.grid
    return low


def _lower_axis_reduce(prog, leaves, scalars, shape, axes, acc, reduce_op):
    """Kernel choice for reducing over `axes` of the (broadcast) `shape`."""
    kept = [d for d in range(len(shape)) if d not in axes]
    full = [_broadcast_strides(a, shape) for a in leaves]
    kshape = [shape[d] for d in kept]
    rshape = [shape[d] for d in axes]
    kmerged, ksets = _merge_dims(kshape, [[s[d] for d in kept] for s in full])
    rmerged, rsets = _merge_dims(rshape, [[s[d] for d in axes] for s in full])
    if not kmerged:
        kmerged, ksets = [1], [[0] for _ in leaves]
    if not rmerged:
        rmerged, rsets = [1], [[0] for _ in leaves]
    K = R = 1
    for d in kmerged:
        K *= d
    for d in rmerged:
        R *= d
    # coalescing decides the strategy: which side holds the unit-stride dimension
    inner_kept = any(s[-1] == 1 for s in ksets)
    inner_red = any(s[-1] == 1 for s in rsets)
    strategy = "col" if (inner_kept and not inner_red) or R < 64 else "row"
    low = Lowered()
    low.lds = 0
    low.fin_count = 0
    low.kind = "axis"
    kdim, rdim = len(kmerged), len(rmerged)
    low.key = ("axis", prog.key(), kdim, rdim, acc, reduce_op, strategy)

    def emit():
        return cg.emit_axis_reduce(prog, kdim, rdim, acc, reduce_op, strategy)
    low.emit = emit
    if strategy == "col":
        low.grid = max(1, min(-(-K // cg.BLOCK), _grid_cap()))
    else:
        low.grid = max(1, min(K, _grid_cap() * 4))
    low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
               + "qq" + "q" * (kdim + rdim) + "q" * ((kdim + rdim) * len(leaves)))
    tail = [K, R] + list(kmerged) + list(rmerged)
    for ks, rs in zip(ksets, rsets):
        tail += list(ks) + list(rs)
    low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
    low.scal, low.tail = list(scalars), tail
    return low


class Replay:
    """Kernel launches recorded by `record()`: calling the object issues them again
    with the same arguments (same inputs, same outputs), without tracing, lowering
    or allocating.  Used to time kernels back to back and to re-run a fixed
    pipeline; it keeps the recorded outputs and scratch buffers alive."""

    def __init__(self):
        self.launches = []      # (function, grid, lds bytes, packed arguments)
        self.keep = []
        self._scratch = []
        self._graph = None

    def __call__(self):
        if self._graph is not None:
            self._graph.launch()
            return
        for func, grid, lds, args in self.launches:
            hiprt.launch(func, grid, cg.BLOCK, lds, args, len(args))

    def as_graph(self):
        """Capture the recorded launches into a HIP graph; later calls replay the
        whole sequence with a single launch."""
        if self._graph is None and self.launches:
            hiprt.Graph.begin()
            try:
                for func, grid, lds, args in self.launches:
                    hiprt.launch(func, grid, cg.BLOCK, lds, args, len(args))
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
        _RECORDING = None
        return False


_STAMP = 0            # bumped whenever tunables or the fusion mode change
_RECENT = collections.deque(maxlen=int(os.environ.get("DELAYREPAY_KEEP", "16")))


def forget():
    """Drop the recently evaluated roots kept alive for plan reuse."""
    _RECENT.clear()


class Plan:
    """Everything needed to launch an evaluated expression again: the lowered
    kernel choice, the leaves it reads, the shape and dtypes it produces.

    A plan is cached on the root node, and the last few evaluated roots are kept
    alive, so re-building the same expression over the same arrays (the body of an
    iterative loop) finds its nodes in the hash-cons table and its plan here: no
    tracing, no layout analysis, no cache-key hashing, only an argument pack and a
    launch.  `valid()` re-checks what could have changed underneath."""

    __slots__ = ("low", "kern", "checks", "stamp", "shape", "out_dtypes", "acc", "leaves",
                 "hazard", "region", "empty", "axes")

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

    def deps(self):
        seen = {}
        for arr in self.leaves:
            seen[id(arr.buf)] = arr.buf
        return tuple((buf, buf.version) for buf in seen.values())


def _fire(plan, out_ptrs, reduce_out=None):
    """Compile on first use, pack the argument block, launch."""
    low = plan.low
    kern = plan.kern
    if kern is None:
        kern = plan.kern = _kernel_for(low, reduce_out is not None)
    ptrs = [buf.ptr + off for buf, off in low.srcs]
    if reduce_out is not None:
        partial = hiprt.malloc(low.fin_count * cg.ITEMSIZE[plan.acc])
        args = kern.packer.pack(*ptrs, partial, *low.scal, *low.tail)
        hiprt.launch(kern.func, low.grid, cg.BLOCK, 0, args, len(args))
        fin = struct.pack("@PPi", partial, reduce_out, low.fin_count)
        hiprt.launch(kern.finalize, 1, cg.BLOCK, 0, fin, len(fin))
        if _RECORDING is not None:
            _RECORDING.launches += [(kern.func, low.grid, 0, args), (kern.finalize, 1, 0, fin)]
            _RECORDING._scratch.append(partial)
        else:
            hiprt.free(partial)  # stream-ordered: safe to recycle once queued
        STATS["launches"] += 2
    else:
        args = kern.packer.pack(*ptrs, *out_ptrs, *low.scal, *low.tail)
        hiprt.launch(kern.func, low.grid, cg.BLOCK, 0, args, len(args))
        if _RECORDING is not None:
            _RECORDING.launches.append((kern.func, low.grid, 0, args))
        STATS["launches"] += 1


# ---------------------------------------------------------------------------
# evaluation entry points
# ---------------------------------------------------------------------------

def _make_plan(tracer, roots, dst=None, reduce_op=None, dry=False, axes=None):
    """Lower traced `roots` (list of (ref, code)) into a Plan.  `dst`: existing
    destination view (single root); `dry`: placeholders instead of device memory."""
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
    if reduce_op:
        shape = tuple(numpy.broadcast_shapes(*[a.shape for a in leaves])) if leaves else ()
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
            plan.low = _lower_axis_reduce(prog, leaves, tracer.scalars, shape, axes, plan.acc,
                                          reduce_op)
            return plan
        plan.shape = ()
        if 0 in shape:
            if reduce_op != "add":
                raise ValueError(f"zero-size array to reduction operation {reduce_op} "
                                 "which has no identity")
            plan.empty = True
            plan.low = None
            return plan
        plan.low = _lower(prog, leaves, tracer.scalars, shape, [plan.acc], [], [], reduce_op)
        return plan
    if dst is None:
        shape = tuple(numpy.broadcast_shapes(*[a.shape for a in leaves])) if leaves else ()
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
    plan.low = _lower(prog, leaves, tracer.scalars, shape, out_codes, out_ptrs, out_strides, None,
                      in_place)
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
        outs = [ndarray(plan.shape, dt) for dt in plan.out_dtypes]
        if not plan.empty:
            _fire(plan, [o.ptr for o in outs])
    if _RECORDING is not None:
        _RECORDING.keep += outs + plan.leaves
    return outs


def _trace_root(tracer, node):
    if _FE is None:
        _bind_frontend()
    if type(node) is _FE.ReduceEx and "array" not in node.__dict__:
        raise TypeError("a reduction must be the root of its own evaluation")
    return tracer.visit(node)


def _run_unfused(ex, evaluated):
    """One kernel per interior node, children first."""
    from .delayarray import NPArray, Scalar, ReduceEx
    nid = id(ex)
    if nid in evaluated:
        return evaluated[nid]
    if isinstance(ex, NPArray):
        return ex.array
    for child in ex.children:
        if not isinstance(child, (Scalar, NPArray)):
            _run_unfused(child, evaluated)
    tracer = Tracer(evaluated)
    if isinstance(ex, ReduceEx):
        root = tracer.visit(ex.children[0])
        out = _launch_fresh(_make_plan(tracer, [root], reduce_op=ex.func.__name__,
                                       axes=ex.axis))[0]
    else:
        root = tracer.visit(ex)
        out = _launch_fresh(_make_plan(tracer, [root]))[0]
    evaluated[nid] = out
    return out


def run(ex):
    """Evaluate one DAG root; returns a new device array owned by the caller
    (cf. cuda.py:91-96)."""
    if not _FUSED:
        return _run_unfused(ex, {})
    d = ex.__dict__
    plan = d.get("_plan")
    if plan is None or not plan.valid():
        if _FE is None:
            _bind_frontend()
        tracer = Tracer()
        if type(ex) is _FE.ReduceEx:
            root = tracer.visit(ex.children[0])
            plan = _make_plan(tracer, [root], reduce_op=ex.func.__name__, axes=ex.axis)
        else:
            root = _trace_root(tracer, ex)
            plan = _make_plan(tracer, [root])
        d["_plan"] = plan
        _RECENT.append(ex)
    else:
        STATS["plan_hits"] += 1
    out = _launch_fresh(plan)[0]
    d["_deps"] = plan.deps()
    return out


def run_multi(exs):
    """Evaluate several roots; roots of equal shape share one kernel (and their
    common sub-expressions)."""
    if not _FUSED:
        return [run(ex) for ex in exs]
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
            tracer = Tracer()
            roots = [_trace_root(tracer, exs[i]) for i in idxs]
            plan = _make_plan(tracer, roots)
            first["_multi"] = (key, plan, [exs[i] for i in idxs])
            _RECENT.append(exs[idxs[0]])
        outs = _launch_fresh(plan)
        deps = plan.deps()
        for i, out in zip(idxs, outs):
            if out.shape != shape:   # every leaf of this root was a broadcast scalar
                out = materialise(out, shape=shape)
            results[i] = out
            exs[i].__dict__["_deps"] = deps
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


def run_into(ex, dst):
    """`dst[...] = ex` as one fused kernel writing the destination view directly."""
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
        tracer = Tracer()
        root = _trace_root(tracer, ex)
        plan = _plan_write(tracer, root, dst)
        d["_into"] = (key, plan, dst.buf)     # holding the buffer keeps its id unique
        _RECENT.append(ex)
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
    from .delayarray import ReduceEx
    if not isinstance(exs, (list, tuple)):
        exs = [exs]
    tracer = Tracer()
    if isinstance(exs[0], ReduceEx):
        root = tracer.visit(exs[0].children[0])
        low = _make_plan(tracer, [root], reduce_op=exs[0].func.__name__, axes=exs[0].axis).low
    elif dst is not None:
        low = _plan_write(tracer, tracer.visit(exs[0]), dst).low
    else:
        low = _make_plan(tracer, [tracer.visit(ex) for ex in exs]).low
    return low, _source(low)[0]


def compile_source(source):
    """hiprtc-compile generated source without loading it (no GPU needed)."""
    return hiprt.compile_only(source, "dr_kernel.hip", COMPILE_OPTS)


# ---------------------------------------------------------------------------
# `np` and `fallback` namespaces of the backend protocol
# ---------------------------------------------------------------------------

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

sys.modules[__name__].np = np
