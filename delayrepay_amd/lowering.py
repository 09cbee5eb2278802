"""Layout analysis and kernel choice of the HIP backend.

Given a traced `Program` and the geometry of its operands, decide which kernel
shape evaluates it (`flat`, `tile2d`/`tile2dv`, `tile3d`, `tile2dt`, `nd`, the `axis_*`
family), build the cache key
(program + layout classes + dtypes + the tunables that shape the source), and
prepare the launch recipe: grid, argument-block format, pointer sources and the
constant tail of the argument block.  The reference has no counterpart: CuPy's
ElementwiseKernel does its own (contiguous-or-generic) indexing (cuda.py:35-43).
"""
import os

from . import codegen as cg
from . import mathlib
from . import hiprt

# Tunables; part of every cache key.  DELAYREPAY_TUNE="unroll=2,bpc=16" overrides.
TUNE = {
    "unroll": 0,      # 16-byte vectors per thread and chunk in flat element-wise kernels
                      # (0: by the number of streams, see `lower`)
    "red_unroll": 0,  # the same for flat kernels with a reduction tail } 0: see `lower`
    "red_blocks": 0,  # most blocks (= partial results) of a reduction kernel }
    "static_scratch": 1,  # partial results go to the library's static scratch array if they fit
    "flat_cap": 0,    # most blocks of a flat element-wise kernel (0: one chunk per block)
    "bpc": 8,         # resident blocks per CU that bound the grid of `nd` kernels
    "ax_blocks": 4096,   # axis reductions: blocks ('col') / waves ('row') worth of work to
    "ax_waves": 32768,   # aim for before the reduced extent is cut into slices
    "ax_rows": 4,        # 'row' strategy: outputs per wave (grid-stride), to amortise set-up
    "ax_narrow": 128,    # kept unit-stride extents up to this many columns: stream the matrix
                         # (sum over the rows, float32, percent of the HBM peak, a lane per column /
                         # the stream: 96 columns 52 / 68, 128: 64 / 71, 200: 52 / 51, 256: 64 / 56)
    "ax_short": 28,      # reduced unit-stride extents up to this length: a lane per output
    "ax_group": 2048,    # ... and up to this length: a group of 8 to 64 lanes per output
    "ax_group_lanes": 0,  # force the group size (0: the one that wastes the fewest unit slots)
    "ax_group_steps": 8,  # most 16-byte units a lane of such a group takes from its row
    "ax_slices": 512,    # most slices (the second pass walks them serially per output)
    "ax_block": 4096,    # reduced unit-stride extents from this length: a block per row slice
    "ax_block_rows": 2,  # ... and this many rows per block when an operand is the same for all
    "ax_block_rows_unroll": 2,   # ... with this many steps in flight
    "ax_stream": 256,    # kept unit-stride extents of 256 vectors or more: blocks to aim for, one
                         # per compute unit (0: off)
    "ax_stream_unroll": 8,   # ... and rows in flight per lane
    "ax_stream_stagger": 1,  # ... and blocks start at different rows of their slices
    "ntl": 1,         # allow non-temporal loads  } see the cache policy in `lower`
    "nts": 1,         # allow non-temporal stores }
    "cache_mib": 32,  # working sets up to this size (the eight L2s together) stay cacheable
    "ntl_mib": 32,    # inputs beyond this size are read with non-temporal loads
    "tw": 128,        # stencil tile width (elements)
    "th": 16,         # stencil tile height (rows)
    "lds": 1,         # stage shifted views through LDS (0: read them directly)
    "svec": 1,        # aligned stencils: 16-byte loads into LDS and 16-byte stores
    "row1d": 1,       # shifted views of one vector: tiled as a matrix of one row
    "gpr": 64,        # vectorised stencil: 16-byte column groups per tile row
    "rpt": 2,         # vectorised stencil: consecutive rows per thread
    "row_gpr": 256,   # vector tiles without a halo group: most column groups per block (0: as
                      # the stencil tiles)
    "xcd": 1,         # vector tiles: a contiguous band of tiles per XCD (1: with a halo group
                      # or unaligned rows, 2: always, 0: never)
    "sntl": 0,        # vectorised stencil: non-temporal loads / stores
    "snts": 1,
    "s3": 1,          # 3-D shifted views of one buffer: LDS window (0: read every view directly)
    "s3_gpr": 64,     # 3-D window: 16-byte column groups per tile row (tile rows = 256 / s3_gpr)
    "s3_rpt": 2,      # 3-D window: tile rows per thread (tile rows = s3_rpt * 256 / s3_gpr)
    "s3_zc": 0,       # 3-D window: planes a block walks; 0 = fewest rounds of resident blocks
    "s3_depth": 1,    # 3-D window: planes in flight in registers
    "uvec": 1,        # 16-byte accesses at element alignment where 16-byte alignment is missing
    "tvec": 1,        # transpose tiles: 16-byte global accesses where alignment allows
    "t_rows": 0,      # transpose tiles: output rows (= contiguous elements of the operand) and
    "t_cols": 0,      # output columns per tile (powers of two; 0: 128 bytes by 1 KB)
    "dmath": 1,       # float64 log/erf from `mathlib` (0: the device library's)
    "softdiv": 2,     # quotients and square roots that only inexact functions read: to one ulp, in
                      # fewer operations (1: float64 only, 2: float32 too, in packed bodies; 0: never)
                      # (2: float32 quotients as well, 4 operations; measured slower)
    "rows_stencil": 384,      # ... shifted views of one matrix among them: rows of at most this many bytes
                      # (5-point stencil, float32, tiled / row kernel: rows of 16: 10 / 36 % of the
                      # HBM peak, of 64: 28 / 40, of 128: 46 / 42, of 256: 66 / 44)
    "rows_elem": 4096,    # element-wise work on rows of at most this many bytes with repeated
                      # operands takes the row kernel (0: the tiled kernel)
    "rowfuse": 1,     # reductions along the last axis inside an expression: one kernel per row
    "row_lanes": 0,   # ... lanes per row (0: by the cost of idle lanes and of units per lane)
    "row_regs": 128,  # ... registers that may hold the row between stages (else it is loaded again)
    "row_wavemap": -1,    # ... each wave of a block takes a quarter of the row (-1: rows of 48 KB up)
    "row_hoist": 1,   # ... values that are the same along a row are computed once per row
    "row_carry": 1,   # ... a costly value read by later stages takes its operand's registers
    "row_pipe": 1,    # ... the next row is loaded while this one is finished and stored
    "row_fence": 1,   # ... the compiler keeps the work of one 16-byte unit together
    "row_recompute": 1,   # ... per-element values are computed again by each stage, not kept
    "row_bpc": 0,     # ... blocks per compute unit at most (0: one pass, a block per set of rows)
    "strided": 1,     # every k-th element of a vector: the flat kernel (0: the general one)
    "table_runs": 1,  # ... and takes this many adjacent runs, one after the other
    "row_ntl": 1,     # row kernels read the operands they keep in registers past the caches
    "xch": 1,         # a lane's adjacent output vectors change lanes through LDS before the store
    "stage_loop": 0,  # ... 1: the tables are copied by a loop (one trip to memory per 4 KB)
    "one_run": 1,     # flat kernels with tables in LDS: one run per block, no loop over runs
    "table_blocks": 4096,  # most workgroups of a flat kernel whose functions keep tables in LDS
    "smath": 1,       # float32 log/erf/exp from `mathlib32` (0: the device library's)
    "pack": 4,        # elements a thread passes through those functions in lock step
    "pack32": 8,      # ... a float32 body with short divisions or square roots
}
for _kv in filter(None, os.environ.get("DELAYREPAY_TUNE", "").split(",")):
    _k, _v = _kv.split("=")
    TUNE[_k.strip()] = int(_v)

_SCALAR_FMT = {"f4": "f", "f8": "d", "i4": "i", "i8": "q", "u4": "I", "u1": "B", "b1": "B"}

# ---------------------------------------------------------------------------
# layout analysis
# ---------------------------------------------------------------------------

def broadcast_strides(arr, shape):
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


def merge_dims(shape, stride_sets):
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

    __slots__ = ("key", "kind", "emit", "fmt", "srcs", "scal", "tail", "grid", "fin_count", "lds",
                 "recipe", "row_out")


# ---------------------------------------------------------------------------
# lowering
# ---------------------------------------------------------------------------

_CUS = None


def grid_cap():
    """Blocks that fill the device `bpc` deep (256 CUs assumed until a device is open)."""
    global _CUS
    if _CUS is None:
        if not hiprt._initialised:
            return 256 * TUNE["bpc"]
        _CUS = hiprt.device_info()["compute_units"]
    return _CUS * TUNE["bpc"]


def _lower_stencil3d(low, prog, leaves, m_leaf, m_out, mshape, out_codes, out_ptrs, scal_fmt,
                     scal_vals, in_place):
    """3-D expression with >= 2 operands that are shifted views of one buffer: stage the
    buffer's window in LDS (`codegen.emit_stencil3d`).  Returns None when the layout does
    not qualify (the general tiled kernel then reads every view directly)."""
    groups = {}
    for i, (a, s) in enumerate(zip(leaves, m_leaf)):
        if s[2] == 1 and s[0] > 0 and s[1] > 0:
            groups.setdefault((id(a.buf), s[0], s[1], prog.leaves[i]), []).append(i)
    best = max(groups.values(), key=len) if groups else []
    if len(best) < 2 or not out_codes:
        return None
    gcode = prog.leaves[best[0]]
    gsize = cg.ITEMSIZE[gcode]
    if gsize not in (4, 8) or gcode not in cg.VEC16:
        return None
    vw = 16 // gsize
    pz, py = m_leaf[best[0]][0], m_leaf[best[0]][1]
    aligned = (all(cg.ITEMSIZE[c] == gsize for c in out_codes)
               and all(st % vw == 0 for st_ in m_out for st in st_[:-1])
               and len({(p // gsize) % vw for p in out_ptrs}) == 1
               and all(p % gsize == 0 for p in out_ptrs)
               and pz % vw == 0 and py % vw == 0)
    if not aligned:
        return None
    def shifts_of(members):
        ref = min(leaves[i].offset for i in members)
        out = {}
        for i in members:
            d = leaves[i].offset - ref
            dz, r = divmod(d, pz)
            if r > pz // 2:
                dz, r = dz + 1, r - pz
            dy, dx = divmod(r, py)
            if dx > py // 2:
                dy, dx = dy + 1, dx - py
            if dz * pz + dy * py + dx != d:
                return ref, None
            out[i] = (dz, dy, dx)
        return ref, out

    ref_off, shifts = shifts_of(best)
    if shifts is None:
        return None
    dz_max = max(v[0] for v in shifts.values())
    dy_min, dy_max = min(v[1] for v in shifts.values()), max(v[1] for v in shifts.values())
    dx_min, dx_max = min(v[2] for v in shifts.values()), max(v[2] for v in shifts.values())
    if min(v[0] for v in shifts.values()) < 0 or dz_max > 4 or dy_max - dy_min > 8 \
            or dx_max - dx_min > 16:
        return None
    gpr, rpt, zc, depth = TUNE["s3_gpr"], TUNE["s3_rpt"], TUNE["s3_zc"], TUNE["s3_depth"]
    ty = cg.BLOCK // gpr * rpt
    Z, Y, W = mshape
    g_buf = leaves[best[0]].buf
    g_ptr = g_buf.ptr + ref_off * gsize
    ph_o = (out_ptrs[0] // gsize) % vw
    ph_g = (g_ptr // gsize) % vw
    # first and last aligned 16-byte vector inside the buffer, relative to the group pointer
    v_lo = -ref_off + (ref_off - ph_g) % vw
    v_hi = g_buf.nbytes // gsize - ref_off - vw
    v_hi -= (v_hi + ph_g) % vw
    if v_hi < v_lo:
        return None
    kinds = []
    for i, st in enumerate(m_leaf):
        if i in shifts:
            kinds.append(("g",) + shifts[i])
        elif not any(st):
            kinds.append(("b",))
        elif st[-1] == 1:
            dv = (cg.ITEMSIZE[prog.leaves[i]] == gsize and st[0] % vw == 0 and st[1] % vw == 0
                  and (leaves[i].ptr // gsize) % vw == ph_o)
            kinds.append(("dv",) if dv else ("d",))
        else:
            kinds.append(("r",))
    kinds = tuple(kinds)
    group = (gcode, dz_max, dy_min, dy_max, dx_min, dx_max)
    lds_bytes = cg.emit_stencil3d(prog, kinds, group, out_codes, gpr, rpt, ph_g, ph_o)[4]
    tiles_x = -(-(W + ph_o) // (gpr * vw))
    tiles_y = -(-Y // ty)
    if zc <= 0:
        # Blocks walk their planes in step, so what counts is how many rounds of resident
        # blocks the grid takes and how long a round is: planes walked plus the planes
        # fetched before the first output.
        slots = grid_cap() // TUNE["bpc"] * max(1, min(8, (160 * 1024) // max(lds_bytes, 1)))
        best = None
        for chunks in range(1, max(1, Z // 8) + 1):
            c = -(-Z // chunks)
            rounds = -(-(tiles_x * tiles_y * -(-Z // c)) // slots)
            cost = rounds * (c + dz_max + 2)
            if best is None or cost < best[0]:
                best = (cost, c)
        zc = best[1]
    tiles_z = -(-Z // zc)
    if lds_bytes > 64 * 1024 or tiles_x * tiles_y * tiles_z >= 2 ** 31 or max(Z, Y, W) >= 2 ** 31 - 4096:
        return None
    snts = bool(TUNE["snts"])
    bands = TUNE["xcd"] != 0
    low.kind = "tile3d"
    low.key = ("tile3d", prog.key(), kinds, group, tuple(out_codes), in_place, ph_g, ph_o, gpr, rpt,
               snts, bands, depth)

    def emit():
        return cg.emit_stencil3d(prog, kinds, group, out_codes, gpr, rpt, ph_g, ph_o,
                                 restrict=not in_place, nt_store=snts, xcd_bands=bands, depth=depth)[0]
    low.emit = emit
    low.grid = tiles_x * tiles_y * tiles_z
    srcs = [(a.buf, a.offset * a.dtype.itemsize) for a, k in zip(leaves, kinds) if k[0] != "g"]
    srcs.append((g_buf, ref_off * gsize))
    fmt = "@" + "P" * (len(srcs) + len(out_ptrs)) + scal_fmt + "iii" + "qqqq" + "iii"
    tail = [Z, Y, W, pz, py, v_lo, v_hi, tiles_x, tiles_y, zc]
    for k, st in zip(kinds, m_leaf):
        if k[0] in ("d", "dv", "r"):
            fmt += "qq"
            tail += [st[0], st[1]]
    for st in m_out:
        fmt += "qq"
        tail += [st[0], st[1]]
    low.fmt = fmt
    low.srcs, low.scal, low.tail = srcs, scal_vals, tail
    return low


def _row_lanes(prog, leaves, kinds, sk, out_codes, row_out, R, V, uniform=None):
    """Lanes per row for the row kernel: the candidate with the least estimated time per
    row.  The estimate has a memory term and an arithmetic term, fitted to measurements on
    MI355X (`a - max(a)` and softmax, float32 and float64, rows of 16 to 4096 elements,
    every candidate; the choice is within 2 points of the best candidate in all but one of
    those 38 cases):

    memory      a wave's load covers `min(lanes, units) * 16` contiguous bytes of a row.  Rows
                whose pitch is no multiple of 128 bytes start inside a cache line, so a short
                stretch touches one line more than it fills (rows of 300 float32, percent of
                the HBM peak with 8 / 16 / 32 / 64 lanes: 44 / 62 / 68 / 77), and a stretch
                below 128 bytes never fills the line it touches (rows of 32 float32 with 2
                lanes of 4 units each: 23); more than four units per lane cost a little, and
                so does a single one;
    arithmetic  idle lanes of the last step and the butterfly (log2 lanes steps per
                reduction, spread over a lane's units) take issue slots that the body needs:
                softmax on rows of 128 float32 with 8 / 16 / 32 lanes: 77 / 75 / 66, on rows
                of 300 with 16 / 32 / 64 lanes: 57 / 68 / 59.
    A block per row pays only from 512 units on (rows of 1024 float32: 64 lanes 79 / 78,
    a block 76 / 63)."""
    units = -(-R // V)
    pitches = [st * a.dtype.itemsize for a, k, st in zip(leaves, kinds, sk) if k == "v" and st]
    pitches += [R * cg.ITEMSIZE[c] for c, u in zip(out_codes, row_out) if not u]
    extra = 0 if all(p % 128 == 0 for p in pitches) else 32 if all(p % 64 == 0 for p in pitches) else 96
    dense = all(st == R for k, st in zip(kinds, sk) if k == "v" and st)
    moved = sum(a.dtype.itemsize for a, k, st in zip(leaves, kinds, sk) if k == "v" and st) \
        + sum(cg.ITEMSIZE[c] for c, u in zip(out_codes, row_out) if not u)
    # per element: what is the same along the row is computed once per row
    work = sum(10 if (name in cg._FLOAT_FUNCS1 or name in cg._FLOAT_FUNCS2 or name in
                      ("divide", "true_divide", "reciprocal")) else 1
               for i, (name, _, _, _) in enumerate(prog.ops)
               if uniform is None or not uniform[i] or name in cg.ROW_REDUCE)
    if any(cdt == "f8" for _, cdt, _, _ in prog.ops):
        work *= 2
    ratio = 0.26 * work / max(moved, 1)
    best = None
    for lanes in (1, 2, 4, 8, 16, 32, 64, cg.BLOCK):
        n = -(-units // lanes)
        if n > cg.ROW_STEPS_MAX:
            continue
        # what one load of a wave covers without a gap: a lane group's stretch of its row
        # or, with one unit per lane and rows that follow each other, the wave's 1 KB
        piece = 1024 if n == 1 and dense else min(lanes, units) * 16
        t_mem = max(128, piece + extra) / piece / (0.95 if n == 1 else 1.0 if n <= 4 else 0.97 if n <= 8 else 0.88)
        butterfly = 8 if lanes == cg.BLOCK else lanes.bit_length() - 1
        t_alu = ratio * lanes * n / units * (1 + 0.15 * butterfly / n)
        t = max(t_mem, t_alu) + 0.25 * min(t_mem, t_alu)
        if best is None or t < best[0]:
            best = (t, lanes)
    if best is None and -(-units // cg.ROW_BLOCKS[-1]) <= cg.ROW_STEPS_LONG:
        return cg.ROW_BLOCKS[-1]        # longer than 256 lanes hold: a block of 512
    return best[1] if best else cg.BLOCK


# Transposes of a matrix with one side of at most this many elements take a lane per index of
# the long side (`codegen.emit_thin_transpose`) when that side is no power of two; powers of
# two have tiles that fit them and move 16 bytes per lane.
THIN_TRANSPOSE = 16
THIN_TRANSPOSE_ALL = False


def block_lanes(low):
    """Lanes per block that the kernel of `low` is launched with: `codegen.BLOCK`, except
    for a row kernel whose block of 512 lanes holds one long row (read from the cache key,
    which every copy of a lowering carries)."""
    if low.kind == "rows" and low.key[6] > cg.BLOCK:
        return low.key[6]
    return cg.BLOCK


def _row_steps_max(G):
    """Units a lane may hold of one operand's row."""
    return cg.ROW_STEPS_LONG if G > cg.BLOCK else cg.ROW_STEPS_MAX


def lower_rows(prog, leaves, scalars, shape, out_codes, whole_rows=False, out_strides=None,
               in_place=False, leaf_strides=None):
    """Expression with reductions along its last axis inside it (`codegen.emit_row_fused`):
    every row is read once, reduced, used again and written once.  `shape` is the shape the
    expression is evaluated at, rows along its last axis; outputs are new dense arrays, of
    that shape or, for roots that are constant along the row, with a last axis of one.
    Raises `codegen.RowFusionUnsupported` for layouts the kernel does not take: the caller
    then evaluates the reductions on their own."""
    if not TUNE["rowfuse"] or len(shape) < 2 or shape[-1] < 2:
        raise cg.RowFusionUnsupported("not a matrix of rows")
    R = shape[-1]
    # (`leaf_strides`: the operands' strides at `shape` where the caller has merged
    # dimensions already, so that a row is the longest run every operand walks as one)
    strides = [list(st) for st in leaf_strides] if leaf_strides is not None \
        else [broadcast_strides(a, shape) for a in leaves]
    kinds = []
    for st in strides:
        if st[-1] not in (0, 1):
            raise cg.RowFusionUnsupported("an operand without unit stride along the row")
        kinds.append("v" if st[-1] == 1 else "k")
    dense = [1] * len(shape)             # a new array of `shape`
    for k in range(len(shape) - 2, -1, -1):
        dense[k] = dense[k + 1] * shape[k + 1]
    # the results: new dense arrays, or (element-wise work written into existing arrays)
    # views whose rows lie one pitch apart
    outs = [dense] * len(out_codes) if out_strides is None else [list(st) for st in out_strides]
    if any(st[-1] != 1 for st in outs if shape[-1] > 1):
        raise cg.RowFusionUnsupported("a destination without unit stride along the row")
    mshape, msets = merge_dims(shape[:-1], [st[:-1] for st in strides] + [st[:-1] for st in outs])
    nl_ = len(strides)
    if len(mshape) == 2 and any(st[0] != st[1] * mshape[1] for st in msets[nl_:]):
        raise cg.RowFusionUnsupported("a destination whose rows do not form one sequence")
    sj = None
    if len(mshape) == 2 and mshape[0] * mshape[1] < 2 ** 31:
        # two levels of rows (a matrix added to every item of a batch before the rows are
        # normalised): the kernel splits the row number
        K, K1 = mshape[0] * mshape[1], mshape[1]
        sk = [st[0] for st in msets[:nl_]]
        sj = [st[1] for st in msets[:nl_]]
        so = [st[1] for st in msets[nl_:]]
    elif len(mshape) > 1:
        raise cg.RowFusionUnsupported("rows that do not form one sequence in every operand")
    else:
        K = mshape[0] if mshape else 1
        sk = [st[0] if st else 0 for st in msets[:nl_]]
        so = [st[0] if st else R for st in msets[nl_:]]
    level, uniform, stages = cg.row_analysis(prog, kinds)
    row_out = []
    for (kind, j), _ in prog.roots:
        row_out.append(uniform[j] if kind == "v" else (kind == "s" or kinds[j] == "k"))
    if whole_rows and any(row_out):
        # the caller's results all have the full shape: one that is the same along a row
        # (a column repeated) would be stored once per row here
        raise cg.RowFusionUnsupported("a result that is constant along the rows")
    V = cg.row_vector(prog, kinds, out_codes, row_out)
    units = -(-R // V)
    G = TUNE["row_lanes"]
    if not G:
        G = _row_lanes(prog, leaves, kinds, [b or a for a, b in zip(sk, sj)] if sj else sk,
                       out_codes, row_out, R, V,
                       uniform if TUNE["row_hoist"] else None)
    steps = -(-units // G)
    if steps > _row_steps_max(G) or K >= 2 ** 40:
        raise cg.RowFusionUnsupported("row too long")
    # An operand's share of its row stays in registers between the stages, as long as all
    # of them fit; operands that are the same for every row (a vector of weights) come from
    # the caches every time.
    own = [k == "v" and (st != 0 or (sj is not None and sj[i] != 0))
           for i, (k, st) in enumerate(zip(kinds, sk))]
    keep = tuple(o and steps * 4 * sum(own) <= TUNE["row_regs"] for o in own)
    footprint = sum(a.nbytes for a in leaves) + sum(K * (1 if u else R) * cg.ITEMSIZE[c]
                                                   for c, u in zip(out_codes, row_out))
    nts = bool(TUNE["nts"]) and footprint > TUNE["cache_mib"] << 20
    ntl = bool(TUNE["ntl"]) and bool(TUNE["row_ntl"]) and sum(a.nbytes for a in leaves) > TUNE["ntl_mib"] << 20
    low = Lowered()
    low.lds = 0
    low.fin_count = 0
    low.kind = "rows"
    low.row_out = tuple(row_out)
    fence, recompute, pipe = bool(TUNE["row_fence"]), bool(TUNE["row_recompute"]), bool(TUNE["row_pipe"])
    carry = bool(TUNE["row_carry"])
    wmap = G >= cg.BLOCK and (steps >= 12 if TUNE["row_wavemap"] < 0 else bool(TUNE["row_wavemap"]))
    hoist = bool(TUNE["row_hoist"])
    low.key = ("rows", prog.key(), tuple(kinds), tuple(out_codes), low.row_out, R, G, keep, nts,
               fence, recompute, pipe, carry, wmap, ntl) + (() if hoist else ("per element",)) \
        + (("two levels",) if sj else ()) + (("over an operand",) if in_place else ())

    def emit():
        return cg.emit_row_fused(prog, kinds, out_codes, row_out, R, G, keep=keep, nt_store=nts,
                                 fence=fence, recompute=recompute, pipeline=pipe, carry_values=carry,
                                 wave_map=wmap, nt_load=ntl, hoist=hoist, outer2=bool(sj),
                                 restrict=not in_place)
    low.emit = emit
    if G >= cg.BLOCK:
        blocks = K
    else:
        blocks = -(-K // (cg.BLOCK // G))
    # One pass: every block takes its rows and ends.  Blocks that stay and stride through
    # the matrix are slower here as they are for flat kernels (`a - max(a, axis=1)` float32,
    # percent of the HBM peak, 2048 blocks that stay / one pass: rows of 64: 67 / 79, of
    # 200: 62 / 74, of 1000: 63 / 80, of 4096: 69 / 72, of 16384: 70 / 71).
    cap = grid_cap() * TUNE["row_bpc"] // max(TUNE["bpc"], 1) if TUNE["row_bpc"] else (1 << 24) - 1
    low.grid = max(1, min(blocks, cap))
    low.fmt = "@" + "P" * (len(leaves) + len(out_codes)) + "".join(_SCALAR_FMT[c] for c in prog.scalars) \
        + "q" * (1 + len(leaves) + len(out_codes)) + ("I" + "q" * len(leaves) if sj else "")
    low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
    low.scal = list(scalars)
    low.tail = [K] + sk + [1 if u else p for u, p in zip(row_out, so)] + ([K1] + sj if sj else [])
    return low


def lower(prog, leaves, scalars, out_shape, out_codes, out_ptrs, out_strides, reduce_op,
           in_place=False):
    """Pick the kernel shape.  `out_ptrs`/`out_strides` describe the destinations
    (element strides at `out_shape`); for a reduction they are empty and the
    partial-sums pointer is appended at launch."""
    if any(name in cg.ROW_REDUCE for name, _, _, _ in prog.ops):
        if reduce_op or in_place or any(p for p in out_ptrs):
            raise cg.RowFusionUnsupported("row reductions inside a write or a reduction over everything")
        return lower_rows(prog, leaves, scalars, tuple(out_shape), out_codes)
    n = 1
    for d in out_shape:
        n *= d
    leaf_strides = [broadcast_strides(a, out_shape) for a in leaves]
    mshape, msets = merge_dims(out_shape, leaf_strides + list(out_strides))
    m_leaf, m_out = msets[:len(leaves)], msets[len(leaves):]
    ndim = len(mshape)
    low = Lowered()
    low.lds = 0
    low.fin_count = 0
    scal_fmt = "".join(_SCALAR_FMT[c] for c in prog.scalars)
    scal_vals = list(scalars)

    flat = ndim <= 1 and all(s == [1] or s == [0] or s == [] for s in m_leaf) \
        and all(s == [1] or s == [] for s in m_out)
    if not flat and ndim == 1 and TUNE["strided"] and all(s == [1] for s in m_out) \
            and all(len(s) == 1 and (0 <= s[0] <= 1 or (s[0] == 2 and a.dtype.itemsize <= 4))
                    for a, s in zip(leaves, m_leaf)):
        # Every second element of a vector (`a[::2]`): the flat kernel with the two vectors
        # that hold a thread's elements loaded whole (x[::2] * 2, 2^26 float32 results: 129 us;
        # the general kernel, which computes an index per element and stores element by
        # element, 139).  From every third element on, two thirds and more of what such
        # vectors bring into the registers is thrown away and the general kernel, one
        # element per lane, is the faster one (x[::3] * 2: 126 us against 141 with vectors
        # and 170 with four element loads per thread).
        flat = True
    if flat and ndim == 1 and not reduce_op and TUNE["lds"] and TUNE["svec"] and TUNE["row1d"] \
            and 4096 <= n < 2 ** 31 - 4096:
        # Shifted views of one vector (differences, 1-D stencils): every view would fetch the
        # same cache lines again through L1.  As a matrix of one row the vector goes through
        # the tiled kernel's LDS window once.  Second difference of 2^27 float32: 65 % of the
        # HBM peak as a flat kernel.
        same = {}
        for a, st, c in zip(leaves, m_leaf, prog.leaves):
            if st == [1]:
                same.setdefault((id(a.buf), c), set()).add(a.offset)
        offs = max(same.values(), key=len) if same else set()
        if len(offs) >= 2 and max(offs) - min(offs) <= 32:
            flat = False
            ndim = 2
            far = 1 << 40               # the pitch of the one row: never multiplied by a row > 0
            mshape = [1] + list(mshape)
            m_leaf = [[far if st == [1] else 0] + list(st) for st in m_leaf]
            m_out = [[far] + list(st) for st in m_out]
    if ndim == 1 and not reduce_op and any(s == [-1] for s in m_leaf) \
            and all(s in ([1], [0], [-1]) for s in m_leaf) and all(s == [1] for s in m_out) \
            and n < 2 ** 31 - 4096:
        # a flipped vector: as a matrix of one row it takes the tiled kernel's reversed loads
        ndim = 2
        far = 1 << 40
        mshape = [1] + list(mshape)
        m_leaf = [[0 if st == [0] else far] + list(st) for st in m_leaf]
        m_out = [[far] + list(st) for st in m_out]
    if flat:
        leaf_class = tuple("b" if (s == [0] and n > 1) else f"s{s[0]}" if s and s[0] > 1 else "c"
                           for s in m_leaf)
        ptrs = [a.ptr for a in leaves]
        # bytes (masks) move as vectors of sixteen; the wider operands beside them then take
        # four or eight vectors per thread
        widths_ok = all(c in cg.VEC16 for c, k in zip(prog.leaves, leaf_class) if k != "b")
        align_ok = all(p % 16 == 0 for p, k in zip(ptrs, leaf_class) if k != "b")
        if not reduce_op:
            widths_ok = widths_ok and all(c in cg.VEC16 for c in out_codes)
            align_ok = align_ok and all(p % 16 == 0 for p in out_ptrs)
        vec = widths_ok and n >= 64 and (align_ok or bool(TUNE["uvec"]))
        ua = vec and not align_ok      # vectors at element alignment
        unroll = TUNE["red_unroll"] if reduce_op else TUNE["unroll"]
        red_cap = TUNE["red_blocks"]
        if reduce_op and not (unroll and red_cap):
            # A stream that is only read is fastest with one block per compute unit and six
            # to eight 16-byte loads in flight per lane.  sum((x-y)**2*w), float64, 2^27,
            # percent of the HBM peak: 4096 blocks x 4 vectors per operand 86.4; 256 blocks x
            # 1 / 2 / 3 vectors 65.8 / 89.3 / 86.6; 384 blocks 81.6; 128 blocks 72.3.  dot of
            # two operands: 256 blocks x 2 / 4 vectors 77.5 / 89.5.  A body with many
            # operations per element needs more waves than that to keep the vector unit busy.
            n_in = max(1, sum(c != "b" for c in leaf_class))
            cheap = {"floor", "ceil", "trunc", "rint", "copysign", "fmax", "fmin"}
            cost = sum(10 if (name in cg._FLOAT_FUNCS1 or name in cg._FLOAT_FUNCS2 or name in
                              ("divide", "true_divide", "reciprocal")) and name not in cheap else 1
                       for name, _, _, _ in prog.ops)
            light = cost <= 4 * n_in + 4
            # one operand: 6 vectors in flight 89.9, 8: 87.1, 4: 75.3.  That holds for float
            # sums of at most one operation per operand.  With one wave per SIMD nothing hides
            # the arithmetic between two batches of loads, so maxima and minima (NaN checks
            # per element), counts of masks (64-bit integer sums) and longer bodies want two
            # blocks per compute unit with half as many vectors each.  One float32 operand,
            # 2^27, 256 x 6 against 512 x 3: max 75.7 / 87.9, count(a > c) 64.9 / 87.4,
            # count((a > c) & (a < d)) 46.5 / 86.1, sum(a*a*a + a) 83.6 / 88.2,
            # sum(where(a > c, a, 0)) 81.5 / 88.4, sum(abs(a)) 86.6 / 87.6.
            per_lane = {1: 6, 2: 4, 3: 2, 4: 2}.get(n_in, 1)
            cus = grid_cap() // TUNE["bpc"]
            bare = (reduce_op == "add" and len(prog.ops) <= n_in
                    and all(c in ("f4", "f8") for c in out_codes))
            if light and not bare:
                per_lane, cus = max(1, per_lane // 2 + per_lane % 2), 2 * cus
            unroll = unroll or (per_lane if light else 4)
            red_cap = red_cap or (cus if light else 4096)
        packed = bool(cg.packs(prog, vec) and TUNE["pack"])
        if not unroll and packed:
            unroll = 1          # the pack below decides
        elif not unroll:
            # More streams want more vectors in flight per thread.  Percent of the HBM peak
            # with 1 / 2 / 4 vectors: one load and one store (Horner) 81.4 / 80.0 / 79.9; two
            # loads and one store (SAXPY, 2^24) 76.3 / 78.9 / 78.8; three float64 loads and
            # two stores with a trivial body 75.0 / 77.6 / 78.8, with Black-Scholes' float32
            # body 73.2 / 73.5 / 71.7.
            streams = sum(c != "b" for c in leaf_class) + len(out_codes)
            unroll = 1 if streams <= 2 else 2
        if packed:
            # float64 functions evaluate a pack of elements in lock step: at least `pack`
            # elements per thread (a vector of doubles holds two)
            size = TUNE["pack"] if prog.own_math or not any(prog.ops[i][1] == "f4" for i in prog.soft_div) \
                else TUNE["pack32"]
            unroll = max(unroll, size // cg.flat_elements(prog, leaf_class, out_codes, reduce_op))
        in_bytes = sum(a.nbytes for a, k in zip(leaves, leaf_class) if k != "b")
        footprint = in_bytes
        if not reduce_op:
            footprint += sum(n * cg.ITEMSIZE[c] for c in out_codes)
        # Cache policy, from measurement: a stream is read once and written once per
        # launch, so beyond what the L2s hold both directions are non-temporal.  On
        # buffers that have left the 256 MB last-level cache since their last use (the
        # case a fresh batch of data presents) that is the faster choice: SAXPY n=2^24
        # 36.3 -> 33.0 us, Horner n=2^26 86.1 -> 82.6 us.  Replaying one kernel over
        # one and the same set of buffers smaller than that cache is the opposite case
        # (29 vs 31 us, 73 vs 83 us): `cache_mib`/`ntl_mib` = 200/320 favour it.
        nts = bool(TUNE["nts"]) and footprint > TUNE["cache_mib"] << 20
        ntl = bool(TUNE["ntl"]) and in_bytes > TUNE["ntl_mib"] << 20
        # Functions that keep tables in LDS: one run per block and no loop over runs.  The
        # kernel then needs 80 vector registers instead of 118 (six waves per SIMD instead
        # of four) and asks for its operands before it copies the tables, so that one wait
        # covers both.  Black-Scholes float64, 2^25 options: blocks that stay for eight runs
        # 241.8 us, one run per block with the tables copied first 279, this 233.8-236.8.
        # the vectors of a strided operand may reach up to k - 1 elements past the last one
        # used: where that is past the buffer's end the last vector step is left to the tail
        guard = any(k[0] == "s" and a.offset + n * int(k[1:]) > a.buf.nbytes // a.dtype.itemsize
                    for a, k in zip(leaves, leaf_class))
        strided = any(k[0] == "s" for k in leaf_class)
        one_run = bool(mathlib.tables(prog.own_math) and vec and not reduce_op and TUNE["one_run"]
                       and not TUNE["flat_cap"] and not strided)
        stage_loop = bool(TUNE["stage_loop"] and mathlib.tables(prog.own_math))
        runs = max(1, TUNE["table_runs"]) if one_run else 1
        low.kind = "flat"
        low.key = ("flat", prog.key(), leaf_class, tuple(out_codes), vec, reduce_op, in_place,
                   unroll, ntl, nts, ua, one_run, stage_loop, bool(TUNE["xch"]), guard, runs)

        def emit():
            src, _ = cg.emit_flat(prog, leaf_class, out_codes, vec, unroll, ntl, nts,
                                  restrict=not in_place, reduce_op=reduce_op, unaligned=ua,
                                  one_run=one_run, stage_loop=stage_loop, exchange=bool(TUNE["xch"]),
                                  guard=guard, runs=runs)
            return src
        low.emit = emit
        E = cg.flat_elements(prog, leaf_class, out_codes, reduce_op) if vec else 1
        chunks = max(1, (n // E) // (cg.BLOCK * unroll))   # one chunk per block ...
        cap = red_cap if reduce_op else (TUNE["flat_cap"] or (1 << 24) - 1)
        if mathlib.tables(prog.own_math) and not TUNE["flat_cap"] and not one_run:
            # the workgroup copies the functions' tables into LDS first: let it stay for
            # several chunks
            cap = min(cap, TUNE["table_blocks"])
        if one_run:     # block c takes run c; one more block takes what is left over
            whole = (n // E) // (cg.BLOCK * unroll * runs)
            low.grid = whole + (1 if n % (E * cg.BLOCK * unroll * runs) else 0)
        else:
            low.grid = min(chunks, cap)
        n_out_ptr = 1 if reduce_op else len(out_ptrs)
        low.fmt = "@" + "P" * (len(ptrs) + n_out_ptr) + scal_fmt + "q"
        low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
        low.scal, low.tail = scal_vals, [n]
        if reduce_op:
            low.fin_count = low.grid
        return low

    # Short rows with operands that repeat along or across them (`points * scale` with
    # points of shape (n, 3), `(x - mean) / std` over a few dozen features): a tile of 256
    # columns leaves most lanes idle (x * v, percent of the HBM peak, tiled / row kernel:
    # rows of 3 float32: 4 / 71, of 16: 10 / 78, of 64: 38 / 77, of 200: 65 / 73, of 300:
    # 55 / 67, of 1024: 76 / 79; of 2000: 72 / 69, of 4096: 77 / 76).  The row kernel without
    # reductions gives each row to a group of lanes sized to it.  Results go to new arrays
    # or into views whose rows lie one pitch apart, also over an operand (`x[...] = x * v`:
    # every element is read before it is written, by the lane that writes it).
    if (TUNE["rows_elem"] and not reduce_op and ndim >= 2 and out_codes
            and mshape[-1] * max(cg.ITEMSIZE[c] for c in out_codes) <= TUNE["rows_elem"]
            and all(s[-1] in (0, 1) for s in m_leaf)
            and (len({id(a.buf) for a in leaves}) == len(leaves) or (
                ndim == 2 and mshape[-1] * max(cg.ITEMSIZE[c] for c in out_codes) <= TUNE["rows_stencil"]))):    # (shifted views of a
        # volume share the 3-D kernel's LDS window; of a matrix with short rows, `x[:, 1:] - x[:, :-1]`,
        # they are read one by one, from the caches: the tiled kernel's window is 256 columns wide)
        try:
            return lower_rows(prog, leaves, scalars, tuple(mshape), out_codes, whole_rows=True,
                              out_strides=m_out, in_place=in_place, leaf_strides=m_leaf)
        except cg.RowFusionUnsupported:
            pass

    # Tiled family: the last merged dimension is walked with unit stride by every output
    # and with stride 1 or 0 by every operand; the dimensions in front of it are the
    # kernel's "rows" (decomposed per row when there are several).
    nouter = ndim - 1
    tiled = (not reduce_op and ndim >= 2 and all(s[-1] == 1 for s in m_out)
             and all(s[-1] in (0, 1, -1) for s in m_leaf))
    # operands walked backwards along the last dimension (flipped views) are read as vectors
    # at element alignment and reversed in registers: only the vector kernel does that
    rev = [i for i, s in enumerate(m_leaf) if s[-1] == -1] if tiled else []
    if rev:
        g0 = cg.ITEMSIZE[out_codes[0]]
        tiled = bool(TUNE["svec"] and TUNE["uvec"] and g0 in (4, 8)
                     and all(cg.ITEMSIZE[c] == g0 for c in out_codes)
                     and all(cg.ITEMSIZE[prog.leaves[i]] == g0 for i in rev)
                     and mshape[-1] >= 4 * (16 // g0))
    rows = 1
    for d in mshape[:-1]:
        rows *= d
    if tiled and ndim == 3 and TUNE["lds"] and TUNE["svec"] and TUNE["s3"] and not rev:
        low3 = _lower_stencil3d(low, prog, leaves, m_leaf, m_out, mshape, out_codes, out_ptrs,
                                scal_fmt, scal_vals, in_place)
        if low3 is not None:
            return low3
    if tiled and rows < 2 ** 31 and mshape[-1] < 2 ** 31 - 4096:
        H, W = rows, mshape[-1]
        tw, th = TUNE["tw"], TUNE["th"]
        kinds = [None] * len(leaves)
        group = None
        # halo group (2-D only): >= 2 leaves that are shifted views of one buffer
        groups = {}
        if ndim == 2 and not rev:
            for i, (a, s) in enumerate(zip(leaves, m_leaf)):
                if s[1] == 1 and s[0] > 0:
                    groups.setdefault((id(a.buf), s[0], prog.leaves[i]), []).append(i)
        best = max(groups.values(), key=len) if groups else []
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
                kinds[i] = (("b",) if not any(s) else ("d",) if s[-1] == 1 else
                            ("dr",) if s[-1] == -1 else ("r",))
        kinds = tuple(kinds)
        low.kind = "tile2d"
        vec_ok = ua = False
        if TUNE["svec"] and out_codes:
            gsize = cg.ITEMSIZE[group[0]] if group is not None else cg.ITEMSIZE[out_codes[0]]
            vw = 16 // gsize if gsize in (4, 8) else 0
            same_size = vw > 0 and all(cg.ITEMSIZE[c] == gsize for c in out_codes)
            vec_ok = (same_size and all(st % vw == 0 for s in m_out for st in s[:-1])
                      and len({(p // gsize) % vw for p in out_ptrs}) == 1
                      and (group is None or g_args[0] % vw == 0))

            def row_aligned(i, phase):
                return (all(st % vw == 0 for st in m_leaf[i][:-1])
                        and (leaves[i].ptr // gsize) % vw == phase)
            sized = [k[0] == "d" and cg.ITEMSIZE[prog.leaves[i]] == gsize
                     for i, k in enumerate(kinds)]
            missed = True
            if vec_ok:
                ph_o = (out_ptrs[0] // gsize) % vw
                dv = [d and row_aligned(i, ph_o) for i, d in enumerate(sized)]
                missed = dv != sized        # some operand would fall back to element loads
            if ((group is None or g_args[0] % vw == 0) and same_size and TUNE["uvec"]
                    and W >= 4 * vw and missed):
                # rows of any pitch and phase move as vectors at element alignment; only a
                # halo group ties the tiles to 16-byte boundaries, those of its own buffer
                # (a stencil over a padded array written to a fresh one, whose rows are a
                # few elements shorter)
                vec_ok = ua = True
                ph_o = 0
                dv = sized
        if vec_ok:
            ph_g = (g_ptr // gsize) % vw if group is not None else 0
            # direct operands whose rows share the outputs' alignment load as vectors
            kinds = tuple(("dv",) if d else k for d, k in zip(dv, kinds))
            gpr, rpt = TUNE["gpr"], TUNE["rpt"]
            if H == 1:                   # one long row: the whole block side by side
                gpr, rpt = cg.BLOCK, 1
            sntl, snts = bool(TUNE["sntl"]), bool(TUNE["snts"])
            streams = all(all(st[:-1]) for st, k in zip(m_leaf, kinds) if k[0] in ("d", "dv", "dr"))
            if group is None and TUNE["row_gpr"] and streams:
                # Nothing is shared between rows: a block takes one stretch of a row, as
                # long as the row allows (up to 4 KB), like a chunk of a flat kernel, and
                # the streams follow the flat kernels' cache policy.  An interior view of
                # 16384^2 float32, percent of the HBM peak: tiles of 8 rows x 256 columns
                # 66, with non-temporal loads 69, 2 rows x 512: 76, 1 row x 1024: 80
                # (a flat copy: 81); more rows per thread are slower (4: 70).  An operand that
                # repeats along some outer dimension keeps the taller tile, whose rows share
                # it in L1.
                gpr = 16
                while gpr < TUNE["row_gpr"] and gpr * vw < W + ph_o:
                    gpr *= 2
                rpt = 1
                in_bytes = sum(a.nbytes for a, k in zip(leaves, kinds) if k[0] in ("d", "dv", "dr"))
                out_bytes = sum(n * cg.ITEMSIZE[c] for c in out_codes)
                snts = bool(TUNE["nts"]) and in_bytes + out_bytes > TUNE["cache_mib"] << 20
                sntl = bool(TUNE["ntl"]) and in_bytes > TUNE["ntl_mib"] << 20
            # A band of consecutive tiles per XCD pays where neighbouring tiles meet in L2:
            # halo rows, or rows that do not start on 16-byte boundaries, whose first and
            # last cache lines are shared with the next tile (3-D inner slice: 66% vs 57%).
            # Plain streams are faster in launch order (row broadcast 16384^2: 79% vs 69%).
            bands = TUNE["xcd"] == 2 or (TUNE["xcd"] == 1 and (group is not None or ua))
            low.key = ("tile2dv", prog.key(), kinds, group, tuple(out_codes), in_place, ph_g, ph_o,
                       gpr, rpt, sntl, snts, bands, nouter, ua)
            tw, th = gpr * vw, (cg.BLOCK // gpr) * rpt

            def emit():
                return cg.emit_stencil_vec(prog, kinds, group, out_codes, gpr, rpt, ph_g, ph_o,
                                           restrict=not in_place, nt_load=sntl, nt_store=snts,
                                           xcd_bands=bands, nouter=nouter, unaligned=ua)[0]
            tiles_x = -(-(W + ph_o) // tw)     # tiles start `ph_o` columns left of the view
        else:
            low.key = ("tile2d", prog.key(), kinds, group, tuple(out_codes), in_place,
                       tuple(sorted(TUNE.items())), nouter)

            def emit():
                return cg.emit_stencil(prog, kinds, group, out_codes, tw, th,
                                       restrict=not in_place, nouter=nouter,
                                       xcd_bands=TUNE["xcd"] != 0)
            tiles_x = -(-W // tw)
        low.emit = emit
        tiles_y = -(-H // th)
        if tiles_x * tiles_y < 2 ** 31:
            low.grid = tiles_x * tiles_y
            srcs = [(a.buf, a.offset * a.dtype.itemsize)
                    for a, k in zip(leaves, kinds) if k[0] != "g"]
            fmt = "@" + "P" * len(srcs)
            tail_vals = []
            if group is not None:
                fmt += "P"
                srcs.append(g_src)
            fmt += "P" * len(out_ptrs) + scal_fmt + "ii"
            tail_vals += [H, W]
            if group is not None:
                fmt += "qqq"
                tail_vals += g_args
            fmt += "i"
            tail_vals.append(tiles_x)
            fmt += "q" * (nouter - 1)
            tail_vals += list(mshape[1:-1])
            for k, s in zip(kinds, m_leaf):
                if k[0] in ("d", "dv", "dr", "r"):
                    fmt += "q" * nouter
                    tail_vals += list(s[:-1])
            for s in m_out:
                fmt += "q" * nouter
                tail_vals += list(s[:-1])
            for a, k in zip(leaves, kinds):
                if vec_ok and k[0] == "dv":
                    fmt += "qq"
                    tail_vals += [-a.offset, a.buf.nbytes // a.dtype.itemsize - a.offset]
            low.fmt = fmt
            low.srcs, low.scal, low.tail = srcs, scal_vals, tail_vals
            return low

    # operands walked along some other output dimension by their unit stride (transposed
    # views): tiles span that dimension and the last one, every further dimension is a batch
    last = ndim - 1
    t_dims = set()
    for st in m_leaf:
        if any(st) and st[last] != 1:
            ones = [d for d in range(last) if st[d] == 1]
            t_dims.add(ones[0] if len(ones) == 1 else -1)
    transposed = (not reduce_op and ndim >= 2 and all(st[last] == 1 for st in m_out)
                  and len(t_dims) == 1 and -1 not in t_dims)
    if transposed:
        tp = next(iter(t_dims))
        batch = [d for d in range(last) if d != tp]
        nbatch_blocks = 1
        for d in batch:
            nbatch_blocks *= mshape[d]
        kinds = tuple(("b",) if not any(st) else ("d",) if st[last] == 1 else ("t",) for st in m_leaf)
        # Tile: 128 bytes of the transposed operand's rows by 1 KB of the output's rows.  What
        # is written contiguously counts for more than what is read contiguously; float32
        # 16384^2, percent of the HBM peak: 64 x 64 elements 66, 128 x 64: 67, 64 x 128: 68,
        # 32 x 256: 73, 16 x 512: 60, 32 x 384: 64.
        # An operand whose columns lie a megabyte or more apart (the reversed axes of a 3-D
        # array) puts every column of a tile on another page: fewer, longer columns then
        # (512 x 512 x 1024 float32 reversed: 32 x 256: 59, 64 x 64: 64, 128 x 64: 67,
        # 128 x 32: 66, 256 x 32: 65).
        short = min(mshape[tp], mshape[last])
        if (not batch and short <= THIN_TRANSPOSE and (short & (short - 1) or THIN_TRANSPOSE_ALL)
                and max(mshape[tp], mshape[last]) >= 4096):
            # one side of a few elements, no power of two (rows of three coordinates): the tiles
            # move single elements on that side; a lane per index of the long side needs no tile
            short_rows = mshape[tp] == short
            n_long = mshape[last] if short_rows else mshape[tp]
            low.kind = "thin_t"
            low.key = ("thin_t", prog.key(), kinds, tuple(out_codes), in_place, short, short_rows)

            def emit_thin():
                return cg.emit_thin_transpose(prog, kinds, out_codes, short, short_rows,
                                              restrict=not in_place)
            low.emit = emit_thin
            low.grid = -(-n_long // cg.BLOCK)
            low.fmt = "@" + "P" * (len(leaves) + len(out_ptrs)) + scal_fmt + "q" \
                + "q" * (sum(k[0] in ("t", "d") for k in kinds) + len(out_ptrs))
            low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
            low.scal = scal_vals
            low.tail = [n_long] + [st[last] for st, k in zip(m_leaf, kinds) if k[0] == "t"] \
                + [st[tp] for st, k in zip(m_leaf, kinds) if k[0] == "d"] + [st[tp] for st in m_out]
            return low
        widest = max(cg.ITEMSIZE[c] for c in list(prog.leaves) + list(out_codes))
        far = max(abs(st[last]) * cg.ITEMSIZE[c] for st, c, k in zip(m_leaf, prog.leaves, kinds)
                  if k[0] == "t") >= 1 << 20
        t_r = TUNE["t_rows"] or (512 if far else 128) // widest
        t_c = TUNE["t_cols"] or (256 if far else 1024) // widest
        if not TUNE["t_rows"] and not TUNE["t_cols"]:
            # A matrix with one short side (points as rows of three coordinates and the three
            # coordinate vectors: `pts.T`): a tile that fits the short side instead of leaving
            # most of its lanes outside the matrix.  `a.T * 2`, float32, percent of the HBM
            # peak with the default tile / the fitted one: (n, 3): 5 / 38, (3, n): 8 / 44,
            # (n, 4): 6 / 75, (n, 8): 12 / 64, (8, n): 17 / 74, (n, 16): 21 / 73, (16, n):
            # 24 / 76, (32, n): 28 / 74; float64 (n, 6): 42 / 61, (6, n): 43 / 63.
            def fitted(extent):
                p2 = 4
                while p2 < extent:
                    p2 *= 2
                return p2
            if mshape[tp] <= 16:
                t_r, t_c = fitted(mshape[tp]), 256
            elif mshape[last] <= 32:
                t_c = fitted(mshape[last])
                t_r = 256 if 257 * t_c * widest <= 48 * 1024 else 128
        lds_bytes = sum((t_r + 1) * t_c * cg.ITEMSIZE[c]
                        for c, k in zip(prog.leaves, kinds) if k[0] == "t")
        if lds_bytes > 64 * 1024:
            t_r = t_c = cg.T_TILE
            lds_bytes = sum((t_r + 1) * t_c * cg.ITEMSIZE[c]
                            for c, k in zip(prog.leaves, kinds) if k[0] == "t")
        if lds_bytes <= 64 * 1024 and (-(-mshape[tp] // t_r) * -(-mshape[last] // t_c)
                                       * nbatch_blocks < 2 ** 31) and len(batch) <= 4:
            H, W = mshape[tp], mshape[last]
            low.kind = "tile2dt"
            # 16 bytes per lane on both sides when every array has the same element
            # size and all rows (of the operands' own layouts) start 16-byte aligned
            sizes = {cg.ITEMSIZE[c] for c in list(prog.leaves) + list(out_codes)}
            vec = 16 // sizes.pop() if len(sizes) == 1 and sizes <= {4, 8} and TUNE["tvec"] else 0
            ua = False
            if vec and all(c in cg.VEC16 for c in list(prog.leaves) + list(out_codes)):
                pitches = [(st[last] if k[0] == "t" else st[tp], a.offset)
                           for a, k, st in zip(leaves, kinds, m_leaf) if k[0] != "b"]
                pitches += [(st[tp], ptr // cg.ITEMSIZE[c]) for ptr, st, c in zip(out_ptrs, m_out, out_codes)
                            if ptr % cg.ITEMSIZE[c] == 0]
                if len(pitches) != len(out_ptrs) + sum(k[0] != "b" for k in kinds):
                    vec = 0
                elif any(pitch % vec or first % vec for pitch, first in pitches) or any(
                        st[d] % vec for st in list(m_leaf) + list(m_out) for d in batch):
                    ua = True               # vectors at element alignment
                    vec = vec if TUNE["uvec"] else 0
            else:
                vec = 0
            out_bytes = sum(n * cg.ITEMSIZE[c] for c in out_codes)
            in_bytes = sum(n * cg.ITEMSIZE[c] for c, k in zip(prog.leaves, kinds) if k[0] != "b")
            nts = bool(vec and TUNE["nts"]) and in_bytes + out_bytes > TUNE["cache_mib"] << 20
            ntl = bool(vec and TUNE["ntl"]) and in_bytes > TUNE["ntl_mib"] << 20
            ua = bool(ua and vec)
            low.key = ("tile2dt", prog.key(), kinds, tuple(out_codes), in_place, vec, ntl, nts, ua,
                       t_r, t_c, len(batch))

            def emit():
                return cg.emit_tile_transpose(prog, kinds, out_codes, restrict=not in_place,
                                              vec=vec, nt_load=ntl, nt_store=nts, unaligned=ua,
                                              tile=(t_r, t_c), nbatch=len(batch))
            low.emit = emit
            tiles_x = -(-W // t_c)
            low.grid = tiles_x * -(-H // t_r) * nbatch_blocks
            fmt = "@" + "P" * (len(leaves) + len(out_ptrs)) + scal_fmt + "iii"
            tail_vals = [H, W, tiles_x]
            for k, s in zip(kinds, m_leaf):
                if k[0] == "t":
                    fmt += "q"
                    tail_vals.append(s[last])
            for k, s in zip(kinds, m_leaf):
                if k[0] == "d":
                    fmt += "q"
                    tail_vals.append(s[tp])
            for s in m_out:
                fmt += "q"
                tail_vals.append(s[tp])
            for d in batch:
                fmt += "q" * (1 + len(m_leaf) + len(m_out))
                tail_vals += [mshape[d]] + [st[d] for st in m_leaf] + [st[d] for st in m_out]
            low.fmt = fmt
            low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
            low.scal, low.tail = scal_vals, tail_vals
            return low

    # general strided kernel
    if ndim == 0:
        mshape, m_leaf, m_out, ndim = [1], [[0] for _ in m_leaf], [[0] for _ in m_out], 1
    index32 = n < 2 ** 31
    low.kind = "nd"
    low.key = ("nd", prog.key(), ndim, tuple(out_codes), index32, reduce_op,
               tuple(sorted(TUNE.items())))

    def emit():
        return cg.emit_nd(prog, ndim, out_codes, index32, reduce_op)
    low.emit = emit
    blocks = -(-n // cg.BLOCK)
    low.grid = max(1, min(blocks, grid_cap()))
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


def lower_axis_reduce(prog, leaves, scalars, shape, axes, acc, reduce_op, slices=None):
    """Kernel choice for reducing over `axes` of the (broadcast) `shape`.

    Returns (first pass, S, K, strategy): when S > 1 the first pass writes S partial
    results per output ([slice][output] for 'col', [output][slice] for 'row') and the
    caller runs a second reduction over them (`slices=1` asks for that second pass).
    Matrices with one short side have kernels of their own: `axis_narrow` (few kept
    columns, dense rows reduced; its partials are laid out like 'col') and
    `axis_short` (short contiguous rows reduced; no partials)."""
    kept = [d for d in range(len(shape)) if d not in axes]
    full = [broadcast_strides(a, shape) for a in leaves]
    kshape = [shape[d] for d in kept]
    rshape = [shape[d] for d in axes]
    kmerged, ksets = merge_dims(kshape, [[s[d] for d in kept] for s in full])
    rmerged, rsets = merge_dims(rshape, [[s[d] for d in axes] for s in full])
    if not kmerged:
        kmerged, ksets = [1], [[0] for _ in leaves]
    if not rmerged:
        rmerged, rsets = [1], [[0] for _ in leaves]
    K = R = 1
    for d in kmerged:
        K *= d
    for d in rmerged:
        R *= d
    # kept dimensions that merge into one sequence of rows, or into two levels of them that
    # the row-wise kernels split again (an operand shared by every item of a batch)
    two = len(kmerged) == 2 and K < 2 ** 31
    one_or_two = len(kmerged) == 1 or two
    two_fmt = "I" + "q" * len(leaves) if two else ""
    two_tail = [kmerged[1]] + [k[1] for k in ksets] if two else []
    two_key = ("two levels",) if two else ()
    # coalescing decides the strategy: which side holds the unit-stride dimension
    # (judged by the operands that carry the traffic: a column of weights beside a matrix
    # must not turn a sum over rows into the strategy for sums along rows)
    big = max([a.size for a in leaves], default=0)
    heavy = [i for i, a in enumerate(leaves) if a.size == big]
    inner_kept = any(ksets[i][-1] == 1 for i in heavy)
    inner_red = any(rsets[i][-1] == 1 for i in heavy)
    strategy = "col" if (inner_kept and not inner_red) else "row"
    def narrow_units():
        """16-byte units per row of the narrow matrix, as `codegen.emit_narrow_cols` counts them
        (a wave's lanes must hold at least one row of them)."""
        widths = {cg.ITEMSIZE[c] for c, r in zip(prog.leaves, rsets) if r[0] == K}
        V = 16 // next(iter(widths)) if len(widths) == 1 and widths <= {4, 8} else 1
        return K // V if K % V == 0 else K
    if (strategy == "col" and slices in (None, 1) and 2 <= K <= TUNE["ax_narrow"]
            and narrow_units() <= cg.WAVE
            and (R >= 4096 or slices == 1)
            and len(kmerged) == 1 and len(rmerged) == 1 and R * K < 2 ** 40
            and all((k[0], r[0]) in ((1, K), (1, 0), (0, 0), (0, 1)) for k, r in zip(ksets, rsets))
            and any((k[0], r[0]) == (1, K) for k, r in zip(ksets, rsets))):
        # a dense matrix with few columns, summed over its rows: read it as one stream
        # (beside it: a row of weights for the columns, a dense vector of weights for the rows)
        kinds = tuple("d" if r[0] == K else "w" if k[0] == 1 else "c" if r[0] == 1 else "b"
                      for k, r in zip(ksets, rsets))
        low = Lowered()
        low.lds = 0
        low.fin_count = 0
        low.kind = "axis_narrow"
        low.key = ("axis_narrow", prog.key(), kinds, acc, reduce_op, K)

        def emit_narrow():
            return cg.emit_narrow_cols(prog, kinds, acc, reduce_op, K)[0]
        low.emit = emit_narrow
        widths = {cg.ITEMSIZE[c] for c, kd in zip(prog.leaves, kinds) if kd == "d"}
        V = 16 // widths.pop() if len(widths) == 1 and widths <= {4, 8} else 1
        V = V if K % V == 0 else 1
        KC = K // V
        LW = (cg.WAVE // KC) * KC
        U = R * KC
        per_block = (cg.BLOCK // cg.WAVE) * LW
        # several passes of four chunks per wave; the partials, one row of K per block,
        # are a narrow matrix again and one more block of this kernel finishes them
        # (which bounds their number: that block walks S * KC units alone)
        S = 1 if slices == 1 else max(1, min(-(-U // (per_block * 4 * 4)), TUNE["ax_blocks"],
                                             max(256, 16384 // KC)))
        low.grid = S
        low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars) + "q")
        low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
        low.scal, low.tail = list(scalars), [U]
        return low, S, K, "col"
    if (strategy == "row" and slices is None and R <= TUNE["ax_short"] and K >= 4096
            and one_or_two and len(rmerged) == 1
            and all(r[0] in (0, 1) for r in rsets) and K < 2 ** 40):
        # many short rows: a lane per output walking its own row, no combining step
        kinds = tuple("v" if r[0] == 1 else "k" for r in rsets)
        low = Lowered()
        low.lds = 0
        low.fin_count = 0
        low.kind = "axis_short"
        low.key = ("axis_short", prog.key(), kinds, acc, reduce_op, R) + two_key

        def emit_short():
            return cg.emit_short_rows(prog, kinds, acc, reduce_op, R, outer2=two)
        low.emit = emit_short
        low.grid = -(-K // cg.BLOCK)
        low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                   + "q" + "q" * len(leaves) + two_fmt)
        low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
        low.scal, low.tail = list(scalars), [K] + [k[0] for k in ksets] + two_tail
        return low, 1, K, "short"
    if (strategy == "row" and slices is None and TUNE["ax_short"] < R <= TUNE["ax_group"]
            and K >= 1024 and one_or_two and len(rmerged) == 1 and TUNE["uvec"]
            and all(r[0] in (0, 1) for r in rsets) and K < 2 ** 40):
        widths = {cg.ITEMSIZE[c] for c, r in zip(prog.leaves, rsets) if r[0] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, r in zip(prog.leaves, rsets) if r[0] == 1):
            # rows of a few hundred elements: a group of lanes per row, sized to the row
            V = 16 // next(iter(widths))
            units = -(-R // V)
            # measured (float32, 2^28 elements, % of 8 TB/s, groups of 8 / 16 lanes): rows of
            # 32: 72 / 56, 100: 76 / 70, 128: 75 / 75, 200: 75 / 77, 250: 76 / 78, 1000: 75 / 76;
            # a whole wave per row: 200: 55, 250: 50, 333: 52; a lane per row: 32: 71, 100: 50
            G = 8 if units <= 32 else 16
            while -(-units // G) > TUNE["ax_group_steps"] and G < cg.WAVE:
                G *= 2
            G = TUNE["ax_group_lanes"] or G
            kinds = tuple("v" if r[0] == 1 else "k" for r in rsets)
            low = Lowered()
            low.lds = 0
            low.fin_count = 0
            low.kind = "axis_group"
            low.key = ("axis_group", prog.key(), kinds, acc, reduce_op, R, G) + two_key

            def emit_group():
                return cg.emit_group_rows(prog, kinds, acc, reduce_op, R, G, outer2=two)
            low.emit = emit_group
            rows_per_block = (cg.BLOCK // cg.WAVE) * (cg.WAVE // G)
            # one pass over the rows per wave (rows of 200 float32: 80.6 % of the HBM peak; four
            # passes 76.5, sixteen 72.9)
            low.grid = max(1, min(-(-K // rows_per_block), 1 << 20))
            low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                       + "q" + "q" * len(leaves) + two_fmt)
            low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
            low.scal, low.tail = list(scalars), [K] + [k[0] for k in ksets] + two_tail
            return low, 1, K, "group"
    if (strategy == "col" and slices is None and len(rmerged) == 1 and len(kmerged) == 1
            and TUNE["ax_stream"] > 0 and TUNE["uvec"] and all(k[0] in (0, 1) for k in ksets)):
        widths = {cg.ITEMSIZE[c] for c, k in zip(prog.leaves, ksets) if k[0] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, k in zip(prog.leaves, ksets) if k[0] == 1):
            V = 16 // next(iter(widths))
            ktiles = -(-K // (cg.BLOCK * V))
            if K >= cg.BLOCK * V and R >= 64:
                # long rows kept: blocks of 256 lanes x one vector stream whole rows together.
                # Sum over axis 0 of 16384^2 float32, percent of the HBM peak by blocks in the
                # grid: 128: 77, 256 (one per compute unit): 80, 512: 79, 1024: 77, 2048: 65,
                # 4096: 61; a lane per column with four waves on four rows (`col`): 72.
                S = max(1, min(-(-TUNE["ax_stream"] // ktiles), R // 32, TUNE["ax_slices"]))
                RS = -(-R // S)
                S = -(-R // RS)
                kinds = tuple("v" if k[0] == 1 else "k" for k in ksets)
                low = Lowered()
                low.lds = 0
                low.fin_count = 0
                low.kind = "axis_stream"
                unroll = TUNE["ax_stream_unroll"]
                stagger = bool(TUNE["ax_stream_stagger"])
                low.key = ("axis_stream", prog.key(), kinds, acc, reduce_op, unroll, stagger)

                def emit_stream():
                    return cg.emit_col_stream(prog, kinds, acc, reduce_op, unroll, stagger=stagger)
                low.emit = emit_stream
                low.grid = max(1, min(ktiles * S, 1 << 20))
                low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                           + "qqqq" + "q" * len(leaves))
                low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
                low.scal, low.tail = list(scalars), [K, R, S, RS] + [r[0] for r in rsets]
                return low, S, K, "col"
    if (strategy == "col" and slices is None and len(rmerged) == 1 and len(kmerged) == 2
            and TUNE["ax_stream"] > 0 and TUNE["uvec"] and all(k[1] in (0, 1) for k in ksets)):
        widths = {cg.ITEMSIZE[c] for c, k in zip(prog.leaves, ksets) if k[1] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, k in zip(prog.leaves, ksets) if k[1] == 1):
            V = 16 // next(iter(widths))
            KO, KI = kmerged
            ktiles = -(-KI // (cg.BLOCK * V))
            if KI >= cg.BLOCK * V and R >= 64:
                # the middle axis of a 3-D array reduced: the same walk down the rows, once per
                # index of the first axis
                S = max(1, min(-(-TUNE["ax_stream"] // (ktiles * KO)), R // 32, TUNE["ax_slices"]))
                RS = -(-R // S)
                S = -(-R // RS)
                kinds = tuple("v" if k[1] == 1 else "k" for k in ksets)
                low = Lowered()
                low.lds = 0
                low.fin_count = 0
                low.kind = "axis_stream"
                unroll = TUNE["ax_stream_unroll"]
                stagger = bool(TUNE["ax_stream_stagger"])
                low.key = ("axis_stream", prog.key(), kinds, acc, reduce_op, unroll, stagger, "outer")

                def emit_stream2():
                    return cg.emit_col_stream(prog, kinds, acc, reduce_op, unroll, outer=True, stagger=stagger)
                low.emit = emit_stream2
                low.grid = max(1, min(ktiles * KO * S, 1 << 20))
                low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                           + "qqqq" + "q" * len(leaves) + "q" + "q" * len(leaves))
                low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
                low.scal = list(scalars)
                low.tail = [KI, R, S, RS] + [r[0] for r in rsets] + [KO] + [k[0] for k in ksets]
                return low, S, K, "col"
    if (strategy == "row" and slices is None and len(rmerged) == 2 and len(kmerged) == 1
            and rmerged[1] >= 1024 and TUNE["ax_block"] > 0 and TUNE["uvec"]
            and all(r[1] in (0, 1) for r in rsets)):
        widths = {cg.ITEMSIZE[c] for c, r in zip(prog.leaves, rsets) if r[1] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, r in zip(prog.leaves, rsets) if r[1] == 1):
            # the first and the last axis of a 3-D array reduced (per-channel statistics): a
            # block takes whole rows of the last axis over a slice of the first
            RO, RI = rmerged
            S = max(1, min(-(-TUNE["ax_blocks"] // K), RO // 4, TUNE["ax_slices"]))
            if K * S < 1024:
                # few channels: a row per block rather than four, to have blocks for every
                # compute unit (sum over (0, 2, 3) of 64 x 3 x 224 x 224 float32: 48 blocks
                # took 78 us, 192 take 24)
                S = max(S, min(-(-TUNE["ax_blocks"] // K), RO, TUNE["ax_slices"]))
            QS = -(-RO // S)
            S = -(-RO // QS)
            kinds = tuple("v" if r[1] == 1 else "k" for r in rsets)
            low = Lowered()
            low.lds = 0
            low.fin_count = 0
            low.kind = "axis_block"
            low.key = ("axis_block", prog.key(), kinds, acc, reduce_op, "outer")

            def emit_block2():
                return cg.emit_block_rows(prog, kinds, acc, reduce_op, outer=True)
            low.emit = emit_block2
            low.grid = max(1, min(K * S, 1 << 20))
            low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                       + "qqqq" + "q" * len(leaves) + "q" + "q" * len(leaves))
            low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
            low.scal = list(scalars)
            low.tail = [K, RI, S, QS] + [k[0] for k in ksets] + [RO] + [r[0] for r in rsets]
            return low, S, K, "row"
    if (strategy == "row" and slices is None and len(rmerged) == 1 and one_or_two
            and R >= TUNE["ax_block"] > 0 and TUNE["uvec"] and all(r[0] in (0, 1) for r in rsets)):
        widths = {cg.ITEMSIZE[c] for c, r in zip(prog.leaves, rsets) if r[0] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, r in zip(prog.leaves, rsets) if r[0] == 1):
            # long rows: a block per row (or per slice of a row, while there are too few rows
            # to fill the device), streamed like a flat reduction
            V = 16 // next(iter(widths))
            S = max(1, min(-(-TUNE["ax_blocks"] // K), R // TUNE["ax_block"], TUNE["ax_slices"]))
            RS = -(-R // S)
            S = -(-R // RS)
            kinds = tuple("v" if r[0] == 1 else "k" for r in rsets)
            # an operand that is the same for every row (the vector of a matrix-vector
            # product) stays in the caches; `a @ x` on 16384^2 float32: 76.8 % of the HBM
            # peak with every load non-temporal
            shared = tuple(i for i, (k, r) in enumerate(zip(ksets, rsets)) if r[0] == 1 and not any(k))
            low = Lowered()
            low.lds = 0
            low.fin_count = 0
            low.kind = "axis_block"
            low.key = ("axis_block", prog.key(), kinds, acc, reduce_op, shared) + two_key
            rows = TUNE["ax_block_rows"]
            if shared and S == 1 and rows > 1 and K >= 1024 * rows and not two:
                # several rows per block: the shared operand is loaded once for all of them
                unroll = TUNE["ax_block_rows_unroll"]
                low.key = ("axis_block", prog.key(), kinds, acc, reduce_op, shared, unroll, rows)

                def emit_rows():
                    return cg.emit_block_rows_shared(prog, kinds, acc, reduce_op, shared, rows, unroll)
                low.emit = emit_rows
                low.grid = max(1, min(-(-K // rows), 1 << 20))
                low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                           + "qq" + "q" * len(leaves))
                low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
                low.scal, low.tail = list(scalars), [K, R] + [k[0] for k in ksets]
                return low, 1, K, "row"

            def emit_block():
                return cg.emit_block_rows(prog, kinds, acc, reduce_op, shared=shared, outer2=two)
            low.emit = emit_block
            low.grid = max(1, min(K * S, 1 << 20))
            low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
                       + "qqqq" + "q" * len(leaves) + two_fmt)
            low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
            low.scal, low.tail = list(scalars), [K, R, S, RS] + [k[0] for k in ksets] + two_tail
            return low, S, K, "row"
    # enough independent pieces to fill the device: cut the reduced extent into slices
    if slices is not None:
        S = slices
    elif strategy == "col":
        ktiles = -(-K // cg.WAVE)
        S = max(1, min(-(-TUNE["ax_blocks"] // ktiles), R // 32, TUNE["ax_slices"]))
    else:
        S = max(1, min(-(-TUNE["ax_waves"] // K), R // 256, TUNE["ax_slices"]))
    RS = -(-R // S)
    S = -(-R // RS)
    low = Lowered()
    low.lds = 0
    low.fin_count = 0
    low.kind = "axis_" + strategy
    kdim, rdim = len(kmerged), len(rmerged)
    row_vec = None
    # short rows gain from 16-byte loads (256 elements: 59% -> 73% of peak), long ones do
    # not (16384: 73% -> 70%): a wave's 256-byte loads already stream them
    if (strategy == "row" and rdim == 1 and TUNE["uvec"] and RS <= 512
            and all(r[0] in (0, 1) for r in rsets)):
        widths = {cg.ITEMSIZE[c] for c, r in zip(prog.leaves, rsets) if r[0] == 1}
        if len(widths) == 1 and widths <= {4, 8} and all(
                c in cg.VEC16 for c, r in zip(prog.leaves, rsets) if r[0] == 1):
            row_vec = tuple("v" if r[0] == 1 else "k" for r in rsets)
    low.key = ("axis", prog.key(), kdim, rdim, acc, reduce_op, strategy, row_vec)

    def emit():
        return cg.emit_axis_reduce(prog, kdim, rdim, acc, reduce_op, strategy, row_vec)
    low.emit = emit
    if strategy == "col":
        low.grid = max(1, min(-(-K // cg.WAVE) * S, 1 << 20))
    else:
        low.grid = max(1, min(-(-(K * S) // (cg.BLOCK // cg.WAVE) // TUNE["ax_rows"]), 1 << 20))
    low.fmt = ("@" + "P" * (len(leaves) + 1) + "".join(_SCALAR_FMT[c] for c in prog.scalars)
               + "qqqq" + "q" * (kdim + rdim) + "q" * ((kdim + rdim) * len(leaves)))
    tail = [K, R, S, RS] + list(kmerged) + list(rmerged)
    for ks, rs in zip(ksets, rsets):
        tail += list(ks) + list(rs)
    low.srcs = [(a.buf, a.offset * a.dtype.itemsize) for a in leaves]
    low.scal, low.tail = list(scalars), tail
    return low, S, K, strategy
