#!/usr/bin/env python3
"""Benchmark of the fused hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME|all]

A step is one pass of the hot path over one batch: build the lazy expression,
trace it, look the kernel up in the cache and launch it on inputs that already
sit in HBM (for the stencil: one sweep; for the reduction: body + finalize).
Prints ONE JSON line.  Its top-level fields describe the largest configuration
(the fused reduction sum((x-y)**2*w), float64, n = 2^27); `configs` carries the
same figures for every configuration and `roofline.min_frac` the lowest fraction
among them.

Cold measurement: MI355X has a 256 MB last-level (Infinity) cache in front of HBM,
so a kernel replayed over one set of buffers smaller than that is partly served
from the cache.  Every workload therefore owns R sets of inputs and outputs with
R x footprint >= 3 x 256 MiB (at least 2) and both the timed steps and the kernel
replays rotate through them, so a buffer has been evicted by the time it comes
round again.  The replay over a single set is kept as `frac_warm`.

Per configuration:
  value / GBps        algorithmic bytes * steps / wall time of the timed region
                      (whole step, host side included), rotating over the R sets
  roofline            algorithmic bytes / kernel duration against 8 TB/s; the duration
                      is measured with HIP events on the library's stream around
                      back-to-back replays of the recorded launches of all R sets,
                      median (and minimum) over REGIONS timed regions
  unfused             the same expression with one kernel per DAG node
  cpu_baseline        the NumPy node-by-node evaluation (oracle/numpy_oracle.py, a port
                      of the reference's CPU backend) on this machine's host cores
  parity (bs32/bs64)  largest result-relative differences from the oracle over all 2^25
                      options (oracle/accuracy.py)
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
LLC_BYTES = 256 << 20          # Infinity Cache
REGIONS = 7                    # timed regions per kernel figure (median and minimum reported)
METRIC = "fused-kernel effective HBM GB/s (% of MI355X peak); Gelem/s vs unfused"


def measured_traffic(name):
    """(HBM bytes per launch, kernel names) of a workload as measured with rocprofv3
    counters (FETCH_SIZE + WRITE_SIZE, calibrated on the copy kernel); the figures live
    in profiles/hbm_traffic.txt as `<workload> <bytes>   # <kernel>[, <kernel>]: ...`
    lines.  The kernel names carry a digest of everything that shapes the generated
    source, so a figure taken from another version of a kernel can be told."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    try:
        with open(path) as fh:
            for ln in fh:
                parts = ln.split()
                if len(parts) >= 2 and parts[0] == name:
                    kernels = []
                    if "#" in ln:
                        kernels = [k.strip() for k in ln.split("#", 1)[1].split(":", 1)[0].split(",")]
                    return int(float(parts[1])), sorted(k for k in kernels if k)
    except OSError:
        pass
    return None, []


def profiled_figure(fname, name):
    """A per-workload figure kept under profiles/ as `<workload> <number>` lines (taken
    with rocprofv3 counters, which this script cannot read while it runs)."""
    path = os.path.join(ROOT, "profiles", fname)
    try:
        with open(path) as fh:
            for ln in fh:
                parts = ln.split()
                if len(parts) >= 2 and parts[0] == name:
                    return float(parts[1])
    except OSError:
        pass
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all",
                    help="sumsq (headline) | saxpy | horner | bs32 | bs64 | jacobi | all (these six); "
                         "dot | axis0 | axis1 | axis1_3d | matvec | rows200 | rowbcast | transpose | "
                         "transpose3d | interior | diff2 | stencil9 | stencil3d | grid | rand | softmax | softmax32k | "
                         "layernorm | rowmax | strided | strided2d | points3 | next (all "
                         "of these: the operations either side of the five configurations); "
                         "matmul32 | matmul64 (the eager matrix product)")
    ap.add_argument("--settle", type=float, default=0.25,
                    help="seconds of untimed load before each timed region (clock ramp-up)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0,
                    help="CPU time spent on the headline workload's baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-copy", action="store_true", help="skip the plain-copy ceiling leg")
    ap.add_argument("--no-parity", action="store_true",
                    help="skip the Black-Scholes error table against the oracle")
    ap.add_argument("--sets", type=int, default=0,
                    help="buffer sets to rotate over (0: enough to defeat the last-level cache)")
    ap.add_argument("--no-unfused", action="store_true", help="skip the un-fused leg")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              f"(--gpus {args.gpus} refused)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import delayrepay_amd as dr
    from delayrepay_amd import hip, hiprt
    from delayrepay_amd.delayarray import ReduceEx
    from oracle import numpy_oracle as orc

    hiprt.init()
    info = hiprt.device_info()
    K, W = args.steps, args.warmup

    def horner_expr(c, x):
        acc = c[8] * x + c[7]
        for i in range(6, -1, -1):
            acc = acc * x + c[i]
        return acc

    def again(leaf):
        """A new device array with the contents of `leaf`, as a new lazy leaf."""
        return dr.NPArray(leaf._force().copy())

    def sets_for(nbytes):
        """Buffer sets so that a set has left the last-level cache before its next turn."""
        if args.sets:
            return args.sets
        return max(2, -(-3 * LLC_BYTES // nbytes))

    # ---- the workloads: R step functions (one per set of device buffers), algorithmic
    #      bytes and elements of one step, and the CPU evaluation of a bounded sample
    def make(name):
        inp = orc.make_inputs(name) if name in ("saxpy", "horner", "bs32", "bs64", "jacobi",
                                                "sumsq") else None
        if name == "saxpy":
            n = inp["x"].size
            R = sets_for(12 * n)
            sets = [(dr.array(inp["x"]), dr.array(inp["y"])) for _ in range(R)]

            def fresh(x=sets[0][0], y=sets[0][1]):
                x, y = again(x), again(y)
                return lambda: hip.run(inp["a"] * x + y)
            return dict(dtype="f32", n=n, nbytes=12 * n, desc="SAXPY z=a*x+y f32 n=2^24", fresh=fresh,
                        steps=[(lambda x=x, y=y: hip.run(inp["a"] * x + y)) for x, y in sets],
                        cpu=lambda: orc.saxpy(inp["a"], inp["x"], inp["y"]), cpu_frac=1.0,
                        cpu_code="oracle/numpy_oracle.py::saxpy")
        if name == "horner":
            n = inp["x"].size
            R = sets_for(8 * n)
            sets = [dr.array(inp["x"]) for _ in range(R)]

            def fresh(x=sets[0]):
                x = again(x)
                return lambda: hip.run(horner_expr(inp["c"], x))
            return dict(dtype="f32", n=n, nbytes=8 * n, fresh=fresh,
                        desc="Horner degree-8 polynomial f32 n=2^26",
                        steps=[(lambda x=x: hip.run(horner_expr(inp["c"], x))) for x in sets],
                        cpu=lambda: orc.horner(inp["c"], inp["x"]), cpu_frac=1.0,
                        cpu_code="oracle/numpy_oracle.py::horner")
        if name in ("bs32", "bs64"):
            n = inp["S"].size
            size = inp["S"].dtype.itemsize
            R = sets_for(5 * size * n)
            sets = [tuple(dr.array(inp[k]) for k in "SKT") for _ in range(R)]
            m = n // 4       # CPU sample: a quarter of the options

            def fresh(first=sets[0]):
                S, K_, T = (again(a) for a in first)
                return lambda: hip.run_multi(list(orc.black_scholes_expr(dr, S, K_, T, inp["r"],
                                                                         inp["sigma"])))
            return dict(dtype="f32" if size == 4 else "f64", n=n, nbytes=5 * size * n, fresh=fresh,
                        desc=f"Black-Scholes call+put {'f32' if size == 4 else 'f64'} n=2^25",
                        steps=[(lambda S=S, K_=K_, T=T: hip.run_multi(list(orc.black_scholes_expr(
                            dr, S, K_, T, inp["r"], inp["sigma"])))) for S, K_, T in sets],
                        cpu=lambda: orc.black_scholes(inp["S"][:m], inp["K"][:m], inp["T"][:m],
                                                      inp["r"], inp["sigma"]), cpu_frac=0.25,
                        cpu_code="oracle/numpy_oracle.py::black_scholes", inputs=inp, sets=sets)
        if name == "jacobi":
            N = inp["u"].shape[0]
            nbytes = 4 * N * N + 4 * (N - 2) * (N - 2)
            R = sets_for(nbytes)
            grids = [dr.array(inp["u"]) for _ in range(R)]

            def sweep(u):
                u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])

            def fresh(u=grids[0]):
                u = again(u)
                return lambda: sweep(u)
            return dict(dtype="f32", n=(N - 2) * (N - 2), nbytes=nbytes, fresh=fresh,
                        desc="Jacobi 5-point f32 8192x8192, per sweep",
                        steps=[(lambda u=u: sweep(u)) for u in grids], pair=True,
                        cpu=lambda: orc.jacobi(inp["u"], 1), cpu_frac=1.0,
                        cpu_code="oracle/numpy_oracle.py::jacobi")
        if name == "sumsq":
            n = inp["x"].size
            R = sets_for(24 * n)
            sets = [tuple(dr.array(inp[k]) for k in "xyw") for _ in range(R)]
            m = n // 4

            def fresh(first=sets[0]):
                x, y, w = (again(a) for a in first)
                return lambda: hip.run(ReduceEx(np.add, (x - y) ** 2 * w))
            return dict(dtype="f64", n=n, nbytes=24 * n, desc="sum((x-y)**2*w) f64 n=2^27", fresh=fresh,
                        steps=[(lambda x=x, y=y, w=w: hip.run(ReduceEx(np.add, (x - y) ** 2 * w)))
                               for x, y, w in sets],
                        cpu=lambda: orc.sumsq(inp["x"][:m], inp["y"][:m], inp["w"][:m]),
                        cpu_frac=0.25, cpu_code="oracle/numpy_oracle.py::sumsq")
        # ---- operations either side of the five configurations (no CPU sample kept small)
        rs = np.random.RandomState(0)
        if name == "dot":
            n = 1 << 27
            hx, hy = rs.standard_normal(n), rs.standard_normal(n)
            sets = [(dr.array(hx), dr.array(hy)) for _ in range(sets_for(16 * n))]
            return dict(dtype="f64", n=n, nbytes=16 * n, desc="dot(x, y) f64 n=2^27 (fused multiply-reduce)",
                        steps=[(lambda x=x, y=y: hip.run(ReduceEx(np.add, x * y))) for x, y in sets],
                        cpu=lambda: np.dot(hx[:n // 4], hy[:n // 4]), cpu_frac=0.25, cpu_code="numpy.dot")
        if name == "grid":
            n = 1 << 26
            c = orc.make_inputs("horner")["c"]
            g = dr.linspace(-2.0, 2.0, n, dtype=np.float32)     # lazy: computed inside the kernel
            m = n // 16
            return dict(dtype="f32", n=n, nbytes=4 * n,
                        desc="Horner degree-8 on linspace(-2, 2, n) f32 n=2^26 (grid generated in the kernel)",
                        steps=[lambda: hip.run(horner_expr(c, g))] * sets_for(4 * n),
                        cpu=lambda: orc.horner(c, np.linspace(-2.0, 2.0, m, dtype=np.float32)),
                        cpu_frac=1 / 16, cpu_code="oracle/numpy_oracle.py::horner on numpy.linspace")
        if name == "rand":
            n = 1 << 26
            u = dr.random.device(0).random(n)                   # lazy: computed inside the kernel
            m = n // 16
            return dict(dtype="f64", n=n, nbytes=8 * n,
                        desc="Philox-4x64-10 uniform doubles n=2^26 written to memory (generated in the kernel)",
                        steps=[lambda: hip.run(u * 1.0)] * sets_for(8 * n),
                        cpu=lambda: np.random.Generator(np.random.Philox(key=0)).random(m),
                        cpu_frac=1 / 16, cpu_code="numpy.random.Generator(Philox).random")
        if name in ("matmul32", "matmul64"):
            N = 8192
            dt = np.float32 if name == "matmul32" else np.float64
            ha, hb = rs.standard_normal((N, N)).astype(dt), rs.standard_normal((N, N)).astype(dt)
            a, b = dr.array(ha), dr.array(hb)
            m = 1024        # CPU sample: a 1024^3 product (NumPy's BLAS, all host cores)
            return dict(dtype="f32" if dt == np.float32 else "f64", n=N * N,
                        nbytes=3 * N * N * ha.itemsize, flops=2 * N ** 3, direct="matmul_mfma_kernel",
                        mfma_peak=157.3 if dt == np.float32 else 78.6,
                        desc=f"a @ b {np.dtype(dt).name} 8192^3 (eager matrix product on the matrix cores)",
                        steps=[lambda: a.dot(b)._force()],
                        cpu=lambda: ha[:m, :m] @ hb[:m, :m], cpu_frac=(m / N) ** 2, cpu_code="numpy.matmul")
        if name == "axis1_3d":
            shape = (256, 512, 1024)
            hv = rs.standard_normal(shape).astype(np.float32)
            vols = [dr.array(hv) for _ in range(sets_for(4 * hv.size))]
            return dict(dtype="f32", n=hv.size, nbytes=4 * hv.size + 4 * shape[0] * shape[2],
                        desc="sum(a, axis=1) f32 256x512x1024 (the middle axis)",
                        steps=[(lambda v=v: hip.run(ReduceEx(np.add, v, (1,)))) for v in vols],
                        cpu=lambda: hv[:64].sum(axis=1), cpu_frac=0.25, cpu_code="numpy.sum")
        if name == "matvec":
            N = 16384
            ha, hx = rs.standard_normal((N, N)).astype(np.float32), rs.standard_normal(N).astype(np.float32)
            x = dr.array(hx)
            mats = [dr.array(ha) for _ in range(sets_for(4 * N * N))]
            return dict(dtype="f32", n=N * N, nbytes=4 * N * N + 8 * N,
                        desc="a @ x f32 16384x16384 (the fused row reduction `@` builds)",
                        steps=[(lambda a=a: hip.run(ReduceEx(np.add, a * x, (1,)))) for a in mats],
                        cpu=lambda: ha[:N // 4] @ hx, cpu_frac=0.25, cpu_code="numpy.matmul")
        if name == "strided":
            n = 1 << 27
            hx = rs.standard_normal(n).astype(np.float32)
            vecs = [dr.array(hx) for _ in range(sets_for(6 * n))]
            return dict(dtype="f32", n=n // 2, nbytes=4 * n,
                        desc="x[::2] * 2 f32 n=2^27 (every second element: 8 B per result are needed, "
                             "12 B are fetched and written, whole cache lines)",
                        steps=[(lambda v=v: hip.run(v[::2] * 2.0)) for v in vecs],
                        cpu=lambda: hx[:n // 4:2] * np.float32(2.0), cpu_frac=0.25, cpu_code="numpy.multiply")
        if name == "strided2d":
            rows, cols = 8192, 16383
            hm = rs.standard_normal((rows, cols)).astype(np.float32)
            mats = [dr.array(hm) for _ in range(sets_for(4 * rows * cols + 4 * rows * 5461))]
            return dict(dtype="f32", n=rows * 5461, nbytes=8 * rows * 5461,
                        desc="m[:, ::3] * 2 f32 8192x16383 (every third element of every row: 8 B per result "
                             "are needed, 16 B are fetched and written)",
                        steps=[(lambda m=m: hip.run(m[:, ::3] * 2.0)) for m in mats],
                        cpu=lambda: hm[:rows // 4, ::3] * np.float32(2.0), cpu_frac=0.25, cpu_code="numpy.multiply")
        if name == "diff2":
            n = 1 << 27
            hx = rs.standard_normal(n).astype(np.float32)
            vecs = [dr.array(hx) for _ in range(sets_for(8 * n))]
            return dict(dtype="f32", n=n - 2, nbytes=8 * n - 8,
                        desc="x[2:] + x[:-2] - 2 x[1:-1] f32 n=2^27 (three shifted views of one vector)",
                        steps=[(lambda v=v: hip.run(v[2:] + v[:-2] - 2.0 * v[1:-1])) for v in vecs],
                        cpu=lambda: hx[2:n // 4] + hx[:n // 4 - 2] - np.float32(2.0) * hx[1:n // 4 - 1],
                        cpu_frac=0.25, cpu_code="numpy.add, numpy.subtract, numpy.multiply")
        if name == "stencil9":
            N = 8192
            hu = rs.uniform(0, 1, (N, N)).astype(np.float32)
            M = N - 2
            grids = [dr.array(hu) for _ in range(sets_for(4 * N * N + 4 * M * M))]

            def nine(u):
                return (u[:-2, :-2] + u[:-2, 1:-1] + u[:-2, 2:] + u[1:-1, :-2] + u[1:-1, 1:-1]
                        + u[1:-1, 2:] + u[2:, :-2] + u[2:, 1:-1] + u[2:, 2:]) * (1.0 / 9.0)
            return dict(dtype="f32", n=M * M, nbytes=4 * N * N + 4 * M * M,
                        desc="9-point stencil f32 8192^2 into a fresh 8190^2 array (rows not 16-byte periodic)",
                        steps=[(lambda u=u: hip.run(nine(u))) for u in grids],
                        cpu=lambda: hu[1:N // 8, 1:-1] + hu[:N // 8 - 1, 1:-1], cpu_frac=1 / 8,
                        cpu_code="numpy.add (two of the nine views)")
        if name == "transpose3d":
            shape = (512, 512, 1024)
            hv = rs.standard_normal(shape).astype(np.float32)
            nel = hv.size
            vols = [dr.array(hv) for _ in range(sets_for(8 * nel))]
            return dict(dtype="f32", n=nel, nbytes=8 * nel,
                        desc="a.T * 2 f32 512x512x1024 (all three axes reversed)",
                        steps=[(lambda v=v: hip.run(v.T * 2.0)) for v in vols],
                        cpu=lambda: hv[:, :, :256].T * np.float32(2.0), cpu_frac=0.25,
                        cpu_code="numpy.multiply")
        if name == "points3":
            n = 1 << 25
            hx = rs.standard_normal((n, 3)).astype(np.float32)
            hs, ht = rs.standard_normal(3).astype(np.float32), rs.standard_normal(3).astype(np.float32)
            pts = [dr.array(hx) for _ in range(sets_for(8 * n * 3))]
            sc, sh = dr.array(hs), dr.array(ht)
            return dict(dtype="f32", n=n * 3, nbytes=8 * n * 3,
                        desc="points * scale + shift f32, 2^25 points of 3 coordinates (rows of 12 "
                             "bytes: the row kernel without reductions, a lane per row)",
                        steps=[(lambda p=p: hip.run(p * sc + sh)) for p in pts],
                        cpu=lambda: hx[:n // 16] * hs + ht, cpu_frac=1 / 16,
                        cpu_code="numpy.multiply, add")
        if name == "softmax32k":
            R, N = 32000, 8192
            ha = rs.standard_normal((N, R)).astype(np.float32)
            mats = [dr.array(ha) for _ in range(sets_for(8 * N * R))]

            def soft(xp, a):
                e = xp.exp(a - a.max(axis=1, keepdims=True))
                return e / e.sum(axis=1, keepdims=True)
            return dict(dtype="f32", n=N * R, nbytes=8 * N * R,
                        desc="softmax along rows of 32000 f32, 8192 rows (a row of 128 KB held in "
                             "the registers of a block of 512 lanes)",
                        steps=[(lambda a=a: hip.run(soft(dr, a))) for a in mats],
                        cpu=lambda: soft(np, ha[:N // 16]), cpu_frac=1 / 16,
                        cpu_code="numpy.max, subtract, exp, sum, divide")
        if name in ("softmax", "layernorm", "rowmax"):
            N = 16384
            ha = rs.standard_normal((N, N)).astype(np.float32)
            mats = [dr.array(ha) for _ in range(sets_for(8 * N * N))]
            if name == "rowmax":
                return dict(dtype="f32", n=N * N, nbytes=8 * N * N,
                            desc="a - max(a, axis=1) f32 16384x16384 (the row kernel with next to no arithmetic)",
                            steps=[(lambda a=a: hip.run(a - a.max(axis=1, keepdims=True))) for a in mats],
                            cpu=lambda: ha[:N // 16] - ha[:N // 16].max(axis=1, keepdims=True), cpu_frac=1 / 16,
                            cpu_code="numpy.max, subtract")
            if name == "softmax":
                def soft(xp, a):
                    e = xp.exp(a - a.max(axis=1, keepdims=True))
                    return e / e.sum(axis=1, keepdims=True)
                return dict(dtype="f32", n=N * N, nbytes=8 * N * N,
                            desc="softmax along the rows f32 16384x16384 (row maximum, sum of "
                                 "exponentials and quotient in one kernel)",
                            steps=[(lambda a=a: hip.run(soft(dr, a))) for a in mats],
                            cpu=lambda: soft(np, ha[:N // 16]), cpu_frac=1 / 16,
                            cpu_code="numpy.max, subtract, exp, sum, divide")
            hg, hb = rs.standard_normal(N).astype(np.float32), rs.standard_normal(N).astype(np.float32)
            g, b = dr.array(hg), dr.array(hb)

            def norm(xp, a, w, c):
                d = a - a.mean(axis=1, keepdims=True)
                return d / xp.sqrt((d * d).mean(axis=1, keepdims=True) + 1e-5) * w + c
            return dict(dtype="f32", n=N * N, nbytes=8 * N * N + 8 * N,
                        desc="layer normalisation along the rows f32 16384x16384 (mean, variance "
                             "and the normalised rows in one kernel)",
                        steps=[(lambda a=a: hip.run(norm(dr, a, g, b))) for a in mats],
                        cpu=lambda: norm(np, ha[:N // 16], hg, hb), cpu_frac=1 / 16,
                        cpu_code="numpy.mean, subtract, multiply, sqrt, divide, add")
        if name in ("axis0", "axis1", "rowbcast", "transpose", "interior", "rows200"):
            N = 16384
            ha = rs.standard_normal((N, N)).astype(np.float32)
            if name in ("axis0", "axis1"):
                ax = int(name[-1])
                mats = [dr.array(ha) for _ in range(sets_for(4 * N * N))]
                return dict(dtype="f32", n=N * N, nbytes=4 * N * N + 4 * N,
                            desc=f"sum(a, axis={ax}) f32 16384x16384",
                            steps=[(lambda a=a: hip.run(ReduceEx(np.add, a, (ax,)))) for a in mats],
                            cpu=lambda: ha[:N // 4].sum(axis=ax), cpu_frac=0.25, cpu_code="numpy.sum")
            if name == "rows200":
                rows = N * N // 200
                hm = ha.reshape(-1)[:rows * 200].reshape(rows, 200)
                mats = [dr.array(hm) for _ in range(sets_for(4 * rows * 200))]
                return dict(dtype="f32", n=rows * 200, nbytes=4 * rows * 200 + 4 * rows,
                            desc=f"sum(a, axis=1) f32 {rows}x200 (rows of 200 contiguous elements)",
                            steps=[(lambda a=a: hip.run(ReduceEx(np.add, a, (1,)))) for a in mats],
                            cpu=lambda: hm[:rows // 4].sum(axis=1), cpu_frac=0.25, cpu_code="numpy.sum")
            mats = [dr.array(ha) for _ in range(sets_for(8 * N * N))]
            if name == "rowbcast":
                hr = rs.standard_normal(N).astype(np.float32)
                r = dr.array(hr)
                return dict(dtype="f32", n=N * N, nbytes=8 * N * N + 4 * N,
                            desc="a + row (broadcast) f32 16384x16384",
                            steps=[(lambda a=a: hip.run(a + r)) for a in mats],
                            cpu=lambda: ha[:N // 4] + hr, cpu_frac=0.25, cpu_code="numpy.add")
            if name == "interior":
                M = N - 2
                return dict(dtype="f32", n=M * M, nbytes=8 * M * M,
                            desc="m[1:-1,1:-1] * 2 f32 16384x16384 into a dense array (no row starts on 16 bytes)",
                            steps=[(lambda a=a: hip.run(a[1:-1, 1:-1] * 2.0)) for a in mats],
                            cpu=lambda: ha[1:N // 4, 1:-1] * np.float32(2.0), cpu_frac=0.25,
                            cpu_code="numpy.multiply")
            return dict(dtype="f32", n=N * N, nbytes=8 * N * N, desc="a.T * 2 f32 16384x16384",
                        steps=[(lambda a=a: hip.run(a.T * 2.0)) for a in mats],
                        cpu=lambda: ha[:, :N // 4].T * np.float32(2.0), cpu_frac=0.25,
                        cpu_code="numpy.multiply")
        if name == "stencil3d":
            N = 512
            hv = rs.uniform(0, 1, (N, N, N)).astype(np.float32)
            M = N - 2
            nbytes = 4 * N ** 3 + 4 * M ** 3
            vols = [dr.array(hv) for _ in range(sets_for(nbytes))]

            def sweep3(v):
                c = v[1:-1, 1:-1, 1:-1]
                v[1:-1, 1:-1, 1:-1] = (v[:-2, 1:-1, 1:-1] + v[2:, 1:-1, 1:-1] + v[1:-1, :-2, 1:-1]
                                       + v[1:-1, 2:, 1:-1] + v[1:-1, 1:-1, :-2] + v[1:-1, 1:-1, 2:]
                                       + c) * (1.0 / 7.0)
            return dict(dtype="f32", n=M ** 3, nbytes=nbytes, pair=True,
                        desc="7-point stencil f32 512^3, per sweep",
                        steps=[(lambda v=v: sweep3(v)) for v in vols],
                        cpu=lambda: hv[1:65, 1:-1, 1:-1] + hv[:64, 1:-1, 1:-1], cpu_frac=64 / N,
                        cpu_code="numpy.add (two of the seven views)")
        raise KeyError(name)

    def kernel_regions(replay, launches_per_replay, reps):
        """Durations (ms per launch group) of REGIONS timed regions of `reps` replays."""
        t_warm = time.perf_counter()
        while time.perf_counter() - t_warm < args.settle / 2:
            for _ in range(4):
                replay()
            hiprt.sync()
        out = []
        for _ in range(REGIONS):
            e0, e1 = hiprt.Event(), hiprt.Event()
            e0.record()
            for _ in range(reps):
                replay()
            e1.record()
            e1.synchronize()
            out.append(e0.elapsed_ms(e1) / (reps * launches_per_replay))
        return out

    def measure(name):
        t_gen = time.perf_counter()
        wl = make(name)
        t_gen = time.perf_counter() - t_gen
        steps = wl["steps"]
        R = len(steps)
        ring = [None] * R                 # the last R results stay alive: outputs rotate, too
        # first call: compile (or cache load) + run
        c0 = hiprt.counters()
        t0 = time.perf_counter()
        ring[0] = steps[0]()
        hiprt.sync()
        first_ms = (time.perf_counter() - t0) * 1e3
        c1 = hiprt.counters()
        for i in range(max(W, R)):
            ring[i % R] = steps[i % R]()
        hiprt.sync()
        # The GPU raises its clocks only under sustained load (an ALU-heavy kernel
        # measures ~25% slower during the first 30 ms): keep it busy before timing.
        t_warm = time.perf_counter()
        i = 0
        while time.perf_counter() - t_warm < args.settle:
            for _ in range(10):
                ring[i % R] = steps[i % R]()
                i += 1
            hiprt.sync()
        # whole-step throughput: exactly K steps, wall clock between two synchronisations
        t0 = time.perf_counter()
        for i in range(K):
            ring[i % R] = steps[i % R]()
        hiprt.sync()
        wall = time.perf_counter() - t0
        ms_per_step = wall / K * 1e3
        # kernel duration: record one step on every set (two for an aliasing update, which
        # alternates between a buffer's two allocations), replay the lot back to back
        per_set = 2 if wl.get("pair") else 1
        direct = wl.get("direct")     # a library kernel, launched without the fusion machinery
        if direct:
            cold = warm = lambda: steps[0]()
            kernel_names = [direct]
        else:
            with hip.record() as cold:
                for _ in range(per_set):
                    for j in range(R):
                        ring[j] = steps[j]()
            with hip.record() as warm:
                for _ in range(per_set):
                    ring[0] = steps[0]()
            names_by_func = {}
            for kern in hip._KERNELS.values():
                nm = kern.source.split('extern "C" __global__')[-1].split("void ")[1].split("(")[0]
                names_by_func[kern.func] = nm
                if kern.finalize:
                    names_by_func[kern.finalize] = nm + "_fin"
            kernel_names = sorted({names_by_func.get(f, "?") for f, *_ in cold.launches})
        reps = max(1, K // (R * per_set))
        cold_ms = kernel_regions(cold, 1 if direct else R * per_set, reps)
        warm_ms = kernel_regions(warm, 1 if direct else per_set, max(1, K // per_set))
        kernel_ms, kernel_min = statistics.median(cold_ms), min(cold_ms)
        warm_med = statistics.median(warm_ms)
        del cold, warm
        frac = wl["nbytes"] / kernel_ms / 1e6 / HBM_PEAK_GBPS
        res = {
            "workload": wl["desc"], "dtype": wl["dtype"], "elements": wl["n"],
            "kernel": kernel_names,
            "algorithmic_bytes": wl["nbytes"],
            "buffer_sets": R,
            "ms_per_step": round(ms_per_step, 5),
            "GBps": round(wl["nbytes"] / ms_per_step / 1e6, 1),
            "Gelem_per_s": round(wl["n"] / ms_per_step / 1e6, 2),
            "kernel_us": round(kernel_ms * 1e3, 2),
            "kernel_us_min": round(kernel_min * 1e3, 2),
            "kernel_us_regions": [round(v * 1e3, 2) for v in cold_ms],
            "kernel_GBps": round(wl["nbytes"] / kernel_ms / 1e6, 1),
            "roofline_frac": round(frac, 4),
            "roofline_frac_best_region": round(wl["nbytes"] / kernel_min / 1e6 / HBM_PEAK_GBPS, 4),
            "kernel_us_warm": round(warm_med * 1e3, 2),
            "roofline_frac_warm": round(wl["nbytes"] / warm_med / 1e6 / HBM_PEAK_GBPS, 4),
            # what limits the kernel (rocprofv3 VALUBusy / traffic in profiles/)
            "bound": {"bs64": "HBM (five float64 streams) and fp64 vector ALU",
                      "bs32": "fp32 vector ALU and HBM", "rand": "vector ALU (64-bit multiplies)",
                      "grid": "vector ALU and HBM", "stencil3d": "cache-line requests per compute unit",
                      "matmul32": "mfma", "matmul64": "mfma"}.get(name, "hbm"),
            **({"TFLOPs": round(wl["flops"] / kernel_ms / 1e9, 1),
                "mfma_frac": round(wl["flops"] / kernel_ms / 1e9 / wl["mfma_peak"], 4),
                "mfma_peak_TFLOPs": wl["mfma_peak"]} if wl.get("flops") else {}),
            "first_call_ms": round(first_ms, 2),
            "compile_ms": round((c1["compile_ns"] - c0["compile_ns"]) / 1e6, 2),
            "input_gen_s": round(t_gen, 2),
        }
        if wl.get("fresh") is not None:
            # A step over arrays never seen before (a new batch of data through the same
            # expression): neither the nodes nor a plan exist, only the structure has been
            # met.  F distinct sets of device arrays, more than the evaluated roots that
            # are kept alive for plan reuse, so that a set's turn never finds its plan.
            F = max(17, min(K, max(17, (96 << 30) // max(wl["nbytes"], 1))))
            fresh_steps = [wl["fresh"]() for _ in range(F)]
            hiprt.sync()
            hits = {"plan_hits": 0, "seen_hits": 0}
            walls, hosts = [], []
            for _ in range(5):
                t_warm = time.perf_counter()
                while time.perf_counter() - t_warm < args.settle / 2:
                    for j in range(R):
                        ring[j] = steps[j]()
                    hiprt.sync()
                s0 = dict(hip.STATS)
                t0 = time.perf_counter()
                for i in range(K):
                    ring[i % R] = fresh_steps[i % F]()
                t1 = time.perf_counter()
                hiprt.sync()
                t2 = time.perf_counter()
                walls.append((t2 - t0) / K)
                hosts.append((t1 - t0) / K)
                for k in hits:
                    hits[k] += hip.STATS[k] - s0[k]
            fresh_s = statistics.median(walls)
            res["fresh_step_us"] = round(fresh_s * 1e6, 2)
            res["fresh_host_us"] = round(statistics.median(hosts) * 1e6, 2)
            res["fresh_GBps"] = round(wl["nbytes"] / fresh_s / 1e9, 1)
            res["fresh_sets"] = F
            res["fresh_plan_hits"] = hits["plan_hits"]            # 0: no step found a plan
            res["fresh_structure_hits"] = hits["seen_hits"]       # steps whose structure had been met
            res["fresh_step_over_kernel"] = round(fresh_s / (kernel_ms * 1e-3), 3)
            del fresh_steps
        valu = profiled_figure("valu_instructions.txt", name)
        if valu is not None:
            # vector-ALU roofline: one wave instruction per SIMD every 4 cycles = 64 lanes
            # per CU and cycle
            peak = info["compute_units"] * 64 * info["clock_khz"] * 1e3
            res["valu_instr_per_element"] = valu
            res["valu_frac"] = round(valu * wl["n"] / (kernel_ms * 1e-3) / peak, 4)
            res["valu_peak_lane_instr_per_s"] = peak
        if "inputs" in wl and not args.no_parity:
            from oracle import accuracy
            inp = wl["inputs"]
            call, put = (a.get() for a in steps[0]())
            ocall, oput = orc.black_scholes(inp["S"], inp["K"], inp["T"], inp["r"], inp["sigma"])
            rep = accuracy.bs_report(call, put, ocall, oput, inp, detail=False)
            res["parity"] = {
                which: {"scaled_max_eps": r["scaled"]["max_eps"], "scaled_index": r["scaled"]["index"],
                        **{f"k{k}": {kk: e[kk] for kk in ("count", "max_ulp", "max_ulp_index", "max_rel",
                                                          "max_rel_index") if kk in e}
                           for k, e in r["subsets"].items() if k in (1, 4, 8)}}
                for which, r in rep.items()}
            res["parity"]["subsets"] = "k: options with |oracle price| >= 2^-k max(S, K)"
            if name == "bs32":
                # Why the float32 bar is wider than two ulp: NumPy's own float32 prices are
                # several ulp from the true ones (the float64 evaluation of the same
                # inputs).  Largest distance from that value, in float32 ulp, of this
                # backend's prices and of NumPy's, on options with |price| >= 2^-k max(S, K).
                truth = orc.black_scholes(*(inp[k].astype(np.float64) for k in "SKT"),
                                          inp["r"], inp["sigma"])
                scale = np.maximum(inp["S"], inp["K"]).astype(np.float64)
                vs = {}
                for which, got, ref, t in (("call", call, ocall, truth[0]), ("put", put, oput, truth[1])):
                    ulp = np.spacing(np.abs(t).astype(np.float32)).astype(np.float64)
                    for k in (1, 2, 4):
                        m = np.abs(t) >= scale * 2.0 ** -k
                        if m.any():
                            vs[f"{which}_k{k}"] = {
                                "device_ulp": round(float(np.max(np.abs(got - t)[m] / ulp[m])), 2),
                                "numpy_float32_ulp": round(float(np.max(np.abs(ref - t)[m] / ulp[m])), 2)}
                res["parity"]["ulp_from_float64_value"] = vs
                del truth, scale
            del call, put, ocall, oput
        if "sets" in wl and not args.no_parity:
            # The stream mix alone: the same three loads and two stores per element with a
            # body of two multiply-adds, launched as this workload's kernel is (the float64
            # kernel keeps its blocks for several runs because of its tables in LDS).
            def mix(S, K_, T):
                return hip.run_multi([S * K_ + T, S - K_ * T])
            res["stream_mix"] = {"body": "S*K+T, S-K*T (same operands and results)"}
            for label, cap in (("one_run_per_block", 0), ("blocks_that_stay", hip.TUNE["table_blocks"])):
                hip.set_tune(flat_cap=cap)
                try:
                    for S, K_, T in wl["sets"]:
                        ring[0] = mix(S, K_, T)
                    with hip.record() as cold_mix:
                        for j, (S, K_, T) in enumerate(wl["sets"]):
                            ring[j] = mix(S, K_, T)
                    mix_ms = statistics.median(kernel_regions(cold_mix, R, max(1, K // R)))
                    del cold_mix
                finally:
                    hip.set_tune(flat_cap=0)
                res["stream_mix"][label] = {"kernel_us": round(mix_ms * 1e3, 2),
                                            "frac": round(wl["nbytes"] / mix_ms / 1e6 / HBM_PEAK_GBPS, 4)}
        if not args.no_unfused:
            # one kernel per node: its temporaries are re-read by the next kernel, so this
            # leg gets the cache policy that suits it (streams stay cacheable up to the
            # size of the last-level cache)
            policy = {k: hip.TUNE[k] for k in ("cache_mib", "ntl_mib")}
            hip.set_tune(cache_mib=200, ntl_mib=320)
            hip.set_fused(False)
            try:
                l0, k0 = hip.STATS["launches"], hiprt.counters()
                t0 = time.perf_counter()
                ring[0] = steps[0]()
                hiprt.sync()
                # first call: every node's kernel compiled, as one translation unit
                res["unfused_first_call_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
                res["unfused_compile_ms"] = round((hiprt.counters()["compile_ns"] - k0["compile_ns"]) / 1e6, 2)
                res["unfused_kernels"] = hip.STATS["launches"] - l0
                ring[0] = steps[0]()
                hiprt.sync()
                reps_u = max(3, K // 4)
                t0 = time.perf_counter()
                for _ in range(reps_u):
                    ring[0] = steps[0]()
                hiprt.sync()
                u_ms = (time.perf_counter() - t0) / reps_u * 1e3
            finally:
                hip.set_fused(True)
                hip.set_tune(**policy)
            res["unfused_ms_per_step"] = round(u_ms, 4)
            res["unfused_Gelem_per_s"] = round(wl["n"] / u_ms / 1e6, 2)
            res["fused_speedup_vs_unfused"] = round(u_ms / ms_per_step, 2)
        if not args.no_cpu:
            wl["cpu"]()                     # warm-up
            times = []
            budget = args.cpu_seconds if name == HEADLINE else 0.0
            t_all = time.perf_counter()
            while len(times) < 3 or time.perf_counter() - t_all < budget:
                t0 = time.perf_counter()
                wl["cpu"]()
                times.append(time.perf_counter() - t0)
            cpu_s = statistics.median(times)
            cpu_bytes = wl["nbytes"] * wl["cpu_frac"]
            res["cpu"] = {"GBps": round(cpu_bytes / cpu_s / 1e9, 2),
                          "Gelem_per_s": round(wl["n"] * wl["cpu_frac"] / cpu_s / 1e9, 3),
                          "seconds": round(cpu_s, 3), "passes": len(times),
                          "sample_fraction": wl["cpu_frac"], "code": wl["cpu_code"]}
        del ring, wl, steps
        return res

    names = {"all": ["sumsq", "saxpy", "horner", "bs32", "bs64", "jacobi"],
             "next": ["dot", "axis0", "axis1", "axis1_3d", "matvec", "rows200", "rowbcast", "transpose",
                      "transpose3d", "interior", "diff2", "stencil9", "stencil3d", "grid", "rand",
                      "softmax", "softmax32k", "layernorm", "rowmax", "strided", "strided2d", "points3"]}.get(args.workload, [args.workload])
    HEADLINE = "sumsq" if "sumsq" in names else names[0]
    results = {}
    for name in names:
        results[name] = measure(name)
        print(f"[bench] {name}: {results[name]}", file=sys.stderr, flush=True)
        hip.forget()
        hiprt.pool_trim()

    # the plain streaming copy (1 GiB in, 1 GiB out): measured ceiling of the memory
    # system for a read+write stream, and the known-size kernel against which the
    # profiler's FETCH_SIZE / WRITE_SIZE counters are calibrated
    copy = None
    if not args.no_copy:
        nb = 1 << 30
        a, b = hip.ndarray((nb // 4,), np.float32), hip.ndarray((nb // 4,), np.float32)
        hiprt.fill32(a.ptr, 0x3F800000, nb // 4)
        for _ in range(3):
            hiprt.copy_kernel(b.ptr, a.ptr, nb)
        hiprt.sync()
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record()
        for _ in range(10):
            hiprt.copy_kernel(b.ptr, a.ptr, nb)
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / 10
        copy = {"bytes_read": nb, "bytes_written": nb, "us": round(ms * 1e3, 1),
                "GBps": round(2 * nb / ms / 1e6, 1), "frac": round(2 * nb / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        del a, b

    head = results[HEADLINE]
    worst = min(results, key=lambda k: results[k]["roofline_frac"])
    line = {
        "metric": METRIC,
        "value": head["GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic (numpy RandomState(0), resident in HBM before timing; "
                f"{head['buffer_sets']} buffer sets in rotation)",
        "config": {"workload": head["workload"], "name": HEADLINE,
                   "elements": head["elements"], "Gelem_per_s": head["Gelem_per_s"],
                   "device": info["name"] or info["arch"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "hbm", "achieved": head["kernel_GBps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["roofline_frac"], "traffic": None,
                     "kernel": head["kernel"][0], "kernel_us": head["kernel_us"],
                     "kernel_us_min": head["kernel_us_min"], "timed_regions": REGIONS,
                     "frac_warm": head["roofline_frac_warm"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"],
                     "min_frac": results[worst]["roofline_frac"], "min_frac_config": worst,
                     "frac_by_config": {k: v["roofline_frac"] for k, v in results.items()}},
        "configs": results,
    }
    if copy is not None:
        line["copy_kernel"] = copy
    # HBM traffic per launch comes from a profiler run (counters cannot be read here): it
    # is quoted only for the very kernels this run launched; a figure taken from another
    # version of a kernel is dropped and flagged
    for name, res in results.items():
        traffic, kernels = measured_traffic(name)
        if traffic is None:
            continue
        ran = sorted(k for k in res["kernel"] if not k.endswith("_fin"))
        if kernels == ran:
            res["hbm_traffic_bytes"] = traffic
            res["hbm_traffic_over_algorithmic"] = round(traffic / res["algorithmic_bytes"], 4)
        else:
            res["hbm_traffic_bytes"] = None
            res["hbm_traffic_stale"] = {"profiled": kernels, "ran": ran}
    if head.get("hbm_traffic_bytes") is not None:
        line["roofline"]["traffic"] = head["hbm_traffic_bytes"]
        line["roofline"]["traffic_source"] = "profiles/hbm_traffic.txt (rocprofv3 --pmc, calibrated)"
    elif "hbm_traffic_stale" in head:
        line["roofline"]["traffic_stale"] = True
    if "cpu" in head:
        line["cpu_baseline"] = {
            "value": head["cpu"]["GBps"], "unit": "GB/s", "cores": 1, "kind": "port",
            "code": head["cpu"]["code"] + " (NumPy node by node, restating the reference's cpu.py)",
            "host_cores_available": os.cpu_count(),
            "sample": f"{head['workload']}: NumPy node-by-node evaluation of "
                      f"{head['cpu']['sample_fraction']:g} of the workload, median of "
                      f"{head['cpu']['passes']} passes ({head['cpu']['seconds']} s per pass); "
                      "NumPy ufuncs run on one core"}
    if "unfused_ms_per_step" in head:
        line["unfused"] = {"ms_per_step": head["unfused_ms_per_step"],
                           "Gelem_per_s": head["unfused_Gelem_per_s"],
                           "kernels": head["unfused_kernels"],
                           "fused_speedup": head["fused_speedup_vs_unfused"]}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
