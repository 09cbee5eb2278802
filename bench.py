#!/usr/bin/env python3
"""Benchmark of the fused hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME|all]

A step is one pass of the hot path over one batch: build the lazy expression,
trace it, look the kernel up in the cache and launch it on inputs that already
sit in HBM (for the stencil: one sweep; for the reduction: body + finalize).
Prints ONE JSON line.  Its top-level fields describe the headline workload
(degree-8 Horner polynomial, float32, n = 2^26); `configs` carries the same
figures for every configuration.

Per configuration:
  value / GBps        algorithmic bytes * steps / wall time of the timed region
                      (whole step, host side included)
  roofline            algorithmic bytes / average kernel duration, measured with HIP
                      events on the library's stream around back-to-back replays of
                      the recorded launches, against 8 TB/s
  unfused             the same expression with one kernel per DAG node
  cpu_baseline        the NumPy node-by-node evaluation (oracle/numpy_oracle.py, a port
                      of the reference's CPU backend) on this machine's host cores
"""
import argparse
import contextlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
METRIC = "fused-kernel effective HBM GB/s (% of MI355X peak); Gelem/s vs unfused"


def measured_traffic(name):
    """HBM bytes per launch of a workload's kernel as measured with rocprofv3
    counters (FETCH_SIZE + WRITE_SIZE, calibrated on the copy kernel); the figures
    live in profiles/hbm_traffic.txt as `<workload> <bytes>` lines."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    try:
        with open(path) as fh:
            for ln in fh:
                parts = ln.split()
                if len(parts) >= 2 and parts[0] == name:
                    return int(float(parts[1]))
    except OSError:
        pass
    return None


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all",
                    help="horner (headline) | saxpy | bs32 | bs64 | jacobi | sumsq | all (these six); "
                         "dot | axis0 | axis1 | rowbcast | transpose | grid | next (these six: the "
                         "operations either side of the five configurations); "
                         "matmul32 | matmul64 (the eager matrix product)")
    ap.add_argument("--settle", type=float, default=0.25,
                    help="seconds of untimed load before each timed region (clock ramp-up)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0,
                    help="CPU time spent on the headline workload's baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-copy", action="store_true", help="skip the plain-copy ceiling leg")
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

    # ---- the workloads: (inputs on device, step function, bytes, elements, cpu function)
    def make(name):
        inp = orc.make_inputs(name) if name in ("saxpy", "horner", "bs32", "bs64", "jacobi",
                                                "sumsq") else None
        if name == "saxpy":
            x, y = dr.array(inp["x"]), dr.array(inp["y"])
            n = inp["x"].size
            return dict(dtype="f32", n=n, nbytes=12 * n, desc="SAXPY z=a*x+y f32 n=2^24",
                        step=lambda: hip.run(inp["a"] * x + y),
                        cpu=lambda: orc.saxpy(inp["a"], inp["x"], inp["y"]), cpu_frac=1.0)
        if name == "horner":
            x = dr.array(inp["x"])
            n = inp["x"].size
            return dict(dtype="f32", n=n, nbytes=8 * n,
                        desc="Horner degree-8 polynomial f32 n=2^26",
                        step=lambda: hip.run(horner_expr(inp["c"], x)),
                        cpu=lambda: orc.horner(inp["c"], inp["x"]), cpu_frac=1.0)
        if name in ("bs32", "bs64"):
            S, K_, T = dr.array(inp["S"]), dr.array(inp["K"]), dr.array(inp["T"])
            n = inp["S"].size
            size = inp["S"].dtype.itemsize
            m = n // 4       # CPU sample: a quarter of the options
            return dict(dtype="f32" if size == 4 else "f64", n=n, nbytes=5 * size * n,
                        desc=f"Black-Scholes call+put {'f32' if size == 4 else 'f64'} n=2^25",
                        step=lambda: hip.run_multi(list(orc.black_scholes_expr(
                            dr, S, K_, T, inp["r"], inp["sigma"]))),
                        cpu=lambda: orc.black_scholes(inp["S"][:m], inp["K"][:m], inp["T"][:m],
                                                      inp["r"], inp["sigma"]), cpu_frac=0.25)
        if name == "jacobi":
            u = dr.array(inp["u"])
            N = inp["u"].shape[0]

            def sweep():
                u[1:-1, 1:-1] = 0.25 * (u[:-2, 1:-1] + u[2:, 1:-1] + u[1:-1, :-2] + u[1:-1, 2:])
            return dict(dtype="f32", n=(N - 2) * (N - 2), nbytes=4 * N * N + 4 * (N - 2) * (N - 2),
                        desc="Jacobi 5-point f32 8192x8192, per sweep", step=sweep, pair=True,
                        cpu=lambda: orc.jacobi(inp["u"], 1), cpu_frac=1.0)
        if name == "sumsq":
            x, y, w = dr.array(inp["x"]), dr.array(inp["y"]), dr.array(inp["w"])
            n = inp["x"].size
            m = n // 4
            return dict(dtype="f64", n=n, nbytes=24 * n, desc="sum((x-y)**2*w) f64 n=2^27",
                        step=lambda: hip.run(ReduceEx(np.add, (x - y) ** 2 * w)),
                        cpu=lambda: orc.sumsq(inp["x"][:m], inp["y"][:m], inp["w"][:m]),
                        cpu_frac=0.25)
        # ---- operations either side of the five configurations (no CPU sample kept small)
        rs = np.random.RandomState(0)
        if name == "dot":
            n = 1 << 27
            hx, hy = rs.standard_normal(n), rs.standard_normal(n)
            x, y = dr.array(hx), dr.array(hy)
            return dict(dtype="f64", n=n, nbytes=16 * n, desc="dot(x, y) f64 n=2^27 (fused multiply-reduce)",
                        step=lambda: hip.run(ReduceEx(np.add, x * y)),
                        cpu=lambda: np.dot(hx[:n // 4], hy[:n // 4]), cpu_frac=0.25)
        if name == "grid":
            n = 1 << 26
            c = orc.make_inputs("horner")["c"]
            g = dr.linspace(-2.0, 2.0, n, dtype=np.float32)     # lazy: computed inside the kernel
            m = n // 16
            return dict(dtype="f32", n=n, nbytes=4 * n,
                        desc="Horner degree-8 on linspace(-2, 2, n) f32 n=2^26 (grid generated in the kernel)",
                        step=lambda: hip.run(horner_expr(c, g)),
                        cpu=lambda: orc.horner(c, np.linspace(-2.0, 2.0, m, dtype=np.float32)),
                        cpu_frac=1 / 16)
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
                        step=lambda: a.dot(b)._force(),
                        cpu=lambda: ha[:m, :m] @ hb[:m, :m], cpu_frac=(m / N) ** 2)
        if name in ("axis0", "axis1", "rowbcast", "transpose"):
            N = 16384
            ha = rs.standard_normal((N, N)).astype(np.float32)
            a = dr.array(ha)
            if name in ("axis0", "axis1"):
                ax = int(name[-1])
                return dict(dtype="f32", n=N * N, nbytes=4 * N * N + 4 * N,
                            desc=f"sum(a, axis={ax}) f32 16384x16384",
                            step=lambda: hip.run(ReduceEx(np.add, a, (ax,))),
                            cpu=lambda: ha[:N // 4].sum(axis=ax), cpu_frac=0.25)
            if name == "rowbcast":
                hr = rs.standard_normal(N).astype(np.float32)
                r = dr.array(hr)
                return dict(dtype="f32", n=N * N, nbytes=8 * N * N + 4 * N,
                            desc="a + row (broadcast) f32 16384x16384",
                            step=lambda: hip.run(a + r), cpu=lambda: ha[:N // 4] + hr, cpu_frac=0.25)
            return dict(dtype="f32", n=N * N, nbytes=8 * N * N, desc="a.T * 2 f32 16384x16384",
                        step=lambda: hip.run(a.T * 2.0),
                        cpu=lambda: ha[:, :N // 4].T * np.float32(2.0), cpu_frac=0.25)
        raise KeyError(name)

    def measure(name):
        t_gen = time.perf_counter()
        wl = make(name)
        t_gen = time.perf_counter() - t_gen
        step = wl["step"]
        # first call: compile (or cache load) + run
        c0 = hiprt.counters()
        t0 = time.perf_counter()
        keep = step()
        hiprt.sync()
        first_ms = (time.perf_counter() - t0) * 1e3
        c1 = hiprt.counters()
        for _ in range(W):
            keep = step()
        hiprt.sync()
        # The GPU raises its clocks only under sustained load (an ALU-heavy kernel
        # measures ~25% slower during the first 30 ms): keep it busy before timing.
        t_warm = time.perf_counter()
        while time.perf_counter() - t_warm < args.settle:
            for _ in range(10):
                keep = step()
            hiprt.sync()
        # whole-step throughput: K steps, wall clock between two synchronisations
        t0 = time.perf_counter()
        for _ in range(K):
            keep = step()
        hiprt.sync()
        wall = time.perf_counter() - t0
        ms_per_step = wall / K * 1e3
        # kernel duration: record the launches of one step (two for the ping-pong
        # stencil, which alternates between two buffers), replay them back to back
        if wl.get("direct"):     # a library kernel, launched without the fusion machinery
            plan = step
        with (hip.record() if not wl.get("direct") else contextlib.nullcontext()) as rec:
            keep = step()
            if wl.get("pair"):
                keep = step()
        if not wl.get("direct"):
            plan = rec
        names_by_func = {}
        for kern in hip._KERNELS.values():
            nm = kern.source.split('extern "C" __global__')[-1].split("void ")[1].split("(")[0]
            names_by_func[kern.func] = nm
            if kern.finalize:
                names_by_func[kern.finalize] = nm + "_fin"
        kernel_names = [wl["direct"]] if wl.get("direct") else \
            sorted({names_by_func.get(f, "?") for f, *_ in plan.launches})
        steps_per_replay = 2 if wl.get("pair") else 1
        reps = max(1, K // steps_per_replay)
        t_warm = time.perf_counter()
        while time.perf_counter() - t_warm < args.settle / 2:
            for _ in range(10):
                plan()
            hiprt.sync()
        e0, e1 = hiprt.Event(), hiprt.Event()
        e0.record()
        for _ in range(reps):
            plan()
        e1.record()
        e1.synchronize()
        kernel_ms = e0.elapsed_ms(e1) / (reps * steps_per_replay)
        del plan
        res = {
            "workload": wl["desc"], "dtype": wl["dtype"], "elements": wl["n"],
            "kernel": kernel_names,
            "algorithmic_bytes": wl["nbytes"],
            "ms_per_step": round(ms_per_step, 5),
            "GBps": round(wl["nbytes"] / ms_per_step / 1e6, 1),
            "Gelem_per_s": round(wl["n"] / ms_per_step / 1e6, 2),
            "kernel_us": round(kernel_ms * 1e3, 2),
            "kernel_GBps": round(wl["nbytes"] / kernel_ms / 1e6, 1),
            "roofline_frac": round(wl["nbytes"] / kernel_ms / 1e6 / HBM_PEAK_GBPS, 4),
            # what limits the kernel (rocprofv3 VALUBusy / traffic in profiles/)
            "bound": {"bs64": "fp64 vector ALU (VALUBusy 89%), not HBM",
                      "bs32": "fp32 vector ALU (VALUBusy ~100%) and HBM",
                      "matmul32": "mfma", "matmul64": "mfma"}.get(name, "hbm"),
            **({"TFLOPs": round(wl["flops"] / kernel_ms / 1e9, 1),
                "mfma_frac": round(wl["flops"] / kernel_ms / 1e9 / wl["mfma_peak"], 4),
                "mfma_peak_TFLOPs": wl["mfma_peak"]} if wl.get("flops") else {}),
            "first_call_ms": round(first_ms, 2),
            "compile_ms": round((c1["compile_ns"] - c0["compile_ns"]) / 1e6, 2),
            "input_gen_s": round(t_gen, 2),
        }
        if not args.no_unfused:
            hip.set_fused(False)
            try:
                l0 = hip.STATS["launches"]
                keep = step()
                hiprt.sync()
                res["unfused_kernels"] = hip.STATS["launches"] - l0
                keep = step()
                hiprt.sync()
                reps_u = max(3, K // 4)
                t0 = time.perf_counter()
                for _ in range(reps_u):
                    keep = step()
                hiprt.sync()
                u_ms = (time.perf_counter() - t0) / reps_u * 1e3
            finally:
                hip.set_fused(True)
            res["unfused_ms_per_step"] = round(u_ms, 4)
            res["unfused_Gelem_per_s"] = round(wl["n"] / u_ms / 1e6, 2)
            res["fused_speedup_vs_unfused"] = round(u_ms / ms_per_step, 2)
        if not args.no_cpu:
            wl["cpu"]()                     # warm-up
            times = []
            budget = args.cpu_seconds if name == "horner" else 0.0
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
                          "sample_fraction": wl["cpu_frac"]}
        del keep, wl
        return res

    names = {"all": ["horner", "saxpy", "bs32", "bs64", "jacobi", "sumsq"],
             "next": ["dot", "axis0", "axis1", "rowbcast", "transpose", "grid"]}.get(args.workload,
                                                                             [args.workload])
    results = {}
    for name in names:
        results[name] = measure(name)
        print(f"[bench] {name}: {results[name]}", file=sys.stderr, flush=True)
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

    head = results.get("horner") or results[names[0]]
    head_name = "horner" if "horner" in results else names[0]
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
        "data": "synthetic (numpy RandomState(0), resident in HBM before timing)",
        "config": {"workload": head["workload"], "name": head_name,
                   "elements": head["elements"], "Gelem_per_s": head["Gelem_per_s"],
                   "device": info["name"] or info["arch"], "compute_units": info["compute_units"]},
        "roofline": {"bound": "hbm", "achieved": head["kernel_GBps"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": head["roofline_frac"], "traffic": None,
                     "kernel": head["kernel"][0], "kernel_us": head["kernel_us"],
                     "algorithmic_bytes_per_launch": head["algorithmic_bytes"]},
        "configs": results,
    }
    if copy is not None:
        line["copy_kernel"] = copy
    traffic = measured_traffic(head_name)
    if traffic is not None:
        line["roofline"]["traffic"] = traffic
        line["roofline"]["traffic_source"] = "profiles/hbm_traffic.txt (rocprofv3 --pmc, calibrated)"
    if "cpu" in head:
        line["cpu_baseline"] = {
            "value": head["cpu"]["GBps"], "unit": "GB/s", "cores": 1, "kind": "port",
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
