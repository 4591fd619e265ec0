"""Benchmark of the fused Elemwise / CAReduce path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Workload (``config.workload``): the CAReduce configuration, float32 (8192, 8192):
sum and max along axis 1, sum along axis 0, sum over all axes, prod along
axis 1.  One step runs the five reductions once on device-resident inputs;
``value`` is their algorithmic bytes divided by the step time (HIP events on the
library's stream around the K timed steps).  ``roofline`` describes the dominant
kernel (the row-form reduction) from per-launch HIP events taken in a second
run of the same K steps; ``cpu_baseline`` times the oracle's C restatement of
the reference's sequential CAReduce loops on this host for the same five
reductions.  ``other_configs`` lists the remaining four configurations,
measured the same way with fewer steps.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0


def _device_function(th, W, graph, vals):
    from theano_amd.hip import HipArray
    ins, outs = graph
    f = th.function(ins, [th.Out(o, device=True) for o in outs])
    dev = [HipArray.from_numpy(v) if v.size > 1 else v for v in vals]
    return f, dev


def _time_steps(hip, step, steps, warmup):
    for _ in range(warmup):
        step()
    hip.sync()
    t0 = time.perf_counter()
    hip.timer_start()
    for _ in range(steps):
        step()
    gpu_ms = hip.timer_stop()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return gpu_ms / steps, wall_ms / steps


def _profile_steps(hip, step, steps):
    with hip.profile() as p:
        for _ in range(steps):
            step()
    return p.kernels


def _cpu_baseline_c2(W):
    """The reference's CAReduce loops (serial, float64 accumulator) restated in
    oracle/careduce.c, run once over the full inputs of the five reductions."""
    from oracle import graph_ref as G
    x = W.c2_inputs("sum_axis1", "full")[0]
    xp = W.c2_inputs("prod_axis1", "full")[0]
    jobs = [(x, "Add", (1,), "float64"), (x, "Maximum", (1,), "float32"), (x, "Add", (0,), "float64"),
            (x, "Add", None, "float64"), (xp, "Mul", (1,), "float64")]
    G.careduce(x[:64], "Add", (1,), "float64", "float32")  # load the library
    t0 = time.perf_counter()
    nbytes = 0
    for arr, op, axis, acc in jobs:
        G.careduce(arr, op, axis, acc, "float32")
        nbytes += arr.nbytes
    dt = time.perf_counter() - t0
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "the five reductions once over the full (8192, 8192) float32 inputs, %.2f s; CAReduce loops "
                      "are single-threaded in the reference" % dt}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the other four configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no sharding); got --gpus %d" % args.gpus)

    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import theano_amd as th
    from theano_amd import hip
    import workloads as W

    hip.init()
    info = hip.device_info()

    # ---- headline: config 2 -----------------------------------------------------------------
    fns = []
    total_bytes = 0
    x_dev = {}
    for case in W.C2_CASES:
        vals = W.c2_inputs(case, "full")
        key = "prod" if case == "prod_axis1" else "normal"
        f, dev = _device_function(th, W, W.c2_graph(case), vals)
        if key in x_dev:
            dev = x_dev[key]
        else:
            x_dev[key] = dev
        fns.append((case, f, dev))
        total_bytes += W.algorithmic_bytes("c2_" + case)

    def step():
        for _, f, dev in fns:
            f(*dev)

    gpu_ms, wall_ms = _time_steps(hip, step, args.steps, args.warmup)
    kernels = _profile_steps(hip, step, args.steps)
    value = total_bytes / (gpu_ms * 1e-3) / 1e9

    # dominant kernel: the one with the largest share of the profiled time
    dom = max(kernels.items(), key=lambda kv: kv[1][1])
    dom_name, (dom_n, dom_ms) = dom
    dom_avg_us = dom_ms / dom_n * 1e3
    per_launch = 8192 * 8192 * 4 + 8192 * 4   # bytes one launch of a row / column reduction moves by definition
    achieved = per_launch / (dom_avg_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None, "kernel": dom_name,
                "avg_launch_us": round(dom_avg_us, 2), "launches": dom_n}

    per_case = {}
    for case, f, dev in fns:
        ms, _ = _time_steps(hip, lambda: f(*dev), max(5, args.steps // 2), 2)
        b = W.algorithmic_bytes("c2_" + case)
        per_case[case] = {"us": round(ms * 1e3, 2), "GB/s": round(b / (ms * 1e-3) / 1e9, 1),
                          "frac_of_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    others = {}
    if not args.no_others:
        specs = [("c1", W.c1_graph(), W.c1_inputs("full"), "c1"),
                 ("c3_fwd", W.c3_graph(with_grad=False), W.c3_inputs("full", with_grad=False), "c3_fwd"),
                 ("c3_fwd_grad", W.c3_graph(), W.c3_inputs("full"), "c3_fwd_grad"),
                 ("c4_elemwise", W.c4_graph("elemwise"), W.c4_inputs("full"), "c4_elemwise"),
                 ("c4_sum", W.c4_graph("sum"), W.c4_inputs("full"), "c4_sum"),
                 ("c4_anyall", W.c4_graph("anyall"), W.c4_inputs("full", "anyall"), "c4_anyall"),
                 ("c5_fwd", W.c5_graph(with_grad=False), W.c5_inputs("full", with_grad=False), "c5_fwd"),
                 ("c5_grad", W.c5_graph(forward=False), W.c5_inputs("full"), "c5_grad")]
        for name, graph, vals, bname in specs:
            f, dev = _device_function(th, W, graph, vals)
            ms, wms = _time_steps(hip, lambda: f(*dev), max(5, args.steps // 5), 2)
            b = W.algorithmic_bytes(bname)
            n_k = sum(1 for n in f.toposort() if type(n.op).__name__ in ("HipElemwise", "HipCAReduce", "HipRowChain"))
            others[name] = {"us": round(ms * 1e3, 2), "GB/s": round(b / (ms * 1e-3) / 1e9, 1),
                            "frac_of_peak": round(b / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "kernels_per_step": n_k}
            del f, dev

    cpu = None if args.no_cpu else _cpu_baseline_c2(W)

    line = {
        "metric": "achieved HBM GB/s for fused Elemwise+CAReduce at 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(gpu_ms, 5), "wall_ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 data, f64 accumulators", "data": "synthetic",
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "config": {"workload": "config 2: CAReduce on float32 (8192, 8192): sum axis=1, max axis=1, sum axis=0, "
                               "sum all axes, prod axis=1; one step = the five reductions",
                   "algorithmic_bytes_per_step": total_bytes, "device": info["arch"],
                   "compute_units": info["compute_units"]},
        "roofline": roofline, "cpu_baseline": cpu, "per_reduction": per_case, "other_configs": others,
        "kernels": {k: {"launches": n, "avg_us": round(ms / n * 1e3, 2)} for k, (n, ms) in kernels.items()},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
