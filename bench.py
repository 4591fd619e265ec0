"""Benchmark of the fused Elemwise / CAReduce path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Workload (``config.workload``): the CAReduce configuration, float32 (8192, 8192):
sum and max along axis 1, sum along axis 0, sum over all axes, prod along
axis 1.  One step runs the five reductions once on device-resident inputs;
``value`` is their algorithmic bytes divided by the step time (HIP events on the
library's stream around the K timed steps).  ``roofline`` describes the dominant
kernel, the row-form reduction behind ``sum(axis=1)``: K launches back to back
between two HIP events on the launch stream, once alternating between two
input arrays and once over one array.  The input is 268 MB and the device's
last-level cache 256 MB, so a launch that follows one over the same array runs
a few percent faster than one that follows a different array; a step holds one
launch of each kind, and the average of the two loops divides the kernel's
algorithmic bytes.  ``cpu_baseline`` times the oracle's C restatement of the
reference's loops on this host.  ``other_configs`` lists the remaining four
configurations (and max_and_argmax of the configuration-2 matrix) over input
sets that rotate (so that no set is still cached when it is used again: ``us``,
the median of nine runs of max(K, 50) steps, ``min_us`` the fastest of them) and over one
set (``same_input_us``), each with the symbols of the kernels it launches.  Every
timed leg starts on a device that has been kept busy for 40 ms (``_settle``).
"""
import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0

# Configurations whose kernels move fewer bytes than the passes they are priced at: config 5 forward runs as
# one held-chain kernel that reads x once and writes y once (2 x 51 380 224 float16 values + the per-channel
# operands), where the configuration counts a statistics pass over x as well.
REAL_BYTES = {"c5_fwd": 2 * 256 * 256 * 28 * 28 * 2 + 2 * 256 * 2}

TRAFFIC_SUMMARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "all_configs_hbm_traffic.txt")


def _traffic(symbol, grid=None):
    """HBM bytes per launch of the kernel `symbol` as the hardware counters measured them (rocprofv3 --pmc
    FETCH_SIZE, then WRITE_SIZE, each scaled by what the same counter reads for the --copy-probe kernel of
    known size): read from the tracked summary of those runs, whose table lines are
    `<kernel symbol> <grid> <launches> <FETCH_SIZE> <WRITE_SIZE> <HBM bytes> ...`.  None, with a warning,
    when the summary has no line for this kernel (its text changed since the counters were taken)."""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            rows = [l.split() for l in f if l.startswith("thx_")]
    except OSError:
        rows = []
    hits = [r for r in rows if r[0] == symbol and len(r) >= 6 and (grid is None or r[1] == str(grid))]
    if not hits:
        sys.stderr.write("bench.py: no measured HBM traffic for %s in %s; roofline.traffic is null\n"
                         % (symbol, os.path.relpath(TRAFFIC_SUMMARY)))
        return None
    return int(float(hits[0][5]))


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


SETTLE_MS = [40.0]


def _settle(hip, step, ms=None, chunk=10):
    """Run `step` until the device has been busy for about `ms` milliseconds.  After an idle period the
    device needs some 20 ms of continuous work to reach its steady clocks: the arithmetic-heavy kernels (the
    held chain of config 5, the tile kernels of config 4, argmax) run 5 - 20 % slower in between, the plain
    streaming reductions do not change.  Untimed."""
    busy = 0.0
    ms = SETTLE_MS[0] if ms is None else ms
    while busy < ms:
        hip.timer_start()
        for _ in range(chunk):
            step()
        busy += hip.timer_stop()


def _symbol(profile_name):
    """Kernel symbol (what rocprofv3 lists) of a 'functor|plan' profile name."""
    functor, plan = profile_name.split("|", 1)
    return "thx_" + "".join(c if c.isalnum() else "_" for c in plan) + "_" + functor


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
    # the same five reductions with OpenMP over the outputs: what the host could do, not what the reference does
    from oracle import cpu_backend as B
    dt_par = sum(B.c2_parallel(xp if which == "prod_axis1" else x, which)[1] for which in W.C2_CASES)
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "elements_per_s": round(nbytes / 4 / dt, 1),
            "sample": "the five reductions once over the full (8192, 8192) float32 inputs, %.2f s; CAReduce loops "
                      "are single-threaded in the reference" % dt,
            "openmp_variant_not_reference_behaviour": {
                "value": round(nbytes / dt_par / 1e9, 3), "unit": "GB/s", "seconds": round(dt_par, 3),
                "cores": int(G.lib().cpu_omp_threads()),
                "note": "same loops with OpenMP over rows / column blocks; the reference's CAReduce has no pragma"}}


def _cpu_baseline_other(name, vals, nbytes):
    """One pass of the reference's host loops for another configuration
    (oracle/cpu_backend.c) over the full-size inputs."""
    from oracle import cpu_backend as B
    from oracle import graph_ref as G
    out = {}
    kinds = {"c3_fwd": ("c3_fwd", "c3_fwd_rowloop")}.get(name, (name,))
    for kind in kinds:
        try:
            _, seconds = B.run(kind, vals)
        except KeyError:
            return None
        label = {"c3_fwd": "Elemwise/CAReduce chain", "c3_fwd_rowloop": "Softmax op row loop"}.get(kind, "node chain")
        serial_only = kind in ("c3_fwd_rowloop",)
        out[label] = {"value": round(nbytes / seconds / 1e9, 3), "unit": "GB/s", "seconds": round(seconds, 4),
                      "cores": 1 if serial_only else int(G.lib().cpu_omp_threads()),
                      "note": "serial loop" if serial_only else "OpenMP Elemwise nodes, serial CAReduce nodes"}
    return out


def _input_sets(vals, min_total=1 << 30, max_sets=8):
    """Device copies of one input list, enough of them that cycling through them keeps any
    one set from surviving in the 256 MB last-level cache between two uses."""
    from theano_amd.hip import HipArray
    nbytes = sum(v.nbytes for v in vals if v.size > 1)
    n = int(min(max_sets, max(2, -(-min_total // max(nbytes, 1)))))
    return [[HipArray.from_numpy(v) if v.size > 1 else v for v in vals] for _ in range(n)]


def _rate(nbytes, ms):
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"us": round(ms * 1e3, 2), "GB/s": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}


def _awkward_shapes(th, hip, steps, warmup):
    """Reductions and elementwise expressions over shapes that are no whole number of vectors, start off a vector
    boundary, have very few rows or columns, or mix layouts: GB/s of the bytes each must move (inputs once, results
    once), with the plan the library chose.  Every case is about 256 MB of input."""
    import numpy as np
    from theano_amd import tensor as T
    from theano_amd.hip import HipArray
    from theano_amd.tensor import nnet
    N = 64 * 1024 * 1024

    def arr(shape, dtype):
        return HipArray.from_numpy(np.ones(shape, dtype))

    def var(dtype, nd, name="x"):
        return T.TensorType(dtype, (False,) * nd)(name)
    cases = []

    def reduce_case(name, dtype, shape, axis, op="sum"):
        x = var(dtype, len(shape))
        out = (T.sum if op == "sum" else T.max)(x, axis=axis)
        cases.append((name, [x], out, [arr(shape, dtype)]))
    sz = {"float32": 4, "float16": 2, "int8": 1}
    reduce_case("sum of 67108863 float32", "float32", (N - 1,), None)
    reduce_case("sum of 134217727 float16", "float16", (2 * N - 1,), None)
    reduce_case("sum of 268435455 int8", "int8", (4 * N - 1,), None)
    reduce_case("sum (22369621, 3) float32 axis 0", "float32", (N // 3, 3), 0)
    reduce_case("max (22369621, 3) float32 axis 0", "float32", (N // 3, 3), 0, "max")
    reduce_case("sum (44739242, 3) float16 axis 0", "float16", (2 * N // 3, 3), 0)
    reduce_case("sum (2164802, 31) float32 axis 0", "float32", (N // 31, 31), 0)
    reduce_case("sum (100, 100, 13421) float16 axes (0, 1)", "float16", (100, 100, 2 * N // 10000), (0, 1))
    reduce_case("sum (2, 33554432) float32 axis 0", "float32", (2, N // 2), 0)
    reduce_case("sum (3, 22369621) float32 axis 0", "float32", (3, N // 3), 0)
    reduce_case("sum (1048576, 4, 4, 4) float32 axis 1", "float32", (N // 64, 4, 4, 4), 1)
    reduce_case("sum (1000, 67107) float32 axis 1", "float32", (1000, N // 1000 - 1), 1)
    for dtype in ("float32", "float16", "int8"):
        n = 4 * N // sz[dtype]
        x, y = var(dtype, 1), var(dtype, 1, "y")
        a, b = arr(n + 8, dtype), arr(n + 8, dtype)
        cases.append(("x[1:] * 2 + y %s" % dtype, [x, y], x * 2 + y,
                      [a.view([n], [sz[dtype]], a.offset + sz[dtype]), b.view([n], [sz[dtype]], b.offset)]))
        rows = n // 1001
        m, row = var(dtype, 2, "m"), T.TensorType(dtype, (True, False))("row")
        cases.append(("(%d, 1001) * 2 + row %s" % (rows, dtype), [m, row], m * 2 + row, [arr((rows, 1001), dtype), arr((1, 1001), dtype)]))
    for shape in ((8192, 8192), (8191, 8193)):
        x, y = var("float32", 2), var("float32", 2, "y")
        cases.append(("x.T * 2 + y %s float32" % (shape,), [x, y], x.T * 2 + y, [arr(shape, "float32"), arr(shape[::-1], "float32")]))
        cases.append(("tanh(x.T) + 1 %s float32" % (shape,), [x], T.tanh(x.T) + 1, [arr(shape, "float32")]))
    for dtype, cols in (("float32", 1000), ("float32", 1001), ("float32", 4097), ("float16", 1001)):
        rows = (2 * N // sz[dtype]) // cols
        x = var(dtype, 2)
        cases.append(("softmax (%d, %d) %s" % (rows, cols, dtype), [x], nnet.softmax(x), [arr((rows, cols), dtype)]))
    out = []
    for name, ins, expr, vals in cases:
        f = th.function(ins, [th.Out(expr, device=True)])
        res = f(*vals)[0]
        nbytes = sum(int(np.prod(v.shape)) * np.dtype(v.dtype).itemsize for v in vals) + int(np.prod(res.shape)) * np.dtype(res.dtype).itemsize
        plan = hip.last_plan()
        del res
        ms, _ = _time_steps(hip, lambda: f(*vals), steps, warmup)
        parts = plan.split("|")
        split = parts[-1][:1] == "s" and parts[-1][1:].isdigit()       # "|s<slices>": a second launch merges them
        out.append(dict(_rate(nbytes, ms), case=name, bytes=nbytes, plan=plan.split("|", 1)[1],
                        kernel=_symbol("|".join(parts[:-1]) if split else plan)))
        print("%-52s %8.1f us %7.0f GB/s  %s" % (name, ms * 1e3, out[-1]["GB/s"], out[-1]["plan"]), file=sys.stderr, flush=True)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the other four configurations")
    ap.add_argument("--settle-ms", type=float, default=40.0,
                    help="milliseconds of untimed work before each timed leg (0 under a counter-collecting profiler, "
                         "which serialises every launch)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a plain streaming kernel (out = -x on the same (8192, 8192) float32 array, "
                         "256 MiB read + 256 MiB written) K times: the known-size kernel that hardware counters "
                         "of the reductions are scaled by")
    ap.add_argument("--awkward-shapes", action="store_true",
                    help="instead of the benchmark: time reductions and elementwise expressions over shapes of odd "
                         "length, alignment and layout (one JSON line of its own)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no sharding); got --gpus %d" % args.gpus)

    root = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, root)
    if not os.path.exists(os.path.join(root, "theano_amd", "csrc", "libthx_hip.so")):   # a fresh checkout
        from theano_amd.csrc import build as lib_build
        lib_build.build()
    import theano_amd as th
    from theano_amd import hip
    import workloads as W

    hip.init()
    info = hip.device_info()
    SETTLE_MS[0] = max(0.0, args.settle_ms)

    if args.awkward_shapes:
        print(json.dumps({"metric": "GB/s of algorithmic bytes over awkward shapes at 1 MI355X", "unit": "GB/s",
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "data": "synthetic",
                          "cases": _awkward_shapes(th, hip, args.steps, args.warmup)}))
        return

    # ---- headline: config 2 -----------------------------------------------------------------
    # The four reductions of x share one device array and prod has its own, as the configuration
    # states; a step runs them in the configuration's order.
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

    if args.copy_probe:
        from theano_amd import tensor as T
        xs = T.fmatrix("x")
        fcopy = th.function([xs], [th.Out(-xs, device=True)])
        for _ in range(args.steps):
            fcopy(*x_dev["normal"])
        hip.sync()

    _settle(hip, step)
    gpu_ms, wall_ms = _time_steps(hip, step, args.steps, args.warmup)
    value = total_bytes / (gpu_ms * 1e-3) / 1e9

    # Each reduction alone, K launches back to back between two events: over two arrays in turn
    # (2 x 268 MB, so neither survives in the 256 MB last-level cache: "us") and over one array
    # ("same_input_us").  A profile pass names the kernels of each reduction.
    two = [x_dev["normal"], x_dev["prod"]]
    per_case, case_kernels = {}, {}
    for case, f, dev in fns:
        turn = [0]

        def rotating():
            f(*two[turn[0] & 1])
            turn[0] += 1

        cold_ms, _ = _time_steps(hip, rotating, args.steps, 2)
        warm_ms, _ = _time_steps(hip, lambda: f(*dev), args.steps, 2)
        per_case[case] = _rate(W.algorithmic_bytes("c2_" + case), cold_ms)
        per_case[case]["same_input_us"] = round(warm_ms * 1e3, 2)
        with hip.profile() as p:
            f(*dev)
        case_kernels[case] = dict((_symbol(k), n) for k, (n, _) in p.kernels.items())
        per_case[case]["kernels"] = sorted(case_kernels[case])

    # Dominant kernel: the row-form reduction behind sum(axis=1).  In a step it runs once on an
    # array that is not cached (after prod's input) and once on one that partly is (the first
    # pass of sum over all axes, after sum(axis=0) of the same array), and the two loops above
    # launch it K times each way, so the mean of the two is its average over the whole run.
    dom = sorted(case_kernels["sum_axis1"])[0]
    cold_us, warm_us = per_case["sum_axis1"]["us"], per_case["sum_axis1"]["same_input_us"]
    dom_avg_us = 0.5 * (cold_us + warm_us)
    per_launch = 8192 * 8192 * 4 + 8192 * 4   # bytes one launch of a row / column reduction moves by definition
    achieved = per_launch / (dom_avg_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": _traffic(dom, 8192 * 256),
                "kernel": dom, "avg_launch_us": round(dom_avg_us, 2), "uncached_input_us": cold_us,
                "same_input_us": warm_us, "algorithmic_bytes_per_launch": per_launch}

    others = {}
    if not args.no_others:
        specs = [("c1", W.c1_graph(), W.c1_inputs("full")),
                 ("c3_fwd", W.c3_graph(with_grad=False), W.c3_inputs("full", with_grad=False)),
                 ("c3_grad", W.c3_graph(forward=False), W.c3_inputs("full")),
                 ("c3_fwd_grad", W.c3_graph(), W.c3_inputs("full")),
                 ("c4_elemwise", W.c4_graph("elemwise"), W.c4_inputs("full")),
                 ("c4_sum", W.c4_graph("sum"), W.c4_inputs("full")),
                 ("c4_anyall", W.c4_graph("anyall"), W.c4_inputs("full", "anyall")),
                 ("c5_fwd", W.c5_graph(with_grad=False), W.c5_inputs("full", with_grad=False)),
                 ("c5_grad", W.c5_graph(forward=False), W.c5_inputs("full")),
                 ("c2_argmax_axis1", W.c2_argmax_graph(1), W.c2_inputs("max_axis1", "full")),
                 ("c2_argmax_axis0", W.c2_argmax_graph(0), W.c2_inputs("max_axis1", "full"))]
        for name, (ins, outs), vals in specs:
            f = th.function(ins, [th.Out(o, device=True) for o in outs])
            sets = _input_sets(vals)
            turn = [0]

            def rotating():
                f(*sets[turn[0] % len(sets)])
                turn[0] += 1

            # nine runs of max(K, 50) steps each on a device at its steady clocks: the median is the figure (`us`),
            # the fastest run is listed beside it (a run of 20 steps lasts under a millisecond, and the start of each
            # run - the first launch after the event - then weighs 0.5 - 1 us per step)
            k_other = max(args.steps, 50)
            _settle(hip, rotating)
            runs = sorted(_time_steps(hip, rotating, k_other, 3)[0] for _ in range(9))
            ms = runs[len(runs) // 2]
            warm_ms = sorted(_time_steps(hip, lambda: f(*sets[0]), k_other, 3)[0] for _ in range(5))[2]
            n_k = sum(1 for n in f.toposort()
                      if type(n.op).__name__ in ("HipElemwise", "HipElemwiseReduce", "HipCAReduce", "HipRowChain", "HipMaxAndArgmax"))
            with hip.profile() as p:
                f(*sets[0])
            others[name] = _rate(W.algorithmic_bytes(name), ms)
            others[name].update({"min_us": round(runs[0] * 1e3, 2), "steps_per_run": k_other, "input_sets": len(sets),
                                 "same_input_us": round(warm_ms * 1e3, 2), "nodes_per_step": n_k,
                                 "kernels": sorted(_symbol(k) for k in p.kernels)})
            if name in REAL_BYTES:
                # what the kernels of this configuration really move (one read of x, one write of y), beside the
                # three passes the configuration is priced at
                real = REAL_BYTES[name]
                others[name]["real_bytes"] = real
                others[name]["real_traffic_frac"] = round(real / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            del f, sets
            if not args.no_cpu:
                cpu_o = _cpu_baseline_other(name, vals, W.algorithmic_bytes(name))
                if cpu_o:
                    others[name]["cpu_baseline"] = cpu_o

    cpu = None if args.no_cpu else _cpu_baseline_c2(W)

    # the weakest timed workload, next to the headline
    fracs = dict(("c2_" + k, v["frac_of_peak"]) for k, v in per_case.items())
    fracs.update((k, v["frac_of_peak"]) for k, v in others.items())
    worst = min(fracs, key=fracs.get)

    line = {
        "metric": "achieved HBM GB/s and % of peak for fused Elemwise+CAReduce at 1 MI355X",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(gpu_ms, 5), "wall_ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32 data, f64 accumulators", "data": "synthetic",
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "elements_per_s": round(5 * 8192 * 8192 / (gpu_ms * 1e-3), 1),
        "config": {"workload": "config 2: CAReduce on float32 (8192, 8192): sum axis=1, max axis=1, sum axis=0, "
                               "sum all axes, prod axis=1; one step = the five reductions",
                   "algorithmic_bytes_per_step": total_bytes, "device": info["arch"],
                   "compute_units": info["compute_units"]},
        "roofline": roofline, "cpu_baseline": cpu,
        "worst_config": {"name": worst, "frac": fracs[worst], "us": (per_case.get(worst[3:]) or others.get(worst))["us"]},
        "per_reduction": per_case, "other_configs": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
