#!/usr/bin/env python3
"""Benchmark of the convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload alexnet]

A step is one forward + backward pass (zeroGradParameters, forward,
updateGradInput and accGradParameters of every module, as nn.Module:backward
does) of the AlexNet-style conv stack at batch 128, fp32, on synthetic inputs
that are resident in HBM before the timed region starts.  Prints ONE JSON line.

Beside the throughput the line carries
  roofline      the GEMM kernels (fp32 MFMA bound): algorithmic flops of all
                GEMM launches of a step (2*M*N*K*B per convolution pass, declared
                at the convolution's launch sites) / their summed HIP-event
                durations, measured in a second, instrumented run of the same K steps.
                `traffic` is the HBM bytes per GEMM launch read from the committed
                rocprofv3 --pmc summary under profiles/, and only when the GEMM
                launches of this run (shapes, tiles, splits) are the ones that
                summary was taken on;
  kernels       the same for every kernel family (HBM-bound ones in GB/s);
  gemm_shapes   every GEMM of the stack on its own (shape, chosen tile and split,
                TFLOP/s): the small-K GEMMs of first layers are HBM-bound themselves;
  hbm_shapes    every im2col / col2im / pad / pooling launch geometry on its own (GB/s);
  column_route  the same steps once more with every convolution on the reference's
                route (im2col, GEMM, col2im): throughput, GEMM roofline, and the
                im2col / col2im figures at the workload's full geometries.  The
                headline run lets the library pick the route per layer (--conv-route
                auto, its default: narrow layers gather straight from a padded image);
  cpu_baseline  the CPU oracle (a port of the reference CPU nn path, OpenMP over
                the batch + an optimised BLAS sgemm where one is found) timed
                on this host on a reduced batch of the same stack.

The stack runs with Sequential.fuse() (every ReLU applied by its neighbours as they store
their results; bit-identical to the separate passes); --no-fuse runs the separate passes.

Other modes
  --workload ref_benchmark   the reference's own micro-benchmark (gpunn/test/benchmark.lua:7-91): seven single
                             layers, updateOutput / updateGradInput / accGradParameters timed separately and
                             reported with its GFLOP/s formula (:118).
  --workload plan_check      the library's GEMM tile/split choice against every forced configuration, per layer and
                             pass of the three stacks and the reference benchmark set (a few minutes).
  --workload hbm_sweep       GB/s of the HBM-bound kernels at the stack's geometries as the launch size grows.
  --summarise kernel-trace|traffic|mfma ...   turns rocprofv3 CSV output into the text summaries kept under
                             profiles/ (see summarise()).
"""
import argparse
import collections
import csv
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "images/sec fwd+bwd, AlexNet-style conv stack b128 fp32; GEMM % fp32 MFMA peak"
PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
ROUTES = {"columns": 0, "auto": 1, "gathered": 2}   # thgpu_conv_set_mode values
# rocprofv3's FETCH_SIZE / WRITE_SIZE read these fractions of the bytes a plain float4 copy kernel of known size
# (64 MiB .. 2 GiB) loads / stores on this GPU: counters are scaled by the inverse.
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def traffic_profile_path(workload, batch, route):
    tag = "" if route == "auto" else "_%s_route" % {"columns": "column", "gathered": "gathered"}[route]
    return os.path.join(ROOT, "profiles", "hbm_traffic_%s_b%d%s_pmc.txt" % (workload, batch, tag))


def measured_gemm_traffic(workload, batch, route, fused, gemm_labels):
    """HBM bytes per GEMM launch from the committed rocprofv3 --pmc summary of this configuration, or (None, why).
    The summary ends in a `bench_check:` JSON line naming the GEMM launches it was taken on; counters cannot be
    read from inside the timed process, so the figure is only carried over when this run launched the same GEMMs."""
    path = traffic_profile_path(workload, batch, route)
    if not os.path.exists(path):
        return None, "no traffic summary %s" % os.path.relpath(path, ROOT)
    check = None
    for line in open(path):
        if line.startswith("bench_check:"):
            check = json.loads(line[len("bench_check:"):])
    if check is None:
        return None, "%s has no bench_check line" % os.path.relpath(path, ROOT)
    if bool(check.get("fused")) != bool(fused):
        return None, "%s was measured with fused=%s" % (os.path.relpath(path, ROOT), check.get("fused"))
    if sorted(check["gemm_launches"]) != sorted(gemm_labels):
        missing = sorted(set(check["gemm_launches"]) - set(gemm_labels))
        extra = sorted(set(gemm_labels) - set(check["gemm_launches"]))
        return None, ("the GEMM launches of this run differ from the ones %s was measured on (not in this run: %s; "
                      "new in this run: %s): re-run the two --pmc passes and bench.py --summarise traffic"
                      % (os.path.relpath(path, ROOT), missing[:3], extra[:3]))
    return check["gemm_bytes_per_launch"], None


def cpu_baseline(workload, sample_batch, budget_s=12.0):
    """Times the CPU oracle on `sample_batch` images of the workload."""
    import numpy as np

    import oracle
    from mcw_cppamp_torch_amd import stacks

    backend = oracle.use_blas(True)
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    oracle.set_threads(cores)
    cfg = stacks.STACKS[workload]
    layers = cfg["layers"]
    net = stacks.build(workload, seed_base=1000)
    params = [(np.array(m.weight), np.array(m.bias)) if hasattr(m, "weight") else None for m in net.modules]
    x = stacks.make_input(workload, sample_batch, seed=1000)
    rng = np.random.Generator(np.random.PCG64(1003))
    go = rng.uniform(-1, 1, stacks.output_shape(workload, sample_batch)).astype(np.float32)

    def step():
        saved, cur = [], x
        for l, p in zip(layers, params):
            if l[0] == "conv":
                _, _, _, kW, kH, dW, dH, pW, pH = l
                out, aux = oracle.conv_updateOutput(cur, p[0], p[1], kH, kW, pH, pW, dH, dW)
            elif l[0] == "pool":
                out, aux = oracle.maxpool_updateOutput(cur, l[2], l[1], l[4], l[3])
            else:
                out, aux = oracle.threshold_updateOutput(cur), None
            saved.append((cur, aux))
            cur = out
        g = go
        for i in range(len(layers) - 1, -1, -1):
            l, p = layers[i], params[i]
            inp, aux = saved[i]
            if l[0] == "conv":
                _, _, _, kW, kH, dW, dH, pW, pH = l
                gi, _ = oracle.conv_updateGradInput(g, p[0], inp.shape, kH, kW, pH, pW, dH, dW)
                gw, gb = np.zeros_like(p[0]), np.zeros_like(p[1])
                oracle.conv_accGradParameters(g, aux, gw, gb, 1.0)
            elif l[0] == "pool":
                gi = oracle.maxpool_updateGradInput(g, aux, inp.shape, l[4], l[3])
            else:
                gi = oracle.threshold_updateGradInput(inp, g)
            g = gi

    step()  # first touch / thread start-up
    times = []
    t_begin = time.perf_counter()
    while len(times) < 15 and (time.perf_counter() - t_begin < budget_s or not times):  # about 10 s of CPU work
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    oracle.use_blas(False)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": sample_batch / med, "unit": "images/s", "cores": cores, "kind": "port",
        "sample": "%s stack fwd+bwd on a batch of %d images, median of %d runs (%.2f s each); sgemm backend: %s"
                  % (workload, sample_batch, len(times), med, backend),
    }


# The reference's micro-benchmark layer set (gpunn/test/benchmark.lua:7-91): ni, no, kw, kh, iw, ih, bs, dw, dh.
REF_BENCHMARK_RUNS = [
    (3, 96, 11, 11, 128, 128, 128, 1, 1),     # first layer
    (64, 128, 9, 9, 64, 64, 128, 1, 1),       # second layer
    (128, 128, 9, 9, 32, 32, 128, 1, 1),      # third layer
    (128, 128, 7, 7, 16, 16, 128, 1, 1),      # fourth layer
    (384, 384, 3, 3, 13, 13, 128, 1, 1),      # small inputs/kernels of the lower end of a network
    (3, 96, 11, 11, 128, 128, 16, 1, 1),      # first layer, tiny batch
    (64, 128, 9, 9, 64, 64, 16, 1, 1),        # second layer, tiny batch
]


def ref_benchmark(args, pkg):
    """gpunn/test/benchmark.lua for nn.SpatialConvolutionMM (its BDHW rows): per layer, `steps` calls of updateOutput,
    of updateGradInput and of accGradParameters, each loop between two synchronisations, GFLOP/s by the reference's
    formula ni*no*kw*kh*(iw-kw+1)*(ih-kh+1)/dw/dh*bs*2/t (:118)."""
    import numpy as np

    from mcw_cppamp_torch_amd import gputorch, nn

    rng = np.random.Generator(np.random.PCG64(77))
    rows, tot_fl, tot_t = [], 0.0, 0.0
    if pkg._lib.lib.thgpu_conv_set_mode(ROUTES[args.conv_route]) != 0:
        sys.exit("bench.py: " + pkg._lib.lib.thgpu_last_error().decode())
    for ni, no, kw, kh, iw, ih, bs, dw, dh in REF_BENCHMARK_RUNS:
        m = nn.SpatialConvolutionMM(ni, no, kw, kh, dw, dh, rng=rng).gpu()
        x = pkg.FloatTensor(rng.standard_normal((bs, ni, ih, iw)).astype(np.float32)).gpu()
        o = m.forward(x)
        flops = ni * no * kw * kh * (iw - kw + 1) * (ih - kh + 1) / dw / dh * bs * 2
        row = {"config": "input %dx%dx%d * ker %dx%dx%dx%d (bs = %d, stride = %d)" % (ni, iw, ih, ni, no, kw, kh, bs, dw)}
        for name, call in (("updateOutput", lambda: m.updateOutput(x)),
                           ("updateGradInput", lambda: m.updateGradInput(x, o)),
                           ("accGradParameters", lambda: m.accGradParameters(x, o))):
            for _ in range(args.warmup):
                call()
            gputorch.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                call()
            gputorch.synchronize()
            tm = (time.perf_counter() - t0) / args.steps
            row[name] = {"gflops": round(flops / tm / 1e9, 1), "ms": round(tm * 1e3, 4),
                         "frac_of_fp32_mfma_peak": round(flops / tm / 1e12 / PEAK_MFMA_F32_TFLOPS, 4)}
            tot_fl += flops
            tot_t += tm
        rows.append(row)
        del m, x, o
    print(json.dumps({
        "metric": "GFLOP/s of nn.SpatialConvolutionMM on the reference's benchmark layer set "
                  "(gpunn/test/benchmark.lua), its own formula",
        "value": round(tot_fl / tot_t / 1e9, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(tot_t * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "seven single layers, three passes each timed on its own; value = all flops / all time",
                   "conv_route": args.conv_route, "device": gputorch.getDeviceProperties()["name"]},
        "layers": rows}))


PLAN_TILES = ["128x128", "192x128", "64x256", "128x256", "256x128", "64x64", "64x128", "96x128", "48x128", "48x256"]
PLAN_SPLITS = [1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16, 20, 24, 28, 32, 40, 48, 59, 64, 96, 128, 170, 256]


def plan_check(args, pkg):
    """How good is the library's own (tile, split) choice?  For every convolution of the AlexNet-, OverFeat- and
    VGG-A-style stacks and of the reference's benchmark set, and every pass, the pass is timed with the library's
    choice and with every tile configuration and reduction split forced in turn (the switches of thgpu_debug_set);
    a row gives the choice, the fastest forced configuration, and the ratio of their times (pad copies, split
    reduction and bias gradient of the pass included on both sides)."""
    import numpy as np

    from mcw_cppamp_torch_amd import gputorch, nn, stacks

    lib = pkg._lib.lib
    rng = np.random.Generator(np.random.PCG64(78))
    shapes = []  # (tag, B, C, H, W, M, kH, kW, sH, sW, pH, pW)
    for name in ("alexnet", "overfeat", "vgg_a"):
        cfg = stacks.STACKS[name]
        for l, (C, H, W), _ in stacks.trace_shapes(cfg["layers"], cfg["input"]):
            if l[0] == "conv":
                shapes.append((name, cfg["batch"], C, H, W, l[2], l[4], l[3], l[6], l[5], l[8], l[7]))
    for ni, no, kw, kh, iw, ih, bs, dw, dh in REF_BENCHMARK_RUNS:
        shapes.append(("ref_benchmark", bs, ni, ih, iw, no, kh, kw, dh, dw, 0, 0))
    only = set(args.plan_stacks.split(",")) if args.plan_stacks else None
    seen, rows = set(), []

    def set_plan(tile, split):
        lib.thgpu_debug_set(b"gemm_tile", tile.encode() if tile else None)
        lib.thgpu_debug_set(b"gemm_split", str(split).encode() if split else None)

    for tag, B, C, H, W, M, kH, kW, sH, sW, pH, pW in shapes:
        key = (B, C, H, W, M, kH, kW, sH, sW, pH, pW)
        if key in seen or (only and tag not in only):
            continue
        seen.add(key)
        m = nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH, rng=rng).gpu()
        x = pkg.FloatTensor(rng.standard_normal((B, C, H, W)).astype(np.float32)).gpu()
        o = m.forward(x)
        passes = (("updateOutput", "gemm_conv_fwd", lambda: m.updateOutput(x)),
                  ("updateGradInput", "gemm_conv_gradinput", lambda: m.updateGradInput(x, o)),
                  ("accGradParameters", "gemm_conv_gradweight", lambda: m.accGradParameters(x, o)))

        def timed(call, label_key, reps):
            """(ms per call, the GEMM's tile and split) for the plan currently set, or None when it cannot run."""
            try:
                call()
                gputorch.synchronize()
                gputorch.prof_reset()
                gputorch.prof_enable(True)
                call()
                gputorch.synchronize()
                labels = [k for k in gputorch.prof_report() if k.startswith(label_key)]
                gputorch.prof_enable(False)
                gputorch.prof_reset()
                t0 = time.perf_counter()
                for _ in range(reps):
                    call()
                gputorch.synchronize()
                ms = (time.perf_counter() - t0) / reps * 1e3
            except pkg.THGPUError:
                gputorch.prof_enable(False)
                gputorch.prof_reset()
                return None
            cfg = labels[0].split("tile=")[1] if labels else "?"
            return ms, cfg

        for pname, label_key, call in passes:
            set_plan(None, None)
            for _ in range(3):
                call()
            auto = min(timed(call, label_key, args.steps) for _ in range(2))
            best = None
            tried = set()
            for tile in PLAN_TILES:
                for split in PLAN_SPLITS:
                    set_plan(tile, split)
                    r = timed(call, label_key, max(2, args.steps // 4))
                    if r is None or r[1] in tried or not r[1].startswith(tile + " "):
                        continue
                    tried.add(r[1])
                    if best is None or r[0] < best[0]:
                        best = r
            set_plan(None, None)
            if best is not None:  # the winner again, at the library choice's repetition count
                tile, split = best[1].split(" split=")
                set_plan(tile, int(split))
                best = min(timed(call, label_key, args.steps) for _ in range(2))
                set_plan(None, None)
                again = min(timed(call, label_key, args.steps) for _ in range(2))
                auto = min(auto, again)
            row = {"stack": tag, "layer": "b%d %d->%d %dx%d k%dx%d s%d p%d" % (B, C, M, H, W, kH, kW, sH, pH),
                   "pass": pname, "choice": auto[1], "choice_ms": round(auto[0], 4),
                   "best_forced": best[1] if best else None, "best_forced_ms": round(best[0], 4) if best else None,
                   "choice_over_best": round(auto[0] / best[0], 4) if best else None}
            rows.append(row)
            print("plan_check %(stack)s %(layer)s %(pass)s: choice %(choice)s %(choice_ms).4f ms, best forced "
                  "%(best_forced)s %(best_forced_ms)s ms, ratio %(choice_over_best)s" % row, file=sys.stderr, flush=True)
        del m, x, o
    ratios = [r["choice_over_best"] for r in rows if r["choice_over_best"]]
    tot_c = sum(r["choice_ms"] for r in rows if r["choice_over_best"])
    tot_b = sum(r["best_forced_ms"] for r in rows if r["choice_over_best"])
    print(json.dumps({
        "metric": "time of the library's own GEMM tile/split choice over the fastest forced configuration, summed "
                  "over all passes of all layers", "value": round(tot_c / tot_b, 4), "unit": "ratio", "n_gpus": 1,
        "steps": args.steps, "warmup": 3, "ms_per_step": round(tot_c, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "every convolution of the alexnet, overfeat, vgg_a stacks and the reference benchmark "
                               "set, three passes each", "worst_ratio": max(ratios) if ratios else None,
                   "device": gputorch.getDeviceProperties()["name"]},
        "rows": rows}))


def hbm_sweep(args, pkg):
    """GB/s of the HBM-bound kernels at the AlexNet-style stack's geometries as the batch, and with it the size of a
    launch, grows from 32 to 2048 images: what a launch of 10-60 us loses to its ramp-up shows as the gap between
    the batch-128 figure and the large-batch one.  HIP-event time per launch, algorithmic bytes as in `kernels`."""
    import numpy as np

    from mcw_cppamp_torch_amd import gputorch, nn

    lib = pkg._lib.lib
    rng = np.random.default_rng(0)

    def dev(shape):
        return pkg.FloatTensor(rng.uniform(-1, 1, shape).astype(np.float32)).gpu()

    def timed(fn, n):
        for _ in range(2):
            fn()
        gputorch.synchronize()
        gputorch.prof_reset()
        gputorch.prof_enable(True)
        for _ in range(n):
            fn()
        gputorch.synchronize()
        rep = gputorch.prof_report()
        gputorch.prof_enable(False)
        gputorch.prof_reset()
        return {k: r for k, r in rep.items() if r["bytes"] > 0 and not k.startswith("gemm_conv")}

    rows = []

    def record(rep, geometry, batch):
        for kn, r in sorted(rep.items()):
            rows.append({"kernel": kn.split(" ")[0], "geometry": geometry, "batch": batch,
                         "mb_per_launch": round(r["bytes"] / r["calls"] / 1e6, 1),
                         "us": round(r["ms"] / r["calls"] * 1e3, 1), "gbs": round(r["bytes"] / r["ms"] / 1e6),
                         "frac": round(r["bytes"] / r["ms"] / 1e6 / PEAK_HBM_GBS, 3)})

    for C, H, k, s in ((64, 55, 3, 2), (192, 27, 3, 2), (256, 13, 3, 2)):
        for B in (32, 128, 512, 2048):
            x = dev((B, C, H, H))
            m = nn.SpatialMaxPooling(k, k, s, s).gpu()
            o = m.forward(x)
            go = dev(o.size())
            m.inputThreshold = 0.0       # the backward of a ReLU in front is applied as gradInput is stored
            record(timed(lambda: (m.forward(x), m.updateGradInput(x, go)), args.steps),
                   "%dx%dx%d k%d s%d" % (C, H, H, k, s), B)
            del x, o, go, m
    lib.thgpu_conv_set_mode(ROUTES["auto"])
    for conv, shape, label in (((3, 64, 11, 11, 4, 4, 2), (3, 224, 224), "conv 3->64 224x224 k11 s4 p2"),
                               ((256, 256, 3, 3, 1, 1, 1), (256, 13, 13), "conv 256->256 13x13 k3 p1")):
        for B in (32, 128, 512):
            m = nn.SpatialConvolutionMM(*conv).gpu()
            x = dev((B,) + shape)
            o = m.forward(x)
            go = dev(o.size())
            record(timed(lambda: (m.forward(x), m.updateGradInput(x, go), m.accGradParameters(x, go)),
                         max(2, args.steps // 4)), label, B)
            del m, x, o, go
    print(json.dumps({
        "metric": "GB/s of the HBM-bound kernels against launch size", "value": max(r["gbs"] for r in rows),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": 2, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "pooling forward / masked backward, pad, col2im, gradBias, split reduction at the "
                               "AlexNet-style geometries, batch 32 .. 2048"}, "rows": rows}))
    if args.table:
        print("%-18s %-30s %6s %10s %9s %8s %6s" % ("kernel", "geometry", "batch", "MB/launch", "us", "GB/s", "frac"),
              file=sys.stderr)
        for r in rows:
            print("%-18s %-30s %6d %10.1f %9.1f %8d %6.3f" % (r["kernel"], r["geometry"], r["batch"], r["mb_per_launch"],
                                                             r["us"], r["gbs"], r["frac"]), file=sys.stderr)


# ---- rocprofv3 output -> the text summaries under profiles/ ----------------------------------------------------------

def _short(name):
    name = name.replace("thgpu::(anonymous namespace)::", "").replace("void ", "").replace("thgpu::", "")
    return re.sub(r"\(.*", "", name)


FAMILIES = [("gemm_fast", "gemm"), ("gemm_generic", "gemm"), ("im2col", "im2col"), ("col2im", "col2im"),
            ("maxpool_bwd", "maxpool_bwd"), ("maxpool_fwd", "maxpool_fwd"), ("threshold_fwd", "threshold_fwd"),
            ("threshold_bwd", "threshold_bwd"), ("split_reduce", "gemm_split_reduce"),
            ("gradbias_partial", "gradbias"), ("gradbias_final", "gradbias_final"), ("fill_kernel", "fill"),
            ("pad_planes", "pad_planes"), ("conv_narrow_forward", "conv_narrow_fwd"),
            ("conv_narrow_gradweight_finish", "conv_narrow_gradweight_finish"),
            ("conv_narrow_gradweight", "conv_narrow_gradweight")]


def _family(kernel_name):
    for key, fam in FAMILIES:
        if key in kernel_name:
            return fam
    return None


def summarise(args):
    """bench.py --summarise kernel-trace STATS.csv BENCH.json STEPS   (rocprofv3 --kernel-trace --stats ... _kernel_stats.csv)
    bench.py --summarise traffic FETCH.csv WRITE.csv BENCH.json STEPS  (two --pmc runs' _counter_collection.csv)
    bench.py --summarise mfma COUNTERS.csv                             (one --pmc run with the SQ_* counters)
    bench.py --summarise hbm-pmc COUNTERS.csv KERNEL_TRACE.csv         (one --pmc run around --workload hbm_sweep)
    bench.py --summarise requests REQ.csv FETCH.csv WRITE.csv REQ_KERNEL_TRACE.csv   (three --pmc runs around hbm_sweep)
    BENCH.json is the line an ordinary run of the same configuration printed; STEPS the steps the profiled runs made
    (warm-up included).  Writes the summary to stdout; `header` lines (the commands) come from --summary-header."""
    kind, files = args.summarise[0], args.summarise[1:]
    out = [l for l in (args.summary_header or "").split("\\n") if l] + [""]
    if kind == "kernel-trace":
        stats, bench, steps = files[0], json.load(open(files[1])), int(files[2])
        out.append("%-66s %6s %12s %10s %6s" % ("kernel", "calls", "total_ms", "avg_us", "%"))
        tot = gemm = 0.0
        gcalls = 0
        for r in csv.DictReader(open(stats)):
            ms = float(r["TotalDurationNs"]) / 1e6
            tot += ms
            if _family(r["Name"]) == "gemm":
                gemm += ms
                gcalls += int(r["Calls"])
            out.append("%-66s %6s %12.3f %10.1f %6.2f" % (_short(r["Name"])[:66], r["Calls"], ms,
                                                           float(r["AverageNs"]) / 1e3, float(r["Percentage"])))
        fl = bench["roofline"]["flops_per_step"]
        out += ["", "All kernels: %.3f ms per step.  GEMM kernels (%d launches per step): %.3f ms per step"
                % (tot / steps, gcalls / steps, gemm / steps),
                "-> %.3f GFLOP of convolution GEMM work per step / %.3f ms = %.1f TFLOP/s = %.1f %% of the %.1f TFLOP/s "
                "fp32 MFMA peak; average GEMM launch %.1f us."
                % (fl / 1e9, gemm / steps, fl / (gemm / steps) / 1e9, fl / (gemm / steps) / 1e9 / PEAK_MFMA_F32_TFLOPS * 100,
                   PEAK_MFMA_F32_TFLOPS, gemm / gcalls * 1e3),
                "bench.py's own HIP-event measurement of the same launches in the same configuration: %.3f ms per step "
                "(%.2f TFLOP/s); its throughput in that run: %.0f images/s (%.3f ms per step)."
                % (bench["roofline"]["ms_per_step"], bench["roofline"]["achieved"], bench["value"], bench["ms_per_step"])]
    elif kind == "traffic":
        def load(path):
            d = collections.OrderedDict()
            for r in csv.DictReader(open(path)):
                d[int(r["Dispatch_Id"])] = (r["Kernel_Name"], float(r["Counter_Value"]))
            return d
        fetch, write = load(files[0]), load(files[1])
        bench, steps = json.load(open(files[2])), int(files[3])
        fam = collections.OrderedDict()
        for k, (name, v) in fetch.items():
            f = _family(name)
            if f is None or k not in write:
                continue
            a = fam.setdefault(f, [0, 0.0, 0.0])
            a[0] += 1
            a[1] += v * FETCH_SCALE / 1024
            a[2] += write[k][1] * WRITE_SCALE / 1024
        alg = {k: v["gbs"] * 1e6 * v["ms_per_step"] / 1048576 for k, v in bench["kernels"].items() if "gbs" in v}
        out.append("Counters are KiB per dispatch; FETCH_SIZE is scaled by %.1f and WRITE_SIZE by %.1f, the factors a plain "
                   "float4 copy kernel of known size (64 MiB .. 2 GiB) gives for the same counters on this GPU."
                   % (FETCH_SCALE, WRITE_SCALE))
        out += ["", "%-22s %9s %12s %12s %12s %15s %8s" % ("kernel family", "launches", "fetch MiB", "write MiB", "total MiB",
                                                        "algorithmic MiB", "ratio"),
                "%-22s %9s %12s %12s %12s %15s %8s" % ("", "per step", "per step", "per step", "per step", "per step", "")]
        total = 0.0
        for f, a in fam.items():
            n, fe, wr = a[0] / steps, a[1] / steps, a[2] / steps
            total += fe + wr
            al = alg.get(f)
            out.append("%-22s %9.1f %12.1f %12.1f %12.1f %15s %8s" % (f, n, fe, wr, fe + wr, ("%.1f" % al) if al else "-",
                                                                    ("%.2f" % ((fe + wr) / al)) if al else "-"))
        g = fam["gemm"]
        per = (g[1] + g[2]) / g[0]
        if "fill" in fam:
            out.append("(fill: the profiled run's first step also writes the zero borders of the padded buffers, once per buffer; a later "
                       "step only zeroes gradWeight / gradBias, the algorithmic figure.)")
        out += ["", "All kernels: %.1f MiB per step." % total,
                "GEMM family: %.1f MiB per step over %d launches = %.1f MiB (%.4g bytes) per launch on average."
                % ((g[1] + g[2]) / steps, g[0] / steps, per, per * 1048576),
                "bench_check: " + json.dumps({
                    "workload": bench["config"]["workload"].split(" ")[0], "batch": bench["config"]["batch"],
                    "route": bench["config"]["conv_route"], "fused": bench["config"].get("relu_fused", False),
                    "gemm_bytes_per_launch": round(per * 1048576), "gemm_launches": [s["gemm"] for s in bench["gemm_shapes"]]})]
    elif kind == "mfma":
        agg = collections.OrderedDict()
        for r in csv.DictReader(open(files[0])):
            if _family(r["Kernel_Name"]) != "gemm":
                continue
            key = (_short(r["Kernel_Name"]), r["Grid_Size"])
            agg.setdefault(key, collections.defaultdict(float))[r["Counter_Name"]] += float(r["Counter_Value"])
            agg[key]["_n_" + r["Counter_Name"]] += 1
        out.append("%-58s %9s %9s %9s %9s %9s" % ("kernel (grid)", "launches", "mfma_busy", "wait_any", "wait_lds", "lds_confl"))
        for (name, grid), c in agg.items():
            n = c["_n_SQ_BUSY_CU_CYCLES"] or 1
            busy = c["SQ_VALU_MFMA_BUSY_CYCLES"] / max(c["SQ_BUSY_CU_CYCLES"], 1) / 4   # per SIMD of a busy CU
            wave = max(c["SQ_WAVE_CYCLES"], 1)
            out.append("%-58s %9d %8.1f%% %8.1f%% %8.1f%% %8.2f%%" % (
                ("%s (%s)" % (name, grid))[:58], n, 100 * busy, 100 * c["SQ_WAIT_INST_ANY"] / wave,
                100 * c["SQ_WAIT_INST_LDS"] / wave, 100 * c["SQ_LDS_BANK_CONFLICT"] / max(c["SQ_ACTIVE_INST_LDS"], 1)))
        out.append("mfma_busy = SQ_VALU_MFMA_BUSY_CYCLES / (4 * SQ_BUSY_CU_CYCLES); wait_* = SQ_WAIT_INST_* / SQ_WAVE_CYCLES; "
                   "lds_confl = SQ_LDS_BANK_CONFLICT / SQ_ACTIVE_INST_LDS.")
    elif kind == "hbm-pmc":
        # COUNTERS.csv of `rocprofv3 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_ANY SQ_WAIT_INST_ANY
        # SQ_INSTS_VALU SQ_INSTS_LDS SQ_INSTS_VMEM --kernel-trace` around `bench.py --workload hbm_sweep`, and the
        # kernel trace of the same run (durations): what a wavefront of each HBM-bound kernel spends its life on.
        dur = {}
        for r in csv.DictReader(open(files[1])):
            dur[int(r["Dispatch_Id"])] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        agg = collections.OrderedDict()
        for r in csv.DictReader(open(files[0])):
            fam = _family(r["Kernel_Name"])
            if fam is None or fam == "gemm":
                continue
            key = (fam, int(r["Grid_Size"]))
            a = agg.setdefault(key, collections.defaultdict(float))
            a[r["Counter_Name"]] += float(r["Counter_Value"])
            if r["Counter_Name"] == "SQ_WAVES":
                a["_launches"] += 1
                a["_ns"] += dur.get(int(r["Dispatch_Id"]), 0)
        out.append("%-18s %11s %8s %9s %10s %8s %8s %7s %6s %6s %6s" % (
            "kernel", "threads", "launches", "us/launch", "waves/SIMD", "life us", "waiting", "on mem", "VALU", "LDS", "VMEM"))
        for (fam, grid), c in agg.items():
            n = max(c["_launches"], 1)
            waves = max(c["SQ_WAVES"], 1)
            us = c["_ns"] / n / 1e3
            wave_cycles = c["SQ_WAVE_CYCLES"] * 4          # the counter ticks once per four cycles
            clocks = c["_ns"] * 2.4                          # 2.4 GHz shader clock
            out.append("%-18s %11d %8d %9.1f %10.2f %8.1f %7.0f%% %6.0f%% %6.0f %6.0f %6.0f" % (
                fam, grid, n, us, wave_cycles / max(clocks, 1) / 1024, wave_cycles / waves / 2400.0,
                100 * c["SQ_WAIT_ANY"] / max(c["SQ_WAVE_CYCLES"], 1), 100 * c["SQ_WAIT_INST_ANY"] / max(c["SQ_WAVE_CYCLES"], 1),
                c["SQ_INSTS_VALU"] / waves, c["SQ_INSTS_LDS"] / waves, c["SQ_INSTS_VMEM"] / waves))
        out.append("waves/SIMD = 4 * SQ_WAVE_CYCLES / (launch duration * 2.4 GHz * 1024 SIMDs), at most 8; life = mean residence of "
                   "a wavefront; waiting = SQ_WAIT_ANY / SQ_WAVE_CYCLES (any wait, barriers included); on mem = SQ_WAIT_INST_ANY / "
                   "SQ_WAVE_CYCLES; VALU / LDS / VMEM = instructions per wavefront.")
    elif kind == "requests":
        # Three --pmc runs around `bench.py --workload hbm_sweep` (TCP_TCC_READ_REQ_sum TCP_TCC_WRITE_REQ_sum; FETCH_SIZE;
        # WRITE_SIZE), each with --kernel-trace: how many requests a kernel sends from the vector caches to the L2 and
        # how many bytes each carries on average -- the request rate, not the byte rate, is what a kernel with short or
        # misaligned runs saturates.
        def load(path):
            d = collections.OrderedDict()
            for r in csv.DictReader(open(path)):
                e = d.setdefault(int(r["Dispatch_Id"]), {"name": r["Kernel_Name"], "grid": int(r["Grid_Size"]), "ns": 0})
                e[r["Counter_Name"]] = float(r["Counter_Value"])
            return d
        req, fetch, write = load(files[0]), load(files[1]), load(files[2])
        for r in csv.DictReader(open(files[3])):             # durations: the kernel trace of the request-counter run
            if int(r["Dispatch_Id"]) in req:
                req[int(r["Dispatch_Id"])]["ns"] = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        agg = collections.OrderedDict()
        for k, e in req.items():
            fam = _family(e["name"])
            if fam is None or fam == "gemm" or k not in fetch or k not in write:
                continue
            a = agg.setdefault((fam, _short(e["name"])[:34], e["grid"]), collections.defaultdict(float))
            a["n"] += 1
            a["ns"] += e["ns"]
            a["rd"] += e.get("TCP_TCC_READ_REQ_sum", 0.0)
            a["wr"] += e.get("TCP_TCC_WRITE_REQ_sum", 0.0)
            a["fetch"] += fetch[k].get("FETCH_SIZE", 0.0) * FETCH_SCALE * 1024
            a["write"] += write[k].get("WRITE_SIZE", 0.0) * WRITE_SCALE * 1024
        out.append("%-34s %10s %8s %9s %10s %10s %9s %9s %8s %8s" % (
            "kernel", "threads", "launches", "us/launch", "read req", "write req", "fetch MiB", "write MiB", "B/rd req",
            "B/wr req"))
        for (fam, name, grid), a in agg.items():
            n = a["n"]
            out.append("%-34s %10d %8d %9.1f %10.0f %10.0f %9.1f %9.1f %8.0f %8.0f" % (
                name, grid, n, a["ns"] / n / 1e3, a["rd"] / n, a["wr"] / n, a["fetch"] / n / 1048576, a["write"] / n / 1048576,
                a["fetch"] / max(a["rd"], 1), a["write"] / max(a["wr"], 1)))
        out.append("read / write req = TCP_TCC_READ_REQ_sum / TCP_TCC_WRITE_REQ_sum per launch; fetch / write MiB = FETCH_SIZE x %.1f, "
                   "WRITE_SIZE x %.1f (memory-side traffic); B/req = memory-side bytes per L2 request of that direction (reads "
                   "served by the L2 lower it, a full request carries 64 bytes of a store or 128 of a load)."
                   % (FETCH_SCALE, WRITE_SCALE))
    else:
        sys.exit("--summarise kernel-trace | traffic | mfma | hbm-pmc | requests")
    print("\n".join(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="alexnet",
                    choices=["alexnet", "overfeat", "vgg_a", "conv1_b16", "ref_benchmark", "hbm_sweep", "plan_check"])
    ap.add_argument("--plan-stacks", default=None,
                    help="plan_check: comma-separated subset of alexnet,overfeat,vgg_a,ref_benchmark")
    ap.add_argument("--table", action="store_true", help="hbm_sweep: also print the rows as a table on stderr")
    ap.add_argument("--batch", type=int, default=None, help="override the workload's batch size")
    ap.add_argument("--cpu-sample-batch", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--conv-route", default="auto", choices=sorted(ROUTES),
                    help="how nn.SpatialConvolutionMM computes: im2col/GEMM/col2im columns, GEMMs that gather from "
                         "the padded image, or the library's choice per layer (its default)")
    ap.add_argument("--no-column-route", action="store_true", help="skip the second measurement on the column route")
    ap.add_argument("--no-fuse", action="store_true", help="run every ReLU as a pass of its own (no Sequential.fuse())")
    ap.add_argument("--reuse-finput", action="store_true",
                    help="accGradParameters trusts the forward pass's finput (the CPU module's behaviour) instead of "
                         "rebuilding it from its input (the reference GPU code's, the library's default)")
    ap.add_argument("--summarise", nargs="+", metavar="ARG", help="see summarise()")
    ap.add_argument("--summary-header", default=None, help="text put at the top of a --summarise output (\\n separated)")
    args = ap.parse_args()
    if args.summarise:
        return summarise(args)
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path is built and measured on a single MI355X "
                 "(--gpus %d is not supported: every GPU box of this build has one GPU, and the value reported "
                 "is that GPU's throughput)" % args.gpus)

    import numpy as np

    import mcw_cppamp_torch_amd as pkg
    from mcw_cppamp_torch_amd import gputorch, stacks

    lib = pkg._lib.lib
    if lib.thgpu_init() != 0:
        sys.exit("no GPU: " + lib.thgpu_last_error().decode())
    lib.thgpu_conv_set_finput_reuse(1 if args.reuse_finput else 0)
    if args.workload == "ref_benchmark":
        return ref_benchmark(args, pkg)
    if args.workload == "hbm_sweep":
        return hbm_sweep(args, pkg)
    if args.workload == "plan_check":
        return plan_check(args, pkg)

    name = args.workload
    B = args.batch or stacks.STACKS[name]["batch"]
    fused = not args.no_fuse
    net = stacks.build(name, seed_base=1000).gpu()
    if fused:
        net.fuse()
    x = pkg.FloatTensor(stacks.make_input(name, B, seed=1000)).gpu()
    rng = np.random.Generator(np.random.PCG64(1003))
    go = pkg.FloatTensor(rng.uniform(-1, 1, stacks.output_shape(name, B)).astype(np.float32)).gpu()

    def step():
        net.zeroGradParameters()
        net.forward(x)
        net.backward(x, go)

    def measure(route, steps, warmup, kernel_timing):
        """Times `steps` steps with the convolutions on `route`, then (kernel_timing) the same steps again with
        every launch bracketed by HIP events on the library's stream."""
        if lib.thgpu_conv_set_mode(ROUTES[route]) != 0:
            sys.exit(lib.thgpu_last_error().decode())
        for _ in range(warmup):
            step()
        gputorch.synchronize()
        ev0, ev1 = gputorch.Event(), gputorch.Event()
        t0 = time.perf_counter()
        ev0.record()
        for _ in range(steps):
            step()
        ev1.record()
        gputorch.synchronize()
        wall = time.perf_counter() - t0
        res = {"ms_per_step": wall * 1e3 / steps, "device_ms_per_step": ev0.elapsed_ms(ev1) / steps,
               "kernels": {}, "roofline": None, "gemm_shapes": [], "hbm_shapes": []}
        if not kernel_timing:
            return res
        kernels, gemm_shapes, hbm_shapes = res["kernels"], res["gemm_shapes"], res["hbm_shapes"]
        gputorch.prof_reset()
        gputorch.prof_enable(True)
        for _ in range(steps):
            step()
        gputorch.synchronize()
        rep = gputorch.prof_report()
        gputorch.prof_enable(False)
        gputorch.prof_reset()
        g_ms = g_fl = other_fl = 0.0
        g_calls = 0
        for kname, r in sorted(rep.items()):
            ms = r["ms"] / steps
            family = kname.split(" ")[0]          # GEMM records are labelled "<family> M=.. J=.. R=.. tile=.. split=.."
            if family.startswith("gemm_conv") or family == "gemm_blas":
                fl = r["flops"] / steps
                ent = kernels.setdefault(family, {"launches_per_step": 0.0, "ms_per_step": 0.0, "bound": "mfma",
                                                  "flops_per_step": 0.0})
                ent["launches_per_step"] += r["calls"] / steps
                ent["ms_per_step"] += ms
                ent["flops_per_step"] += fl
                gemm_shapes.append({"gemm": kname, "launches_per_step": r["calls"] / steps,
                                    "ms_per_step": round(ms, 4), "tflops": round(fl / ms / 1e9, 2),
                                    "frac": round(fl / ms / 1e9 / PEAK_MFMA_F32_TFLOPS, 4)})
                g_ms += ms
                g_fl += fl
                g_calls += r["calls"]
                continue
            # HBM-bound kernels: im2col / col2im / pooling records carry their geometry after the family name
            ent = kernels.setdefault(family, {"launches_per_step": 0.0, "ms_per_step": 0.0, "bytes_per_step": 0.0})
            ent["launches_per_step"] += r["calls"] / steps
            ent["ms_per_step"] += ms
            ent["bytes_per_step"] += r["bytes"] / steps
            if r["flops"] > 0:       # a convolution pass computed outside the GEMM kernels (conv_narrow_fwd): bound by
                other_fl += r["flops"] / steps          # its stores, listed with the HBM kernels; its flops are the layer's
                ent["flops_per_step"] = ent.get("flops_per_step", 0.0) + r["flops"] / steps
            if family != kname and r["bytes"] > 0:
                by = r["bytes"] / steps
                hbm_shapes.append({"kernel": kname, "launches_per_step": r["calls"] / steps,
                                   "ms_per_step": round(ms, 4), "gbs": round(by / ms / 1e6, 1),
                                   "frac": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)})
        for ent in kernels.values():
            if ent.get("bound") == "mfma":
                fl, ms = ent.pop("flops_per_step"), ent["ms_per_step"]
                ent.update(ms_per_step=round(ms, 4), tflops=round(fl / ms / 1e9, 2),
                           frac=round(fl / ms / 1e9 / PEAK_MFMA_F32_TFLOPS, 4))
            else:
                by, ms = ent.pop("bytes_per_step"), ent["ms_per_step"]
                ent["ms_per_step"] = round(ms, 4)
                if "flops_per_step" in ent:
                    ent["tflops"] = round(ent.pop("flops_per_step") / ms / 1e9, 2)
                if by > 0:
                    ent.update(bound="hbm", gbs=round(by / ms / 1e6, 1), frac=round(by / ms / 1e6 / PEAK_HBM_GBS, 4))
        if g_ms > 0:
            traffic, why = measured_gemm_traffic(name, B, route, fused, [s["gemm"] for s in gemm_shapes])
            if why:
                print("bench.py: roofline.traffic is null: " + why, file=sys.stderr)
            algorithmic = stacks.work(name, B)["gemm_flops"]
            if abs(g_fl + other_fl - algorithmic) > 1e-6 * algorithmic:
                sys.exit("bench.py: the convolution launches of a step declare %.6g flops, the stack's 3 x 2*M*N*K*B is %.6g"
                         % (g_fl + other_fl, algorithmic))
            res["roofline"] = {
                "bound": "mfma", "kernel": "gemm_fast_kernel<...> (all conv GEMM launches of a step)",
                "achieved": round(g_fl / g_ms / 1e9, 2), "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s",
                "frac": round(g_fl / g_ms / 1e9 / PEAK_MFMA_F32_TFLOPS, 4),
                "traffic": traffic, "traffic_note": why,
                "launches_per_step": g_calls / steps, "ms_per_step": round(g_ms, 4),
                "flops_per_step": g_fl,
            }
        return res

    main_run = measure(args.conv_route, args.steps, args.warmup, not args.no_kernel_timing)
    ms_per_step = main_run["ms_per_step"]
    kernels, roofline = main_run["kernels"], main_run["roofline"]
    gemm_shapes, hbm_shapes = main_run["gemm_shapes"], main_run["hbm_shapes"]

    # The same steps with every convolution on the column route (im2col, GEMM, col2im), for the figures of
    # those kernels at this workload's full geometries.
    column_route = None
    if args.conv_route != "columns" and not args.no_column_route:
        col = measure("columns", args.steps, 2, not args.no_kernel_timing)
        column_route = {
            "value": round(B / (col["ms_per_step"] / 1e3), 2), "unit": "images/s",
            "ms_per_step": round(col["ms_per_step"], 4), "roofline": col["roofline"],
            "kernels": {k: v for k, v in col["kernels"].items() if k in ("im2col", "col2im") or k.startswith("gemm_conv")},
            "hbm_shapes": [h for h in col["hbm_shapes"] if h["kernel"].startswith(("im2col", "col2im"))],
        }
        if lib.thgpu_conv_set_mode(ROUTES[args.conv_route]) != 0:
            sys.exit(lib.thgpu_last_error().decode())

    # Host<->device copies of one batch (blocking, pageable host memory), outside the timed region.
    host_x = stacks.make_input(name, B, seed=1000)
    t1 = time.perf_counter()
    x.copy(host_x)
    gputorch.synchronize()
    h2d_ms = (time.perf_counter() - t1) * 1e3
    t1 = time.perf_counter()
    net.gradInput.float()
    d2h_ms = (time.perf_counter() - t1) * 1e3

    w = stacks.work(name, B)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(name, min(args.cpu_sample_batch, B))

    line = {
        "metric": METRIC, "value": round(B / (ms_per_step / 1e3), 2), "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s conv stack, batch %d, input %s, fwd+bwd (zeroGradParameters, forward, "
                               "updateGradInput, accGradParameters)" % (name, B, "x".join(map(str, stacks.STACKS[name]["input"]))),
                   "batch": B, "conv_route": args.conv_route, "relu_fused": fused, "finput_reuse": bool(args.reuse_finput),
                   "device": gputorch.getDeviceProperties()["name"]},
        "device_ms_per_step": round(main_run["device_ms_per_step"], 4),
        "transfers": {"h2d_input_ms": round(h2d_ms, 3), "d2h_gradinput_ms": round(d2h_ms, 3),
                      "images_per_s_including_transfers": round(B / ((ms_per_step + h2d_ms + d2h_ms) / 1e3), 1)},
        "gemm_tflops_over_whole_step": round(w["gemm_flops"] / (ms_per_step / 1e3) / 1e12, 2),
        "roofline": roofline, "cpu_baseline": cpu, "kernels": kernels, "gemm_shapes": gemm_shapes,
        "hbm_shapes": hbm_shapes, "column_route": column_route,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
