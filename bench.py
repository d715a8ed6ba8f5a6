#!/usr/bin/env python3
"""Benchmark of the convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload alexnet]

A step is one forward + backward pass (zeroGradParameters, forward,
updateGradInput and accGradParameters of every module, as nn.Module:backward
does) of the AlexNet-style conv stack at batch 128, fp32, on synthetic inputs
that are resident in HBM before the timed region starts.  Prints ONE JSON line.

Beside the throughput the line carries
  roofline      the GEMM kernels (fp32 MFMA bound): algorithmic flops of all
                GEMM launches of a step / their summed HIP-event durations,
                measured in a second, instrumented run of the same K steps;
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
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "images/sec fwd+bwd, AlexNet-style conv stack b128 fp32; GEMM % fp32 MFMA peak"
PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM bytes per GEMM launch (average over the 15 launches of a step), from two rocprofv3 --pmc runs of this
# script (FETCH_SIZE x 2.0 and WRITE_SIZE x 1.0, the factors a plain copy kernel of known size gives);
# the summary with the commands is profiles/hbm_traffic_alexnet_b128_pmc.txt.  Counters cannot be read
# from inside the timed process, so the figure is carried here for the configuration it was measured on.
MEASURED_GEMM_TRAFFIC_BYTES_PER_LAUNCH = {("alexnet", 128, "auto"): 1.750e8, ("alexnet", 128, "columns"): 5.339e8}
ROUTES = {"columns": 0, "auto": 1, "gathered": 2}   # thgpu_conv_set_mode values


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="alexnet", choices=["alexnet", "overfeat", "vgg_a", "conv1_b16"])
    ap.add_argument("--batch", type=int, default=None, help="override the workload's batch size")
    ap.add_argument("--cpu-sample-batch", type=int, default=128)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--conv-route", default="auto", choices=sorted(ROUTES),
                    help="how nn.SpatialConvolutionMM computes: im2col/GEMM/col2im columns, GEMMs that gather from "
                         "the padded image, or the library's choice per layer (its default)")
    ap.add_argument("--no-column-route", action="store_true", help="skip the second measurement on the column route")
    args = ap.parse_args()
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

    name = args.workload
    B = args.batch or stacks.STACKS[name]["batch"]
    net = stacks.build(name, seed_base=1000).gpu()
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
        g_ms = g_fl = 0.0
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
                if by > 0:
                    ent.update(bound="hbm", gbs=round(by / ms / 1e6, 1), frac=round(by / ms / 1e6 / PEAK_HBM_GBS, 4))
        if g_ms > 0:
            res["roofline"] = {
                "bound": "mfma", "kernel": "gemm_fast_kernel<...> (all conv GEMM launches of a step)",
                "achieved": round(g_fl / g_ms / 1e9, 2), "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s",
                "frac": round(g_fl / g_ms / 1e9 / PEAK_MFMA_F32_TFLOPS, 4),
                "traffic": MEASURED_GEMM_TRAFFIC_BYTES_PER_LAUNCH.get((name, B, route)),
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
                   "batch": B, "conv_route": args.conv_route, "device": gputorch.getDeviceProperties()["name"]},
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
