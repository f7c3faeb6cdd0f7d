#!/usr/bin/env python3
"""Benchmark of the REEF hot path on one MI355X.

Workload (N=1): ResNet-152 forward pass, batch 1, fp32 NCHW 3x224x224, seeded
synthetic input and weights, one real-time client -- one "step" is one
inference through the executor's real-time (DKP-capable) kernels.  Inputs and
weights are resident in HBM before the timed region.

Prints ONE JSON line: the metric, the roofline of the dominant kernel family
(the fp32 implicit-GEMM convolution on the matrix cores) measured live with
device events on the stream the kernels run on, and a CPU baseline (the CPU
oracle executing the identical graph on the host cores).
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

FP32_MFMA_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix peak
HBM_PEAK_GBS = 8000.0


def percentile(a, q):
    return float(np.percentile(np.asarray(a, np.float64), q))


def cpu_baseline(model_dir, name, x, budget_s=30.0):
    """The CPU oracle (a port of the same graph to plain C loops, OpenMP over the
    host cores) timed on whole inferences of the same workload."""
    from oracle import oracle as O
    model = json.load(open(os.path.join(model_dir, name + ".json")))
    orc = O.GraphOracle(model, os.path.join(model_dir, name + ".param"))
    orc.set_input("data", x)
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    times = []
    t_start = time.time()
    while len(times) < 3 and (time.time() - t_start) < budget_s:
        t0 = time.time()
        orc.run()
        times.append(time.time() - t0)
    return {"value": round(min(times) * 1e3, 2), "unit": "ms", "cores": cores, "kind": "port",
            "sample": "%d whole ResNet-152 batch-1 inferences (22.56 GFLOP each), best of them"
                      % len(times)}, orc


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--kernel-iters", type=int, default=20)
    ap.add_argument("--model", default="resnet152")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--workdir", default=None)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (replicas per GPU share nothing); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from reef_amd import binding as B
    from reef_amd.modelgen import nets

    layers = {"resnet152": 152, "resnet18": 18}[args.model]
    g = nets.resnet(layers)
    tmp = tempfile.TemporaryDirectory(dir=args.workdir)
    d = g.write(os.path.join(tmp.name, g.name))
    d = os.path.dirname(d)
    x = nets.image_input(g.name, (3, 224, 224))

    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe.set_input_checked("data", x)

    # ---- whole-model latency: W warm-up steps, then exactly K timed steps -------------
    t0 = time.perf_counter()
    lat_us, dev_us = exe.time_model(B.RUN_DEFAULT, args.warmup, args.steps)
    wall_s = time.perf_counter() - t0
    ms_per_step = float(lat_us.sum()) / args.steps / 1e3
    p50, p99 = percentile(lat_us, 50) / 1e3, percentile(lat_us, 99) / 1e3

    # ---- per-kernel durations (device events around back-to-back launches) ------------
    n = exe.num_kernels()
    kus = np.array([exe.time_kernel(i, B.RUN_DEFAULT, 3, args.kernel_iters) for i in range(n)])
    names = [k["name"].split("#")[0] for k in g.kernels]
    flops = np.array(g.kernel_flops, np.float64)
    by = {}
    for i, nm in enumerate(names):
        e = by.setdefault(nm, {"us": 0.0, "flops": 0.0, "bytes": 0.0, "launches": 0})
        e["us"] += kus[i]
        e["flops"] += flops[i]
        e["bytes"] += g.kernel_bytes[i]
        e["launches"] += 1
    conv = {k: v for k, v in by.items() if k.startswith("reef_conv2d_")}
    dom = max(conv, key=lambda k: conv[k]["us"])
    dom_e = conv[dom]
    dom_tflops = dom_e["flops"] / dom_e["us"] / 1e6
    conv_us = sum(v["us"] for v in conv.values())
    conv_flops = sum(v["flops"] for v in conv.values())
    best_i = int(np.argmax(np.where(flops > 0, flops / np.maximum(kus, 1e-3), 0)))

    out = {
        "metric": "ResNet-152 batch-1 RT latency p99 (solo RT client)",
        "value": round(p99, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "ResNet-152 v2 (TVM relay.testing wiring, BN folded), batch 1, fp32 NCHW "
                               "3x224x224, seeded He-normal weights; one RT client, no BE load",
                   "kernels_per_inference": n, "gflop_per_inference": round(g.flops / 1e9, 3)},
        "rt_latency_ms": {"p50": round(p50, 4), "p99": round(p99, 4),
                          "mean_device": round(float(dev_us.mean()) / 1e3, 4)},
        "model_tflops": round(g.flops / (ms_per_step * 1e-3) / 1e12, 3),
        "conv_tflops_all_layers": round(conv_flops / conv_us / 1e6, 3),
        "best_layer": {"kernel": names[best_i], "attrs": g.kernels[best_i]["attrs"][:12],
                       "tflops": round(float(flops[best_i] / kus[best_i] / 1e6), 2)},
        "sum_kernel_us": round(float(kus.sum()), 1),
        "roofline": {
            "bound": "mfma",
            "kernel": dom,
            "achieved": round(dom_tflops, 3),
            "peak": FP32_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(dom_tflops / FP32_MFMA_PEAK_TFLOPS, 4),
            "traffic": None,
            "launches_per_inference": dom_e["launches"],
            "avg_launch_us": round(dom_e["us"] / dom_e["launches"], 3),
            "avg_launch_gflop": round(dom_e["flops"] / dom_e["launches"] / 1e9, 4),
        },
        "per_kernel": {k: {"launches": v["launches"], "avg_us": round(v["us"] / v["launches"], 3),
                           "tflops": round(v["flops"] / v["us"] / 1e6, 3),
                           "gbs": round(v["bytes"] / v["us"] / 1e3, 1)} for k, v in sorted(by.items())},
        "timed_region_wall_s": round(wall_s, 3),
    }
    if not args.no_cpu:
        cb, orc = cpu_baseline(d, g.name, x)
        out["cpu_baseline"] = cb
        got = exe.get_output()
        ref = orc.get("output")
        out["parity_max_abs_err_vs_oracle"] = float(np.abs(got - ref).max())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
