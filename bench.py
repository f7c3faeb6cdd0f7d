#!/usr/bin/env python3
"""Benchmark of the REEF hot path on one MI355X.

Workload (N=1): one real-time client running ResNet-152 (batch 1, fp32 NCHW
3x224x224) with Poisson arrivals, mean interval 20 ms, while 4 best-effort
clients loop DenseNet-201 (growth 32, batch 1, 224x224) on the same GPU through
one REEFScheduler.  All weights and inputs are seeded synthetic data, resident
in HBM before the timed region.  One "step" is one real-time request; the
value is the p99 of its latency (submit -> result ready at the scheduler API)
over exactly --steps recorded requests, after --warmup unrecorded ones.

The same JSON line carries
  * the same real-time request stream served with no best-effort load (same
    seed, same arrival times), for the "within 5 % of solo" comparison;
  * preemption latency (flag raised -> every best-effort stream drained);
  * best-effort throughput with and without the real-time client;
  * the roofline of the dominant kernel family of ResNet-152 (fp32 implicit-GEMM
    convolution on the matrix cores), timed with device events on the stream
    the kernels are launched on;
  * a CPU baseline: the same ResNet-152 graph executed by the CPU oracle on the
    host cores;
  * the convolution tiles on two device-filling layers (`steady_state_conv`), to separate what
    the K loop sustains from what a batch-1 launch allows;
  * two further co-location scenarios (dynamic kernel padding with a
    MobileNetV2 best-effort client; Inception-v3 real-time with two BERT-base
    best-effort clients), shorter runs.

Standard output is ONE compact JSON line (a few KB: the contract fields, `roofline`,
`cpu_baseline` and a handful of scalars to read beside `value`).  Everything else -- every
co-location leg in full, the per-kernel and per-shape tables, the schedule modes -- goes to
the file named by --detail-out.  After every co-location leg the real-time model's and every
best-effort model's storages are compared bit for bit with a solo run of the same model
(`corun_outputs_bit_identical`); a difference makes the run exit non-zero.
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
MEAN_INTERVAL_US = 20000.0
SEED = 0x5EEF


def pct(a, q):
    return round(float(np.percentile(np.asarray(a, np.float64), q)) / 1e3, 4)


def cpu_baseline(model_dir, name, x, budget_s=30.0):
    """The CPU oracle (a port of the same graph to plain C loops, OpenMP over the
    host cores) timed on whole inferences of the same model."""
    from oracle import oracle as O
    model = json.load(open(os.path.join(model_dir, name + ".json")))
    orc = O.GraphOracle(model, os.path.join(model_dir, name + ".param"))
    orc.set_input("data", x)
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    times = []
    t_start = time.time()
    while len(times) < 5 and (time.time() - t_start) < budget_s:
        t0 = time.time()
        orc.run()
        times.append(time.time() - t0)
    return {"value": round(min(times) * 1e3, 2), "unit": "ms", "cores": cores, "kind": "port",
            "sample": "%d whole ResNet-152 batch-1 inferences (22.56 GFLOP each) by the CPU oracle "
                      "(C, OpenMP), best of them; TVM is not installed, so this stands in for the "
                      "TVM-llvm build of the model" % len(times)}, orc


def torch_cpu_baseline(g, x, budget_s=20.0):
    """The same ResNet-152 (pre-activation, folded batch norms: the network nets.resnet builds,
    parameters taken in order of definition) as a torch.nn.functional program on the host cores
    (oneDNN), fp32.  Returns None where torch is not importable."""
    try:
        import torch
        import torch.nn.functional as F
    except Exception:
        return None
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    torch.set_num_threads(threads)
    params = [torch.from_numpy(np.asarray(a, np.float32)) for k, a in g.params
              if not k.endswith("k")]       # without the packed copies of the 3x3 weights

    def forward():
        it = iter(params)
        take = lambda *shape: next(it).reshape(shape)
        units, filters = [3, 8, 36, 3], [64, 256, 512, 1024, 2048]
        t = torch.from_numpy(x)[None] + take(1, 3, 1, 1)
        t = F.relu(F.conv2d(t, take(64, 3, 7, 7), take(64), stride=2, padding=3))
        act = F.relu(F.max_pool2d(t, 3, 2, 1) + take(1, 64, 1, 1))
        raw = None
        for si, n in enumerate(units):
            cout, mid = filters[si + 1], filters[si + 1] // 4
            for ui in range(n):
                first, last = ui == 0, ui == n - 1
                stride = (1 if si == 0 else 2) if first else 1
                cin = act.shape[1]
                if first:   # conv1 and the projection shortcut: one stacked filter [conv1 | shortcut]
                    both = F.conv2d(act, take(mid + cout, cin, 1, 1), None, stride=stride)
                    y = F.relu(both + take(1, mid + cout, 1, 1))[:, :mid]
                    sc = both[:, mid:]
                else:
                    y = F.relu(F.conv2d(act, take(mid, cin, 1, 1), take(mid)))
                    sc = raw
                y = F.relu(F.conv2d(y, take(mid, mid, 3, 3), take(mid), padding=1))
                w3 = take(cout, mid, 1, 1)
                if last and si == 3:
                    act = F.relu((F.conv2d(y, w3) + sc) * take(1, cout, 1, 1) + take(1, cout, 1, 1))
                elif last:
                    act = F.relu(F.conv2d(y, w3, take(cout)) + sc)
                else:
                    raw = F.conv2d(y, w3) + sc
                    act = F.relu(raw + take(1, cout, 1, 1))
        t = act.mean(dim=(2, 3))
        return F.linear(t, take(1000, 2048), take(1000))

    with torch.no_grad():
        logits = forward()
        times = []
        t_start = time.time()
        while len(times) < 10 and (time.time() - t_start) < budget_s:
            t0 = time.time()
            forward()
            times.append(time.time() - t0)
    return {"value": round(min(times) * 1e3, 2), "unit": "ms", "threads": threads,
            "sample": "%d whole inferences of the same network as torch.nn.functional calls "
                      "(torch %s, CPU, fp32), best of them" % (len(times), torch.__version__)}, logits.numpy().ravel()


def kernel_sources_sha256():
    """Fingerprint of the device code the committed counter summaries were taken with."""
    import hashlib
    h = hashlib.sha256()
    base = os.path.join(ROOT, "reef_amd", "csrc", "kernels")
    for f in sorted(os.listdir(base)) + ["../../../include/reef_kernels.h"]:
        with open(os.path.join(base, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def solo_kernel_table(models, name, iters):
    """Per kernel symbol of one model run alone: launches, average duration, and the fraction of
    each roofline (matrix-core FLOPs and HBM bytes, algorithmic)."""
    from reef_amd import binding as B
    g, d = models[name]
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    key, x = model_input(name)
    exe.set_input_checked(key, x)
    exe.execute()
    by = {}
    for i, k in enumerate(g.kernels):
        us = exe.time_kernel(i, B.RUN_DEFAULT, 3, iters)
        e = by.setdefault(k["name"].split("#")[0], {"us": 0.0, "flops": 0.0, "bytes": 0.0, "launches": 0})
        e["us"] += us
        e["flops"] += g.kernel_flops[i]
        e["bytes"] += g.kernel_bytes[i]
        e["launches"] += 1
    _, dev_us = exe.time_model(B.RUN_DEFAULT, 10, 50)
    exe.close()
    return {"model_device_ms": round(float(dev_us.mean()) / 1e3, 4),
            "kernels": {k: {"launches": v["launches"], "avg_us": round(v["us"] / v["launches"], 3),
                            "frac_mfma_peak": round(v["flops"] / v["us"] / 1e6 / FP32_MFMA_PEAK_TFLOPS, 4),
                            "gbs": round(v["bytes"] / v["us"] / 1e3, 1),
                            "frac_hbm_peak": round(v["bytes"] / v["us"] / 1e3 / HBM_PEAK_GBS, 4)}
                        for k, v in sorted(by.items())}}


def steady_state_conv(root, iters):
    """The staged convolution tiles on two layers large enough to fill the device (12544 and
    3136 output pixels): what the K loop sustains when a launch is not latency bound."""
    from reef_amd import binding as B
    from reef_amd.modelgen import builder as MB
    from reef_amd.modelgen import tiling
    cases = [("3x3 256->256 @112x112", 256, 112, 256, 3, 1, "128x64"),
             ("1x1 1024->1024 @56x56", 1024, 56, 1024, 1, 0, "64x64")]
    g = MB.GraphBuilder("steady")
    meta = []
    for label, cin, hw, cout, k, pad, tile in cases:
        x = g.input("in_%d_%d" % (cin, hw), (cin, hw, hw))
        g.conv2d(x, cout, k, 1, pad, bias=True, act=MB.ACT_RELU,
                 force=tiling.forced(tile, cout, hw * hw, cin * k * k, 1, k * k))
        meta.append((label, tile, len(g.kernels) - 1, 2.0 * cout * hw * hw * cin * k * k))
    d = os.path.dirname(g.write(os.path.join(root, g.name)))
    exe = B.Executor.from_dir(d, g.name, B.BASE)
    out = []
    for label, tile, idx, fl in meta:
        us = exe.time_kernel(idx, B.RUN_DEFAULT, 3, iters)
        out.append({"layer": label, "kernel": g.kernels[idx]["name"].split("#")[0], "us": round(us, 2),
                    "tflops": round(fl / us / 1e6, 2),
                    "frac_mfma_peak": round(fl / us / 1e6 / FP32_MFMA_PEAK_TFLOPS, 4)})
    exe.close()
    return out


def calibrate_copy(mib, root):
    """A plain copy kernel over a known number of bytes: what the memory counters read for
    it fixes their scale."""
    from reef_amd import binding as B
    from reef_amd.modelgen import builder as MB
    n = mib * 1024 * 1024 // 4
    g = MB.GraphBuilder("copycal")
    x = g.input("data", (n,))
    g.copy_into(x, g.temp((n,), name="output"), 0)
    d = os.path.dirname(g.write(os.path.join(root, g.name)))
    exe = B.Executor.from_dir(d, g.name, B.BASE)
    for _ in range(20):
        exe.execute()
    exe.close()


def write_models(names, root, measured_profiles=True):
    """Writes each model directory; its <model>.profile.json (per-kernel latencies that drive
    dynamic kernel padding) is then measured on this device, replacing the generator's
    estimate."""
    from reef_amd import profiler
    from reef_amd.modelgen import nets
    out = {}
    for n in names:
        g = nets.BUILDERS[n]()
        d = os.path.dirname(g.write(os.path.join(root, g.name)))
        if measured_profiles:
            t0 = time.perf_counter()
            profiler.write_profile(d, g.name, iters=5, warmup=1)
            print("bench: measured profile of %s in %.1f s" % (n, time.perf_counter() - t0), file=sys.stderr)
        out[n] = (g, d)
    return out


def model_input(name):
    from reef_amd.modelgen import nets
    if name == "bert_base":
        return "input0", nets.token_input(name, 128, 30522)
    side = 299 if name == "inceptionv3" else 224
    return "data", nets.image_input(name, (3, side, side))


class SoloBits:
    """Every float storage a model's kernels write, after one uninterrupted run of the model
    alone: what the same model must hold, bit for bit, after a co-location leg -- preempted and
    restarted, padded into real-time launches or sharing its launches with best-effort work
    (the two guarantees of src/reef/test/test.cpp:448-536)."""

    def __init__(self, models, name):
        from reef_amd import binding as B
        g, d = models[name]
        self.name = name
        self.model = json.load(open(os.path.join(d, g.name + ".json")))
        written = set()
        for k in self.model["kernels"]:
            written.update(k["args"])
        # not inputs, parameters, arrival counters or the split-K workspaces (scratch whose
        # content depends on how the kernel was launched)
        self.idx = [i for i in sorted(written)
                    if self.model["storage"][i]["stype"] == "float32"
                    and self.model["storage"][i]["name"] not in ("data", "input0", "reef_sync")
                    and not self.model["storage"][i]["name"].startswith("p")]
        key, x = model_input(name)
        exe = B.Executor.from_dir(d, g.name, B.HYBRID)
        exe.set_input_checked(key, x)
        exe.execute()
        self.state = {i: exe.get_data(i, self.model["storage"][i]["size"]) for i in self.idx}
        exe.close()

    def differs(self, sched, mid):
        """None, or a description of the first storage of model `mid` that differs."""
        for i in self.idx:
            got = sched.get_data(mid, i, self.model["storage"][i]["size"])
            if not np.array_equal(got, self.state[i]):
                bad = int(np.flatnonzero(got != self.state[i])[0])
                return "%s storage %d element %d: %r vs solo %r" % (self.name, i, bad, float(got[bad]),
                                                                    float(self.state[i][bad]))
        for i, st in enumerate(self.model["storage"]):
            if st["name"] == "reef_sync" and sched.get_data(mid, i, st["size"], np.int32).any():
                return "%s: split-K arrival counters left non-zero" % self.name
        return None


_SOLO_BITS = {}


def solo_bits(models, name):
    if name not in _SOLO_BITS:
        _SOLO_BITS[name] = SoloBits(models, name)
    return _SOLO_BITS[name]


def summarize(r, sched, n_be):
    lat = r["rt_latency_us"]
    return {"rt_ms": {"p50": pct(lat, 50), "p99": pct(lat, 99), "mean": round(float(lat.mean()) / 1e3, 4),
                      "max": round(float(lat.max()) / 1e3, 4)},
            "rt_exec_ms": {"p50": pct(r["rt_exec_us"], 50), "p99": pct(r["rt_exec_us"], 99)},
            "rt_queue_ms": {"p50": pct(r["rt_queue_us"], 50), "p99": pct(r["rt_queue_us"], 99)},
            "be_inferences_per_s": round(float(r["be_completed"].sum()) / r["span_s"], 2) if n_be else 0.0,
            "be_completed": [int(v) for v in r["be_completed"]],
            "be_preempted": [int(v) for v in r["be_preempted"]],
            "be_padded": [int(v) for v in r["be_padded"]],
            "span_s": round(r["span_s"], 3)}


def corun(models, rt_name, be_name, n_be, mode, requests, warmup, wait_sync=True, solo=True,
          dkp_slack=None, interval_us=MEAN_INTERVAL_US):
    """One scheduler, one real-time model, n_be best-effort clients of one model."""
    from reef_amd import binding as B
    s = B.Scheduler(mode)
    s.set_wait_sync(wait_sync)
    if dkp_slack is not None:
        s.set_dkp_slack_percent(dkp_slack)
    g_rt, d_rt = models[rt_name]
    rt = s.load_model(d_rt, g_rt.name)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt)
    key, x = model_input(rt_name)
    assert s.set_input(rt, x, key) == 0
    bes = []
    g_be, d_be = models[be_name]
    bkey, bx = model_input(be_name)
    for _ in range(n_be):
        m = s.load_model(d_be, g_be.name)
        s.bind_model_queue(s.create_queue(B.QUEUE_BE), m)
        assert s.set_input(m, bx, bkey) == 0
        bes.append(m)
    s.run()
    out = {"mode": {B.MODE_REEF: "REEF (reset-based preemption + dynamic kernel padding)",
                    B.MODE_RESET: "Reset (reset-based preemption only)",
                    B.MODE_WAITPREEMPT: "WaitPreempt (flag, then wait for everything launched)",
                    B.MODE_NOPREEMPT: "NoPreempt (wait for the best-effort runs in flight)",
                    B.MODE_MULTISTREAM: "MultiStream (no switch: real-time kernels beside best-effort ones)"}[mode],
           "rt_model": g_rt.name, "be_model": g_be.name, "be_clients": n_be}
    if solo:
        r0 = s.run_load(rt, [], requests, warmup=warmup, mean_interval_us=interval_us, seed=SEED)
        out["solo"] = summarize(r0, s, 0)
    rb = s.run_load(rt, bes, 0, be_only_ms=1500)
    out["be_only_inferences_per_s"] = round(float(rb["be_completed"].sum()) / rb["span_s"], 2)
    r1 = s.run_load(rt, bes, requests, warmup=warmup, mean_interval_us=interval_us, seed=SEED)
    out["loaded"] = summarize(r1, s, n_be)
    ps = s.preempt_samples()
    ps = ps[-(requests):] if len(ps) > requests else ps
    out["preempt_us"] = {"n": int(len(ps)), "mean": round(float(ps.mean()), 2) if len(ps) else None,
                         "p50": float(np.percentile(ps, 50)) if len(ps) else None,
                         "p99": float(np.percentile(ps, 99)) if len(ps) else None,
                         "max": int(ps.max()) if len(ps) else None,
                         "what": "host span: flag stored into device memory -> host queues dropped -> "
                                 "every best-effort stream has no kernel left on the device"
                                 if wait_sync else "host span without waiting for the device to drain"}
    dev = s.preempt_device_samples()
    late = s.preempt_device_late()
    late = late[:len(dev)] if len(late) >= len(dev) else np.zeros(len(dev), bool)
    if len(dev) > requests:
        dev, late = dev[-requests:], late[-requests:]
    on_dev = dev[~late]
    out["preempt_us"]["device"] = {
        "n": int(len(dev)), "mean": round(float(dev.mean()), 2) if len(dev) else None,
        "p50": round(float(np.percentile(dev, 50)), 2) if len(dev) else None,
        "p99": round(float(np.percentile(dev, 99)), 2) if len(dev) else None,
        "max": round(float(dev.max()), 2) if len(dev) else None,
        "clock_sync_err_us": round(s.clock_sync_error_us(), 2),
        "late_launch_samples": int(late.sum()),
        "without_late_launches": {"n": int(len(on_dev)),
                                  "mean": round(float(on_dev.mean()), 2) if len(on_dev) else None,
                                  "p99": round(float(np.percentile(on_dev, 99)), 2) if len(on_dev) else None,
                                  "max": round(float(on_dev.max()), 2) if len(on_dev) else None},
        "what": "flag store (host clock) -> the last best-effort workgroup that was on the device has left "
                "(device wall clock written by that workgroup, mapped to the host clock).  late_launch_samples: "
                "preemptions during which a stream was handing a launch to the runtime; that launch reaches the "
                "device later, finds the flag and leaves, and the sample runs until its exit (without_late_launches "
                "leaves those samples out)"}
    out["preempt_phase_ns"] = s.preempt_phases()
    out["padded_kernels"] = int(s.padded_kernels())
    out["kernel_select_ns"] = int(s.avg_kernel_sel_latency())
    # the clients stopped after their current task; every best-effort model completes one more
    # uninterrupted inference so that its final state is that of a whole run, then every model
    # of this scheduler must hold the bits of its solo run
    if n_be:
        s.run_load(rt, bes, 0, be_only_ms=40)
    why = solo_bits(models, rt_name).differs(s, rt)
    for m in bes:
        why = why or solo_bits(models, be_name).differs(s, m)
    out["outputs_bit_identical_to_solo"] = why is None
    if why is not None:
        out["outputs_differ"] = why
        print("bench: co-run outputs differ from the solo run: %s" % why, file=sys.stderr)
    s.shutdown()
    s.close()
    return out


def corun_legs(detail):
    """Every co-location leg (a dict with a `loaded` summary) anywhere in the full result."""
    legs = []

    def walk(v):
        if isinstance(v, dict):
            if "loaded" in v and "outputs_bit_identical_to_solo" in v:
                legs.append(v)
            for k, w in v.items():
                if k != "schedule_modes":
                    walk(w)
    walk(detail)
    return legs


COMPACT_LIMIT = 6144


def compact_line(detail):
    """The one line of standard output: the contract fields, `roofline`, `cpu_baseline` and the few
    scalars needed to read `value` (with --steps 20 the p99 is the largest of 20 Poisson-queued
    requests: `rt_p50_ms` and the execution-only percentiles say what a request costs without
    the queueing).  Kept below COMPACT_LIMIT bytes whatever the full result holds."""
    keep = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
            "scaling", "vs_baseline", "dtype", "data", "config")
    line = {k: detail.get(k) for k in keep}
    rf = detail.get("roofline") or {}
    line["roofline"] = {k: rf.get(k) for k in ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic",
                                                "launches_per_inference", "avg_launch_us", "avg_launch_gflop")}
    cb = detail.get("cpu_baseline")
    if cb is not None:
        line["cpu_baseline"] = {k: cb.get(k) for k in ("value", "unit", "cores", "kind", "sample")}
        line["cpu_baseline"]["sample"] = str(line["cpu_baseline"]["sample"])[:300]
        if "oracle" in cb:
            line["cpu_baseline"]["oracle_ms"] = cb["oracle"]["value"]
    head = detail.get("corun_resnet152_4x_densenet201") or {}
    loaded, solo = head.get("loaded") or {}, head.get("solo") or {}
    pre = head.get("preempt_us") or {}
    dev = pre.get("device") or {}

    def at(dct, *path):
        for k in path:
            dct = dct.get(k) if isinstance(dct, dict) else None
        return dct
    line.update({
        "rt_p50_ms": at(loaded, "rt_ms", "p50"),
        "rt_exec_p50_ms": at(loaded, "rt_exec_ms", "p50"),
        "rt_exec_p99_ms": at(loaded, "rt_exec_ms", "p99"),
        "rt_solo_p50_ms": at(solo, "rt_ms", "p50"),
        "rt_solo_p99_ms": at(solo, "rt_ms", "p99"),
        "rt_p99_vs_solo": detail.get("rt_p99_vs_solo"),
        "rt_p50_vs_solo": detail.get("rt_p50_vs_solo"),
        "rt_exec_p99_vs_solo": detail.get("rt_exec_p99_vs_solo"),
        "preempt_host_us": {k: pre.get(k) for k in ("mean", "p99", "max")} if pre else None,
        "preempt_device_us": {k: dev.get(k) for k in ("mean", "p99", "max")} if dev else None,
        "be_inferences_per_s": loaded.get("be_inferences_per_s"),
        "be_only_inferences_per_s": head.get("be_only_inferences_per_s"),
        "solo_device_ms": at(detail, "solo_back_to_back_ms", "mean_device"),
        "rt_launches_per_inference": at(detail, "config", "rt_kernels_per_inference"),
        "model_tflops": detail.get("model_tflops"),
        "conv_tflops_all_layers": detail.get("conv_tflops_all_layers"),
        "corun_outputs_bit_identical": detail.get("corun_outputs_bit_identical"),
        "parity_logits_max_rel_err_vs_oracle": detail.get("parity_logits_max_rel_err_vs_oracle"),
    })
    other = {}
    for key, label in (("corun_dkp_mobilenetv2", "cfg4_rt_resnet152_be_mobilenetv2"),
                       ("corun_inceptionv3_2x_bert", "cfg5_rt_inceptionv3_be_2x_bert_base")):
        leg = detail.get(key)
        if leg is None:
            continue
        reset = None
        if "reef" in leg:
            leg, reset = leg["reef"], leg.get("reset")
        other[label] = {"rt_exec_p50_ms": at(leg, "loaded", "rt_exec_ms", "p50"),
                        "rt_solo_exec_p50_ms": at(leg, "solo", "rt_exec_ms", "p50"),
                        "be_inferences_per_s": at(leg, "loaded", "be_inferences_per_s"),
                        "padded_kernels": leg.get("padded_kernels"),
                        "preempt_device_us_p99": at(leg, "preempt_us", "device", "p99")}
        if reset is not None:
            other[label]["be_inferences_per_s_reset_mode"] = at(reset, "loaded", "be_inferences_per_s")
    leg16 = detail.get("corun_16_be_queues")
    if leg16 is not None:
        other["headline_with_16_be_queues"] = {"rt_p50_ms": at(leg16, "loaded", "rt_ms", "p50"),
                                               "rt_exec_p99_ms": at(leg16, "loaded", "rt_exec_ms", "p99"),
                                               "be_inferences_per_s": at(leg16, "loaded", "be_inferences_per_s"),
                                               "preempt_device_us_p99": at(leg16, "preempt_us", "device", "p99")}
    if other:
        line["other_configs"] = other
    for nm in ("mobilenetv2", "bert_base"):
        v = at(detail, "solo_kernels_" + nm, "model_device_ms")
        if v is not None:
            line.setdefault("solo_device_ms_other_models", {})[nm] = v
    text = json.dumps(line, separators=(",", ":"))
    for drop in ("solo_device_ms_other_models", "other_configs"):   # never reached at today's sizes
        if len(text) <= COMPACT_LIMIT:
            break
        line.pop(drop, None)
        text = json.dumps(line, separators=(",", ":"))
    return text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400, help="recorded real-time requests")
    ap.add_argument("--warmup", type=int, default=40, help="real-time requests before recording")
    ap.add_argument("--kernel-iters", type=int, default=20)
    ap.add_argument("--configs", default="3,4,5,6,7,8",
                    help="co-location scenarios to run (3 is the headline; 6 = dynamic kernel padding under "
                         "a real-time request every 2 ms; 7 = the headline workload in every schedule mode; "
                         "8 = the headline workload with 16 best-effort queues)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--solo-only", action="store_true",
                    help="only the solo ResNet-152 executor part (whole-model and per-kernel timing); "
                         "the value is then the solo p99 -- this is the command the kernel profiles "
                         "under profiles/ are taken with")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="also run a plain copy kernel over this many MiB 20 times (scale for the "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--workdir", default=None)
    ap.add_argument("--detail-out", default=None, metavar="FILE",
                    help="where the full result goes (every co-location leg, per-kernel and per-shape tables); "
                         "default gpurun_out/bench_detail.json beside this file")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (replicas per GPU share nothing); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    configs = [int(c) for c in args.configs.split(",") if c]

    from reef_amd import binding as B

    tmp = tempfile.TemporaryDirectory(dir=args.workdir)
    names = ["resnet152"] if args.solo_only else ["resnet152", "densenet201"]
    if args.solo_only:
        configs = []
    if 4 in configs or 6 in configs:
        names.append("mobilenetv2")
    if 5 in configs:
        names += ["inceptionv3", "bert_base"]
    models = write_models(names, tmp.name, measured_profiles=not args.solo_only)
    g, d = models["resnet152"]
    _, x = model_input("resnet152")

    if args.calibrate_copy:
        calibrate_copy(args.calibrate_copy, tmp.name)

    # ---- headline: RT ResNet-152 + 4 BE DenseNet-201 ----------------------------------
    head = reset_only = no_drain_wait = None
    wall_s = 0.0
    if not args.solo_only:
        t0 = time.perf_counter()
        head = corun(models, "resnet152", "densenet201", 4, B.MODE_REEF, args.steps, args.warmup)
        wall_s = time.perf_counter() - t0
        reset_only = corun(models, "resnet152", "densenet201", 4, B.MODE_RESET, args.steps, args.warmup,
                           solo=False)
        # the scheduler's own default, as in the reference (scheduler.cpp:41): a preemption does not
        # wait for the device to drain -- the real-time kernels queue up behind the leaving ones.
        # The headline run waits, because only then is the length of a preemption measured.
        no_drain_wait = corun(models, "resnet152", "densenet201", 4, B.MODE_REEF, args.steps, args.warmup,
                              wait_sync=False, solo=False)

    # ---- solo executor: whole-model device time and per-kernel durations ---------------
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe.set_input_checked("data", x)
    t0 = time.perf_counter()
    solo_iters = args.steps if args.solo_only else 200
    lat_us, dev_us = exe.time_model(B.RUN_DEFAULT, args.warmup if args.solo_only else 20, solo_iters)
    if args.solo_only:
        wall_s = time.perf_counter() - t0
    n = exe.num_kernels()
    # Per kernel: the average of back-to-back launches of the kernel alone (its operands cached
    # after the first), corrected to what the kernel costs inside a pass of the model, where it
    # finds its weights in HBM and its input wherever the previous layer left it: one launch
    # between two events in the model's order minus the same directly after itself.  Everything
    # below (roofline, tables) uses the in-model figure; their sum is checked against the
    # device time of a whole pass.
    kus_b2b = np.array([exe.time_kernel(i, B.RUN_DEFAULT, 3, args.kernel_iters) for i in range(n)])
    order = np.array([exe.time_kernel_in_model(i, B.RUN_DEFAULT, 5) for i in range(n)])
    extra = order[:, 0] - order[:, 1]
    # the two events around the single launch keep its neighbours from overlapping its start and
    # its end, so the corrections overshoot a little: one common factor makes the figures add up
    # to the device time of a whole pass
    alpha = float(np.clip((float(dev_us.mean()) - kus_b2b.sum()) / max(extra.sum(), 1e-6), 0.0, 1.0))
    kus = np.maximum(kus_b2b + alpha * extra, 0.5 * kus_b2b)
    names_k = [k["name"].split("#")[0] for k in g.kernels]
    flops = np.array(g.kernel_flops, np.float64)
    by = {}
    for i, nm in enumerate(names_k):
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
    # HBM bytes per launch from the committed counter runs -- only while the device code is the
    # code those runs were taken with
    traffic = None
    traffic_note = "no counter summary committed"
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        tj = json.load(open(tpath))
        if tj.get("kernel_sources_sha256") != kernel_sources_sha256():
            traffic_note = "profiles/traffic.json was taken with other kernel sources: not reported"
        else:
            traffic = tj.get("bytes_per_launch", {}).get(dom)
            traffic_note = "profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel)"
    # every distinct convolution shape of the model
    shapes = {}
    for i, nm in enumerate(names_k):
        if not nm.startswith("reef_conv2d_"):
            continue
        a = g.kernels[i]["attrs"]
        e = shapes.setdefault((tuple(a[:12]), nm), {"us": 0.0, "flops": 0.0, "n": 0})
        e["us"] += kus[i]
        e["flops"] += flops[i]
        e["n"] += 1
    conv_shapes = [{"cin_h_w": list(sh[:3]), "cout_ho_wo": list(sh[3:6]), "k": list(sh[6:8]), "stride": list(sh[8:10]),
                    "kernel": nm, "launches": e["n"], "avg_us": round(e["us"] / e["n"], 2),
                    "tflops": round(e["flops"] / e["us"] / 1e6, 2),
                    "frac_mfma_peak": round(e["flops"] / e["us"] / 1e6 / FP32_MFMA_PEAK_TFLOPS, 4)}
                   for (sh, nm), e in sorted(shapes.items(), key=lambda kv: -kv[1]["us"])]

    if args.solo_only:
        p99 = pct(lat_us, 99)
        solo_p99 = p99
    else:
        p99 = head["loaded"]["rt_ms"]["p99"]
        solo_p99 = head["solo"]["rt_ms"]["p99"]
    out = {
        "metric": "ResNet-152 RT p99 latency, solo, back to back" if args.solo_only
                  else "ResNet-152 RT p99 latency w/ 4 BE clients",
        "value": p99,
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(float(lat_us.mean()) / 1e3, 4) if args.solo_only else head["loaded"]["rt_ms"]["mean"],
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "RT ResNet-152 (batch 1, fp32 NCHW 3x224x224, Poisson arrivals mean 20 ms, "
                               "seed 0x5EEF) + 4 BE clients looping DenseNet-201 (growth 32, batch 1, "
                               "224x224); seeded He-normal weights; REEF mode",
                   "rt_kernels_per_inference": n, "rt_gflop_per_inference": round(g.flops / 1e9, 3)},
        "rt_p99_vs_solo": round(p99 / solo_p99, 4),
        "rt_p50_vs_solo": None if args.solo_only
        else round(head["loaded"]["rt_ms"]["p50"] / head["solo"]["rt_ms"]["p50"], 4),
        "rt_exec_p99_vs_solo": None if args.solo_only
        else round(head["loaded"]["rt_exec_ms"]["p99"] / head["solo"]["rt_exec_ms"]["p99"], 4),
        "preempt_us": None if args.solo_only else head["preempt_us"],
        "corun_resnet152_4x_densenet201": head,
        "corun_reset_mode": reset_only,
        "corun_without_drain_wait": no_drain_wait,
        "solo_back_to_back_ms": {"p50": pct(lat_us, 50), "p99": pct(lat_us, 99),
                                 "mean_device": round(float(dev_us.mean()) / 1e3, 4)},
        "model_tflops": round(g.flops / float(dev_us.mean()) / 1e6, 3),
        "conv_tflops_all_layers": round(conv_flops / conv_us / 1e6, 3),
        "best_layer": {"kernel": names_k[best_i], "attrs": g.kernels[best_i]["attrs"][:12],
                       "tflops": round(float(flops[best_i] / kus[best_i] / 1e6), 2)},
        "sum_kernel_us": round(float(kus.sum()), 1),
        "sum_kernel_us_back_to_back": round(float(kus_b2b.sum()), 1),
        "sum_kernel_us_in_model_unscaled": round(float((kus_b2b + extra).sum()), 1),
        "in_model_correction_factor": round(alpha, 3),
        "roofline": {
            "bound": "mfma",
            "kernel": dom,
            "achieved": round(dom_tflops, 3),
            "peak": FP32_MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(dom_tflops / FP32_MFMA_PEAK_TFLOPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_note,
            "launches_per_inference": dom_e["launches"],
            "avg_launch_us": round(dom_e["us"] / dom_e["launches"], 3),
            "avg_launch_us_back_to_back": round(float(sum(kus_b2b[i] for i, nm in enumerate(names_k) if nm == dom))
                                                / dom_e["launches"], 3),
            "avg_launch_us_what": "launch inside a pass of the model (operands as a real inference finds them); "
                                  "back_to_back: the kernel repeated alone, operands cached",
            "avg_launch_gflop": round(dom_e["flops"] / dom_e["launches"] / 1e9, 4),
        },
        "per_kernel": {k: {"launches": v["launches"], "avg_us": round(v["us"] / v["launches"], 3),
                           "tflops": round(v["flops"] / v["us"] / 1e6, 3),
                           "frac_mfma_peak": round(v["flops"] / v["us"] / 1e6 / FP32_MFMA_PEAK_TFLOPS, 4),
                           "gbs": round(v["bytes"] / v["us"] / 1e3, 1),
                           "frac_hbm_peak": round(v["bytes"] / v["us"] / 1e3 / HBM_PEAK_GBS, 4)}
                       for k, v in sorted(by.items())},
        "conv_shapes": conv_shapes,
        "timed_region_wall_s": round(wall_s, 3),
    }
    # the classifier's logits (input of the last kernel, the softmax): a saturated softmax
    # output would agree with anything
    logits_idx = g.kernels[-1]["args"][0]
    got = exe.get_data(logits_idx, g.storage[logits_idx]["size"])
    exe.close()
    out["steady_state_conv"] = steady_state_conv(tmp.name, max(args.kernel_iters, 5))
    if 4 in configs:
        k = max(args.steps // 2, 50)
        out["corun_dkp_mobilenetv2"] = {
            "reef": corun(models, "resnet152", "mobilenetv2", 1, B.MODE_REEF, k, 20),
            "reset": corun(models, "resnet152", "mobilenetv2", 1, B.MODE_RESET, k, 20, solo=False)}
    if 5 in configs:
        k = max(args.steps // 2, 50)
        out["corun_inceptionv3_2x_bert"] = corun(models, "inceptionv3", "bert_base", 2, B.MODE_REEF, k, 20)
    if 6 in configs:
        # dynamic kernel padding where it can matter: real-time requests every 2 ms on average
        # keep the device busy about three quarters of the time
        k = max(args.steps, 200)
        out["corun_dkp_high_rt_load"] = {
            "rt_mean_interval_us": 2000.0,
            "reef_slack50": corun(models, "resnet152", "mobilenetv2", 1, B.MODE_REEF, k, 20, interval_us=2000.0),
            "reef_slack100": corun(models, "resnet152", "mobilenetv2", 1, B.MODE_REEF, k, 20, solo=False,
                                   dkp_slack=100, interval_us=2000.0),
            "reset": corun(models, "resnet152", "mobilenetv2", 1, B.MODE_RESET, k, 20, solo=False,
                           interval_us=2000.0)}
    if 8 in configs and head is not None:
        # the headline pair with 16 best-effort queues instead of 4: the launch windows of the 16
        # streams share the pool of feeder threads (four host threads, not sixteen)
        k = max(args.steps // 2, 50)
        out["corun_16_be_queues"] = corun(models, "resnet152", "densenet201", 16, B.MODE_REEF, k, 20, solo=False)
    if not args.solo_only:
        # the bandwidth-bound families are where they matter: MobileNetV2 (depthwise) and BERT-base
        for extra in ("mobilenetv2", "bert_base"):
            if extra in models:
                out["solo_kernels_" + extra] = solo_kernel_table(models, extra, max(args.kernel_iters // 2, 5))
    if 7 in configs and head is not None:
        # the reference's evaluation baselines (scheduler.h:22-28) on the headline workload
        k = max(args.steps // 4, 50)
        runs = {"REEF": head, "Reset": reset_only}
        for label, m in (("WaitPreempt", B.MODE_WAITPREEMPT), ("NoPreempt", B.MODE_NOPREEMPT),
                         ("MultiStream", B.MODE_MULTISTREAM)):
            runs[label] = corun(models, "resnet152", "densenet201", 4, m, k, 20, solo=False)
        out["schedule_modes"] = {
            label: {"rt_ms_p50": r["loaded"]["rt_ms"]["p50"], "rt_ms_p99": r["loaded"]["rt_ms"]["p99"],
                    "rt_exec_ms_p50": r["loaded"]["rt_exec_ms"]["p50"],
                    "rt_exec_ms_p99": r["loaded"]["rt_exec_ms"]["p99"],
                    "be_inferences_per_s": r["loaded"]["be_inferences_per_s"],
                    "switch_us_mean": r["preempt_us"]["mean"], "switch_us_p99": r["preempt_us"]["p99"],
                    "rt_requests": r["preempt_us"]["n"],
                    "outputs_bit_identical_to_solo": r.get("outputs_bit_identical_to_solo")}
            for label, r in runs.items()}
    if not args.no_cpu:
        # two stand-ins for "the model compiled by TVM for llvm" (TVM is not installed): the CPU
        # oracle and the same network as torch.nn.functional calls.  The stated baseline is the
        # faster of the two; the other is kept beside it.
        cb, orc = cpu_baseline(d, g.name, x)
        ref = np.asarray(orc.storage[logits_idx], np.float64)
        out["parity_logits_max_rel_err_vs_oracle"] = float(np.abs(got - ref).max() / np.abs(ref).max())
        tc = torch_cpu_baseline(g, x)
        if tc is not None:
            out["parity_logits_max_rel_err_vs_torch_cpu"] = float(np.abs(got - tc[1]).max() / np.abs(tc[1]).max())
        if tc is not None and tc[0]["value"] < cb["value"]:
            out["cpu_baseline"] = {"value": tc[0]["value"], "unit": "ms", "cores": tc[0]["threads"], "kind": "port",
                                   "sample": tc[0]["sample"] + "; stands in for the TVM-llvm build of the model "
                                             "(TVM is not installed)",
                                   "oracle": {"value": cb["value"], "unit": "ms", "cores": cb["cores"],
                                              "sample": cb["sample"]}}
        else:
            out["cpu_baseline"] = cb
            if tc is not None:
                out["cpu_baseline"]["torch_cpu"] = tc[0]
    identical = [leg.get("outputs_bit_identical_to_solo") for leg in corun_legs(out)]
    identical += [m.get("outputs_bit_identical_to_solo") for m in out.get("schedule_modes", {}).values()]
    out["corun_outputs_bit_identical"] = all(identical) if identical else None
    line = compact_line(out)
    detail_path = args.detail_out or os.path.join(ROOT, "gpurun_out", "bench_detail.json")
    try:
        os.makedirs(os.path.dirname(os.path.abspath(detail_path)), exist_ok=True)
        with open(detail_path, "w") as f:
            json.dump(out, f)
        print("bench: full tables and every co-location leg in %s" % detail_path, file=sys.stderr)
    except OSError as e:
        print("bench: could not write %s (%s)" % (detail_path, e), file=sys.stderr)
    sys.stdout.flush()
    print(line)
    if out["corun_outputs_bit_identical"] is False:
        sys.exit(1)


if __name__ == "__main__":
    main()
