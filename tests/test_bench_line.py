"""bench.py prints ONE compact JSON line on standard output (the full result goes to a file).
The line is built from the full result by bench.compact_line; here from a canned result that is
larger than any real one (every co-location leg with its prose, long tables), so that the line
stays small and complete whatever the run produced."""
import json

import bench


def leg(n_be=4):
    summary = {"rt_ms": {"p50": 1.284, "p99": 2.306, "mean": 1.41, "max": 2.9},
               "rt_exec_ms": {"p50": 1.265, "p99": 1.286}, "rt_queue_ms": {"p50": 0.018, "p99": 1.0},
               "be_inferences_per_s": 1449.0, "be_completed": [500] * n_be, "be_preempted": [90] * n_be,
               "be_padded": [12] * n_be, "span_s": 8.1}
    return {"mode": "REEF (reset-based preemption + dynamic kernel padding)", "rt_model": "resnet152",
            "be_model": "densenet201", "be_clients": n_be, "solo": summary, "loaded": summary,
            "be_only_inferences_per_s": 1551.0,
            "preempt_us": {"n": 400, "mean": 16.5, "p50": 16.0, "p99": 26.0, "max": 30, "what": "x" * 600,
                           "device": {"n": 400, "mean": 19.9, "p50": 19.8, "p99": 34.0, "max": 40.5,
                                      "clock_sync_err_us": 1.1, "late_launch_samples": 24,
                                      "without_late_launches": {"n": 376, "mean": 19.0, "p99": 33.0, "max": 40.0},
                                      "what": "y" * 700}},
            "preempt_phase_ns": {"flag_ns": 300, "drop_ns": 1000, "drain_ns": 14900},
            "padded_kernels": 1772, "kernel_select_ns": 61, "outputs_bit_identical_to_solo": True}


def canned():
    head = leg()
    return {
        "metric": "ResNet-152 RT p99 latency w/ 4 BE clients", "value": 2.306, "unit": "ms", "n_gpus": 1,
        "steps": 400, "warmup": 40, "ms_per_step": 1.41, "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "RT ResNet-152 (batch 1, fp32 NCHW 3x224x224, Poisson arrivals mean 20 ms, seed "
                               "0x5EEF) + 4 BE clients looping DenseNet-201 (growth 32, batch 1, 224x224); seeded "
                               "He-normal weights; REEF mode",
                   "rt_kernels_per_inference": 156, "rt_gflop_per_inference": 22.564},
        "rt_p99_vs_solo": 0.983, "rt_p50_vs_solo": 0.98, "rt_exec_p99_vs_solo": 1.001,
        "preempt_us": head["preempt_us"], "corun_resnet152_4x_densenet201": head, "corun_reset_mode": leg(),
        "corun_without_drain_wait": leg(),
        "solo_back_to_back_ms": {"p50": 1.27, "p99": 1.29, "mean_device": 1.248}, "model_tflops": 18.1,
        "conv_tflops_all_layers": 18.4,
        "roofline": {"bound": "mfma", "kernel": "reef_conv2d_d1_16x32k4", "achieved": 14.6, "peak": 157.3,
                     "unit": "TFLOP/s", "frac": 0.0928, "traffic": 7590000, "traffic_source": "z" * 120,
                     "launches_per_inference": 83, "avg_launch_us": 7.06, "avg_launch_us_back_to_back": 6.6,
                     "avg_launch_us_what": "w" * 200, "avg_launch_gflop": 0.1028},
        "per_kernel": {"reef_kernel_symbol_%d" % i: {"launches": 3, "avg_us": 7.1, "tflops": 14.0,
                                                     "frac_mfma_peak": 0.09, "gbs": 400.0, "frac_hbm_peak": 0.05}
                       for i in range(40)},
        "conv_shapes": [{"cin_h_w": [256, 14, 14], "cout_ho_wo": [1024, 14, 14], "k": [1, 1], "stride": [1, 1],
                         "kernel": "reef_conv2d_d1_16x32k4", "launches": 36, "avg_us": 7.0, "tflops": 14.6,
                         "frac_mfma_peak": 0.093}] * 60,
        "corun_dkp_mobilenetv2": {"reef": leg(1), "reset": leg(1)},
        "corun_inceptionv3_2x_bert": leg(2),
        "corun_dkp_high_rt_load": {"rt_mean_interval_us": 2000.0, "reef_slack50": leg(1), "reef_slack100": leg(1),
                                   "reset": leg(1)},
        "solo_kernels_mobilenetv2": {"model_device_ms": 0.26, "kernels": {"k%d" % i: {"avg_us": 4.0} for i in range(12)}},
        "solo_kernels_bert_base": {"model_device_ms": 0.98, "kernels": {"k%d" % i: {"avg_us": 4.0} for i in range(12)}},
        "schedule_modes": {m: {"rt_ms_p50": 1.3, "outputs_bit_identical_to_solo": True}
                           for m in ("REEF", "Reset", "WaitPreempt", "NoPreempt", "MultiStream")},
        "cpu_baseline": {"value": 26.1, "unit": "ms", "cores": 16, "kind": "port", "sample": "s" * 250,
                         "oracle": {"value": 181.0, "unit": "ms", "cores": 16, "sample": "t" * 250}},
        "parity_logits_max_rel_err_vs_oracle": 1.1e-6, "corun_outputs_bit_identical": True,
    }


def test_compact_line_is_small_parses_and_carries_the_contract():
    detail = canned()
    assert len(json.dumps(detail)) > 20000            # the full result is what no longer fits a line
    line = bench.compact_line(detail)
    assert "\n" not in line and len(line) < 8192 and len(line) <= bench.COMPACT_LIMIT
    got = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in got, key
    assert got["value"] == 2.306 and got["config"]["workload"].startswith("RT ResNet-152")
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in got["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in got["cpu_baseline"], key
    assert got["cpu_baseline"]["value"] == 26.1 and got["cpu_baseline"]["oracle_ms"] == 181.0
    # what to read beside a p99 over few requests
    assert got["rt_p50_ms"] == 1.284 and got["rt_exec_p99_ms"] == 1.286 and got["rt_p99_vs_solo"] == 0.983
    assert got["preempt_device_us"]["p99"] == 34.0 and got["preempt_host_us"]["max"] == 30
    assert got["corun_outputs_bit_identical"] is True
    assert got["other_configs"]["cfg4_rt_resnet152_be_mobilenetv2"]["be_inferences_per_s_reset_mode"] == 1449.0
    # the tables and the legs themselves are not on the line
    assert "per_kernel" not in got and "conv_shapes" not in got and "schedule_modes" not in got


def test_compact_line_of_a_solo_only_run():
    detail = canned()
    for key in list(detail):
        if key.startswith("corun_") or key.startswith("solo_kernels_") or key == "schedule_modes":
            del detail[key]
    detail.pop("cpu_baseline")
    detail["corun_outputs_bit_identical"] = None
    got = json.loads(bench.compact_line(detail))
    assert got["roofline"]["frac"] == 0.0928 and got["rt_p50_ms"] is None and "cpu_baseline" not in got


def test_every_leg_of_the_full_result_is_found_for_the_bit_identity_summary():
    detail = canned()
    assert len(bench.corun_legs(detail)) == 9
    detail["corun_dkp_high_rt_load"]["reset"]["outputs_bit_identical_to_solo"] = False
    assert not all(leg_["outputs_bit_identical_to_solo"] for leg_ in bench.corun_legs(detail))
