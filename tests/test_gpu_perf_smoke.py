"""Timing helpers run and return sane numbers (not a benchmark)."""
import pytest

from reef_amd import binding as B
from reef_amd.modelgen import nets
from tests.helpers import write_model

pytestmark = pytest.mark.gpu


def test_time_kernel_and_model(tmp_path):
    g = nets.resnet(18, image=(3, 64, 64), classes=10, name="tiny")
    d = write_model(g, tmp_path)
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    us = exe.time_kernel(1, warmup=2, iters=10)
    assert 0.5 < us < 5000
    lat, dev = exe.time_model(warmup=2, iters=5)
    assert (lat > 0).all() and (dev > 0).all()
    # one launch between two events: inside a pass of the model and directly after itself
    in_model, after_itself = exe.time_kernel_in_model(1, samples=3)
    assert 0.5 < after_itself < 5000 and 0.5 < in_model < 5000
    # the padding flavour on a few CUs, once with the caches overwritten first
    info = exe.kernel_info(1)
    cus = 8 if info["block_num"] >= 8 else 0
    warm = exe.time_kernel_dkp_single(1, 1, min(info["block_num"], 8), cus, None, 3)
    evict = B.DeviceBuffer(64 << 20)
    cold = exe.time_kernel_dkp_single(1, 1, min(info["block_num"], 8), cus, evict, 3)
    evict.free()
    assert 0.5 < warm < 5000 and 0.5 < cold < 5000
    exe.close()


def test_measured_profile_has_both_resolutions(tmp_path):
    """<model>.profile.json as the reference reads it (integer microseconds, model.cpp:57-80)
    plus the nanosecond keys the padding decision uses here."""
    import json
    import os
    from reef_amd import profiler
    g = nets.resnet(18, image=(3, 32, 32), classes=10, name="tinyp")
    d = write_model(g, tmp_path)
    prof = profiler.write_profile(d, g.name, iters=3, warmup=1)
    back = json.load(open(os.path.join(d, g.name + ".profile.json")))
    assert back == prof and prof["model_latency"] > 0
    assert len(prof["kernel_latency"]) == len(g.kernels)
    for v in prof["kernel_latency"].values():
        assert v["total_latency"] >= 1 and all(x >= 1 for x in v["latency"])
        assert v["total_latency_ns"] >= 500 and len(v["latency_ns"]) == len(v["latency"]) >= 1
        assert abs(v["total_latency"] * 1000 - v["total_latency_ns"]) < 1000
