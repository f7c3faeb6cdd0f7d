"""Executors and scheduler on the recording backend (no GPU): argument binding,
launch geometry per flavour, error codes, preemption rollback and idempotence,
dynamic kernel padding bookkeeping.  The backend executes every completed
"kernel" with the CPU oracle, so outputs are real."""
import ctypes
import json
import os
import time

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd.modelgen import nets
from tests.fakehal import FakeHal
from tests.helpers import write_model

THREE = np.full(8192, 3.0, np.float32)


@pytest.fixture()
def fake():
    f = FakeHal().install()
    yield f
    f.remove()


@pytest.fixture(scope="module")
def small_dirs(tmp_path_factory):
    out = {}
    for g in (nets.mocked_kernel(), nets.resnet(18, image=(3, 32, 32), classes=16, name="tiny18")):
        out[g.name] = (g, write_model(g, tmp_path_factory.mktemp(g.name)))
    return out


def oracle_output(g, d, x):
    model = json.load(open(os.path.join(d, g.name + ".json")))
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    orc.set_input("data", x)
    return orc.run().copy()


@pytest.mark.parametrize("kind,pre", [(B.BASE, False), (B.TRANS, False), (B.HYBRID, False), (B.HYBRID, True)])
def test_mocked_model_all_flavours(fake, small_dirs, kind, pre):
    g, d = small_dirs["mocked_kernel"]
    exe = B.Executor.from_dir(d, g.name, kind)
    for n in "abc":
        exe.set_input_checked(n, THREE)
    exe.execute_preemptable() if pre else exe.execute()
    np.testing.assert_array_equal(exe.get_output(), np.full(8192, 18.0, np.float32))
    log = fake.log()
    assert [e[0] for e in log] == ["add", "multiply"]
    if kind == B.BASE or pre:
        assert all(e[2] == 64 and e[3] == 128 for e in log)      # grid/block from the JSON
    else:
        assert all(e[2] == 256 * 1 and e[3] == 128 for e in log)  # num_cus * min_occupancy, flat block


@pytest.mark.parametrize("kind,pre", [(B.BASE, False), (B.TRANS, False), (B.HYBRID, True)])
def test_resnet_binding_matches_graph_oracle(fake, small_dirs, kind, pre):
    g, d = small_dirs["tiny18"]
    x = nets.image_input("t", (3, 32, 32))
    exe = B.Executor.from_dir(d, g.name, kind)
    exe.set_input_checked("data", x)
    exe.execute_preemptable() if pre else exe.execute()
    np.testing.assert_array_equal(exe.get_output(), oracle_output(g, d, x))
    assert exe.num_kernels() == len(g.kernels) == len(fake.log())
    if pre:
        assert exe.read_task_slots() == [k["launch_params"][0] for k in g.kernels]


@pytest.mark.parametrize("kind", [B.BASE, B.TRANS, B.HYBRID])
def test_whole_model_runs_replay_one_recorded_submission(fake, small_dirs, kind):
    """With graph launch on, execute() records the model's launch sequence on first use and
    replays it as one submission afterwards; off means one launch call per kernel.  Both ways
    run the same kernels with the same arguments."""
    g, d = small_dirs["tiny18"]
    x = nets.image_input("t", (3, 32, 32))
    want = oracle_output(g, d, x)
    exe = B.Executor.from_dir(d, g.name, kind)
    exe.set_graph_launch(True)
    exe.set_input_checked("data", x)
    n = exe.num_kernels()
    for run in range(3):
        exe.execute()
        np.testing.assert_array_equal(exe.get_output(), want)
        assert fake.lib.fake_hal_graph_launches() == run + 1
        assert fake.lib.fake_hal_launches() == n * (run + 1)
    log_graph = fake.log()[-n:]
    exe.set_graph_launch(False)
    exe.execute()
    np.testing.assert_array_equal(exe.get_output(), want)
    assert fake.lib.fake_hal_graph_launches() == 3
    assert fake.log()[-n:] == log_graph
    # partial runs never go through the recording
    exe.set_graph_launch(True)
    exe.execute_to(n - 1)
    assert fake.lib.fake_hal_graph_launches() == 3


def test_executor_error_codes(fake, small_dirs, tmp_path):
    g, d = small_dirs["mocked_kernel"]
    exe = B.Executor.from_dir(d, g.name, B.BASE)
    assert exe.set_input("nope", THREE) == 2            # NotFound
    assert exe.set_input("a", THREE[:100]) == 3         # OutOfRange: shorter than the storage
    assert exe.get_data_size("output") == 8192 * 4
    with pytest.raises(B.ReefError) as ei:
        exe.get_output(10)                              # buffer too small -> Fail
    assert ei.value.status == 1
    with pytest.raises(B.ReefError) as ei:
        exe.execute_to(99)
    assert ei.value.status == 3
    with pytest.raises(B.ReefError) as ei:
        exe.execute_kernel(2)
    assert ei.value.status == 3
    with pytest.raises(B.ReefError) as ei:               # missing graph file
        B.Executor(B.BASE).load(str(tmp_path / "none.json"), os.path.join(d, g.name + ".raw.co"))
    assert ei.value.status == 2
    with pytest.raises(B.ReefError) as ei:               # missing code object
        B.Executor(B.BASE).load(os.path.join(d, g.name + ".json"), str(tmp_path / "none.co"))
    assert ei.value.status == 1
    fake.set_missing("multiply")
    with pytest.raises(B.ReefError) as ei:               # symbol not in the code object
        B.Executor.from_dir(d, g.name, B.BASE)
    assert ei.value.status == 1


def test_trans_needs_proxy_kernel(fake, small_dirs):
    g, d = small_dirs["mocked_kernel"]
    fake.set_missing("merge_framework_3")
    with pytest.raises(B.ReefError):
        B.Executor.from_dir(d, g.name, B.TRANS)


def test_min_occupancy_and_kernel_info(fake, small_dirs):
    g, d = small_dirs["tiny18"]
    fake.set_kernel_resource("reef_eltwise", lds=0, vgprs=128, sgprs=32)
    exe = B.Executor.from_dir(d, g.name, B.TRANS)
    for i, k in enumerate(g.kernels):
        info = exe.kernel_info(i)
        blocks = k["launch_params"][0]
        assert info["block_num"] == blocks
        occ = B.lib().reef_gpuconfig_calculate_occupancy(info["lds"], info["vgprs"], info["sgprs"], 0, 256)
        assert info["min_occupancy"] == max(1, min(-(-blocks // 256), occ))


def run_scheduler_until(s, tid, timeout=20.0):
    t0 = time.time()
    while time.time() - t0 < timeout:
        if s.task_info(tid)["state"] == B.STATE_FINISH:
            return True
        time.sleep(0.001)
    return False


@pytest.mark.parametrize("qtype", [B.QUEUE_RT, B.QUEUE_BE])
@pytest.mark.parametrize("mode", [B.MODE_REEF, B.MODE_RESET, B.MODE_WAITPREEMPT, B.MODE_NOPREEMPT])
def test_scheduler_single_task(fake, small_dirs, qtype, mode):
    g, d = small_dirs["mocked_kernel"]
    s = B.Scheduler(mode)
    assert s.mode() == mode
    s.run()
    mid = s.load_model(d, g.name)
    qid = s.create_queue(qtype)
    assert s.bind_model_queue(qid, mid) == 0
    for n in "abc":
        assert s.set_input(mid, THREE, n) == 0
    tid = s.new_task(mid)
    assert s.wait_task(tid) == 0
    np.testing.assert_array_equal(s.get_output(mid, 8192), np.full(8192, 18.0, np.float32))
    assert s.wait_task(tid + 100) == 2       # NotFound
    assert s.new_task_status(mid + 5) == 3   # OutOfRange
    s.shutdown()


def test_scheduler_preempt_rollback_and_idempotence(fake, small_dirs):
    """A best-effort task is interrupted by a real-time task: queued launches are
    dropped, in-flight kernels see the flag and skip, the task restarts from the
    rolled-back kernel, and its output equals the uninterrupted result."""
    gb, db = small_dirs["tiny18"]
    gm, dm = small_dirs["mocked_kernel"]
    x = nets.image_input("t", (3, 32, 32))
    ref = oracle_output(gb, db, x)
    fake.lib.fake_hal_set_auto_progress(1)
    s = B.Scheduler(B.MODE_RESET)
    s.run()
    be_mid = s.load_model(db, gb.name)
    rt_mid = s.load_model(dm, gm.name)
    be_q, rt_q = s.create_queue(B.QUEUE_BE), s.create_queue(B.QUEUE_RT)
    s.bind_model_queue(be_q, be_mid)
    s.bind_model_queue(rt_q, rt_mid)
    s.set_input(be_mid, x, "data")
    for n in "abc":
        s.set_input(rt_mid, THREE, n)
    be_tid = s.new_task(be_mid)
    t0 = time.time()
    while fake.lib.fake_hal_completed() < 3 and time.time() - t0 < 10:
        time.sleep(0.0002)
    rt_tid = s.new_task(rt_mid)
    assert s.wait_task(rt_tid) == 0 and s.wait_task(be_tid) == 0
    np.testing.assert_array_equal(s.get_output(rt_mid, 8192), np.full(8192, 18.0, np.float32))
    np.testing.assert_array_equal(s.get_output(be_mid, 16), ref)
    be, rt = s.task_info(be_tid), s.task_info(rt_tid)
    if be["preempted"]:
        assert fake.lib.fake_hal_dropped() > 0 or fake.skipped > 0
        assert rt["start"] >= be["start"] and be["end"] >= rt["end"]
        assert s.preempt_times() == 1
        # more launches than kernels: the tail was launched twice
        assert fake.lib.fake_hal_launches() > len(gb.kernels) + 2
    s.shutdown()
    assert be["preempted"], "the real-time task arrived after the best-effort task had finished"


def test_scheduler_dkp_pads_to_completion(fake, small_dirs):
    """scheduler.mocked_kernel of the reference (src/reef/test/test.cpp:491-536):
    best-effort mocked model + real-time network queued before run()."""
    gr, dr = small_dirs["tiny18"]
    gm, dm = small_dirs["mocked_kernel"]
    x = nets.image_input("t", (3, 32, 32))
    ref = oracle_output(gr, dr, x)
    # profile: make every real-time kernel long enough to host the mocked kernels
    prof = json.load(open(os.path.join(dr, gr.name + ".profile.json")))
    for v in prof["kernel_latency"].values():
        v["total_latency"] = 100
    json.dump(prof, open(os.path.join(dr, gr.name + ".profile.json"), "w"))
    s = B.Scheduler(B.MODE_REEF)
    rt_mid = s.load_model(dr, gr.name)
    be_mid = s.load_model(dm, gm.name)
    rt_q, be_q = s.create_queue(B.QUEUE_RT), s.create_queue(B.QUEUE_BE)
    s.bind_model_queue(rt_q, rt_mid)
    s.bind_model_queue(be_q, be_mid)
    s.set_input(rt_mid, x, "data")
    for n in "abc":
        s.set_input(be_mid, THREE, n)
    be_tid = s.new_task(be_mid)
    rt_tid = s.new_task(rt_mid)
    s.run()
    assert s.wait_task(be_tid) == 0 and s.wait_task(rt_tid) == 0
    np.testing.assert_array_equal(s.get_output(rt_mid, 16), ref)
    np.testing.assert_array_equal(s.get_output(be_mid, 8192), np.full(8192, 18.0, np.float32))
    be = s.task_info(be_tid)
    assert be["padded"] and be["padded_to_complete"] and not be["preempted"]
    merged = [e for e in fake.log() if e[0].startswith("merge_framework_")]
    assert len(merged) == s.padded_kernels() >= 2
    assert s.avg_kernel_sel_latency() >= 0
    s.shutdown()


def test_load_generator_counts_and_outputs(fake, small_dirs):
    """The in-process clients (request loops of src/example/rpc_client_cont.cpp:20-36): one open-loop
    real-time client with exponential gaps, two closed-loop best-effort clients.  Every recorded
    request has submit <= start <= end, best-effort clients complete work, and the models'
    outputs stay those of the oracle whatever got preempted on the way."""
    gb, db = small_dirs["tiny18"]
    gm, dm = small_dirs["mocked_kernel"]
    x = nets.image_input("t", (3, 32, 32))
    ref = oracle_output(gb, db, x)
    fake.lib.fake_hal_set_auto_progress(4)
    s = B.Scheduler(B.MODE_RESET)
    s.set_wait_sync(True)
    rt_mid = s.load_model(dm, gm.name)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt_mid)
    for n in "abc":
        s.set_input(rt_mid, THREE, n)
    bes = []
    for _ in range(2):
        m = s.load_model(db, gb.name)
        s.bind_model_queue(s.create_queue(B.QUEUE_BE), m)
        s.set_input(m, x, "data")
        bes.append(m)
    s.run()
    r = s.run_load(rt_mid, bes, requests=24, warmup=3, mean_interval_us=25000.0, seed=7)
    assert len(r["rt_latency_us"]) == 24
    assert (r["rt_queue_us"] >= 0).all() and (r["rt_exec_us"] >= 0).all()
    np.testing.assert_allclose(r["rt_latency_us"], r["rt_queue_us"] + r["rt_exec_us"], atol=1e-3)
    assert r["span_s"] > 24 * 0.005
    assert r["be_completed"].sum() > 0 and (r["be_preempted"] <= r["be_completed"]).all()
    assert s.preempt_times() > 0
    ph = s.preempt_phases()
    assert ph["flag_ns"] >= 0 and ph["drop_ns"] >= 0 and ph["drain_ns"] >= 0
    np.testing.assert_array_equal(s.get_output(rt_mid, 8192), np.full(8192, 18.0, np.float32))
    for m in bes:
        np.testing.assert_array_equal(s.get_output(m, 16), ref)
    # best-effort only
    r2 = s.run_load(rt_mid, bes, requests=0, be_only_ms=1500)
    assert len(r2["rt_latency_us"]) == 0 and r2["be_completed"].sum() > 0
    s.shutdown()


def test_dkp_slack_limits_padding(fake):
    """set_dkp_slack_percent: best-effort work must fit the given share of the real-time kernel's
    latency (100 = be.latency <= rt.latency, src/reef/server/scheduler.cpp:565-572)."""
    L = B.lib()
    rt = (ctypes.c_int * 7)(64, 1, 256, 64, 32, 0, 100)       # 64 blocks, latency 100 us
    be = (ctypes.c_int * 7)(512, 1, 256, 64, 32, 0, 0)
    lat = (ctypes.c_int * 4)(60, 70, 90, 120)                 # per occupancy 1..4
    proxy = (ctypes.c_int * 3)(64, 32, 0)
    out = (ctypes.c_int * 8)()
    got = {}
    for slack in (100, 80, 65, 50):
        assert L.reef_dkp_decide_slack(rt, be, lat, 4, 0, proxy, 256, 8, slack, out) == 0
        got[slack] = list(out)
    assert got[100][0] == 1 and got[100][2] == 3     # occupancy 3: 90 <= 100
    assert got[80][0] == 1 and got[80][2] == 2       # 70 <= 80
    assert got[65][0] == 1 and got[65][2] == 1       # 60 <= 65
    assert got[50][0] == 0                           # nothing fits half the latency
    # be_blocks = (256 - partition) * (budget / be_latency) * be_occ
    part = got[100][4]
    assert got[100][5] == min(512, (256 - part) * (100 // 90) * 3)
    assert got[65][5] == min(512, (256 - part) * (65 // 60) * 1)


def test_finished_best_effort_task_is_never_run_or_counted_twice(fake, small_dirs):
    """A real-time task that arrives in the instant a best-effort task completes must not find
    the completed task at the head of its queue: it would be padded into real-time kernels a
    second time and counted out of the pending tasks twice.  Many short best-effort tasks with
    real-time arrivals at random moments; afterwards every task is finished exactly once (the
    pending count is back at zero, not below) and outputs are intact."""
    gm, dm = small_dirs["mocked_kernel"]
    gr, dr = small_dirs["tiny18"]
    x = nets.image_input("t", (3, 32, 32))
    ref = oracle_output(gr, dr, x)
    prof = json.load(open(os.path.join(dr, gr.name + ".profile.json")))
    for v in prof["kernel_latency"].values():
        v["total_latency"] = 100      # every real-time kernel can host the mocked kernels
    json.dump(prof, open(os.path.join(dr, gr.name + ".profile.json"), "w"))
    fake.lib.fake_hal_set_auto_progress(2)
    s = B.Scheduler(B.MODE_REEF)
    rt_mid = s.load_model(dr, gr.name)
    be_mid = s.load_model(dm, gm.name)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt_mid)
    s.bind_model_queue(s.create_queue(B.QUEUE_BE), be_mid)
    s.set_input(rt_mid, x, "data")
    for n in "abc":
        s.set_input(be_mid, THREE, n)
    s.run()
    rng = np.random.default_rng(5)
    for rep in range(60):
        be_tid = s.new_task(be_mid)
        time.sleep(float(rng.uniform(0, 0.002)))
        rt_tid = s.new_task(rt_mid)
        be2 = s.new_task(be_mid)
        for t in (be_tid, rt_tid, be2):
            assert run_scheduler_until(s, t), "task %d never finished (rep %d)" % (t, rep)
        np.testing.assert_array_equal(s.get_output(be_mid, 8192), np.full(8192, 18.0, np.float32))
    t0 = time.time()
    while s.pending_tasks() != 0 and time.time() - t0 < 2:
        time.sleep(0.001)
    assert s.pending_tasks() == 0
    np.testing.assert_array_equal(s.get_output(rt_mid, 16), ref)
    s.shutdown()


def test_wait_preempt_second_run_restarts_at_the_interrupted_kernel(fake, small_dirs):
    """Wait-based preemption (src/reef/server/scheduler.cpp:348-372) finds the restart point from
    per-kernel completion counters.  The counters of a model survive a run, so a second,
    interrupted run must not mistake the first run's counts for its own: its output still
    equals the uninterrupted result and the interrupted tail is launched again."""
    gb, db = small_dirs["tiny18"]
    gm, dm = small_dirs["mocked_kernel"]
    x = nets.image_input("t", (3, 32, 32))
    ref = oracle_output(gb, db, x)
    fake.lib.fake_hal_set_auto_progress(1)
    s = B.Scheduler(B.MODE_WAITPREEMPT)
    s.run()
    be_mid = s.load_model(db, gb.name)
    rt_mid = s.load_model(dm, gm.name)
    s.bind_model_queue(s.create_queue(B.QUEUE_BE), be_mid)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt_mid)
    s.set_input(be_mid, x, "data")
    for n in "abc":
        s.set_input(rt_mid, THREE, n)
    # a clean first run leaves every counter at its kernel's workgroup count
    assert s.wait_task(s.new_task(be_mid)) == 0
    np.testing.assert_array_equal(s.get_output(be_mid, 16), ref)
    n_kernels = len(gb.kernels)
    preempted = 0
    for rep in range(6):
        # a different input each time, so a skipped kernel would leave stale activations behind
        xi = (x * (1.0 + 0.25 * rep)).astype(np.float32)
        want = oracle_output(gb, db, xi)
        s.set_input(be_mid, xi, "data")
        done0 = fake.lib.fake_hal_completed()
        launches0 = fake.lib.fake_hal_launches()
        be_tid = s.new_task(be_mid)
        t0 = time.time()
        while fake.lib.fake_hal_completed() < done0 + 3 + rep and time.time() - t0 < 10:
            time.sleep(0.0002)
        rt_tid = s.new_task(rt_mid)
        assert s.wait_task(rt_tid) == 0 and s.wait_task(be_tid) == 0
        np.testing.assert_array_equal(s.get_output(be_mid, 16), want)
        if s.task_info(be_tid)["preempted"]:
            preempted += 1
            # everything the model has was launched at least once in this run
            assert fake.lib.fake_hal_launches() - launches0 >= n_kernels + 2
    assert preempted > 0, "no run was interrupted"
    s.shutdown()


@pytest.mark.parametrize("mode", [B.MODE_NOPREEMPT, B.MODE_MULTISTREAM, B.MODE_WAITPREEMPT])
def test_real_time_arrival_during_a_best_effort_run_in_the_baseline_modes(fake, small_dirs, mode):
    """The evaluation baselines of the reference (src/reef/server/scheduler.h:22-28) under contention:
    a real-time task arrives while a best-effort run is on the device.
      NoPreempt    waits for everything launched, then runs the real-time task (scheduler.cpp:381-392);
      MultiStream  switches nothing: the real-time kernels go to their own stream beside the
                   best-effort ones (scheduler.cpp:402-403);
      WaitPreempt  raises the flag, waits, restarts at the first incomplete kernel (scheduler.cpp:348-372).
    Whatever the interleaving, both outputs are those of an undisturbed run, over several runs."""
    gb, db = small_dirs["tiny18"]
    gm, dm = small_dirs["mocked_kernel"]
    x = nets.image_input("t", (3, 32, 32))
    fake.lib.fake_hal_set_auto_progress(1)
    s = B.Scheduler(mode)
    s.run()
    be_mid = s.load_model(db, gb.name)
    rt_mid = s.load_model(dm, gm.name)
    s.bind_model_queue(s.create_queue(B.QUEUE_BE), be_mid)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt_mid)
    for n in "abc":
        s.set_input(rt_mid, THREE, n)
    overlapped = 0
    for rep in range(5):
        xi = (x * (1.0 + 0.5 * rep)).astype(np.float32)
        want = oracle_output(gb, db, xi)
        s.set_input(be_mid, xi, "data")
        done0 = fake.lib.fake_hal_completed()
        be_tid = s.new_task(be_mid)
        t0 = time.time()
        while fake.lib.fake_hal_completed() < done0 + 2 + rep and time.time() - t0 < 10:
            time.sleep(0.0002)
        rt_tid = s.new_task(rt_mid)
        assert s.wait_task(rt_tid) == 0 and s.wait_task(be_tid) == 0
        np.testing.assert_array_equal(s.get_output(rt_mid, 8192), np.full(8192, 18.0, np.float32))
        np.testing.assert_array_equal(s.get_output(be_mid, 16), want)
        be, rt = s.task_info(be_tid), s.task_info(rt_tid)
        if rt["start"] >= be["start"] and be["end"] >= rt["start"]:
            overlapped += 1
            if mode == B.MODE_NOPREEMPT:
                assert not be["preempted"]
    assert overlapped > 0, "no real-time task arrived during a best-effort run"
    assert s.preempt_times() >= overlapped
    s.shutdown()


def test_be_stream_cap_is_fixed_once_a_best_effort_queue_exists(fake, small_dirs):
    s = B.Scheduler(B.MODE_RESET)
    assert s.set_be_stream_cap(3) == 0
    assert s.set_be_stream_cap(0) == 1           # a window of zero kernels makes no sense
    s.create_queue(B.QUEUE_BE)
    assert s.set_be_stream_cap(1) == 1           # Fail: the stream exists with a window of 3


def test_tile_choice_outside_the_measured_table():
    """A shape the measured table does not hold is scored by two cost models in the same unit:
    batch-1 layers go to the direct family (or the row form for 3x3 / stride 1 / padding 1), a
    device-filling layer stays on a staged tile, and a filter the direct family is not compiled
    for never gets a direct tile."""
    from reef_amd.modelgen import tiling
    assert (200, 169, 200 * 9, 0) not in tiling.TUNED
    t = tiling.choose(200, 169, 1800, fused=True, taps=9, direct=True, rows=True, image=(13, 13))
    assert (t["tile"] in tiling.ROW_TILES or t["tile"] in tiling.DIRECT_TILES) and t["k_chunk"] % 144 == 0
    t = tiling.choose(200, 169, 1800, fused=True, taps=9, direct=True)
    assert t["tile"] in tiling.DIRECT_TILES and t["tasks"] == t["split_k"] * t["m_tiles"] * t["n_tiles"]
    assert t["split_k"] > 1 and t["fused"]            # 143 tiles alone would leave CUs idle
    t = tiling.choose(200, 169, 1800, fused=True, taps=9, direct=False)
    assert t["tile"] not in tiling.DIRECT_TILES and t["tile"] not in tiling.ROW_TILES
    t = tiling.choose(512, 200 * 200, 4608, fused=True, taps=9, direct=True)
    assert t["tile"] not in tiling.DIRECT_TILES          # 40000 pixels x 512 channels fill the device
    t = tiling.choose(96, 500, 16 * 40, fused=True, taps=16, direct=tiling.direct_ok(40, 4, 4))
    assert t["tile"] not in tiling.DIRECT_TILES
    # both models answer in microseconds of one launch
    g = tiling.forced("16x32k4", 256, 196, 1024, 2, 1)
    assert 4.0 < tiling.direct_cost("16x32k4", g, True) < 12.0


def test_a_model_generated_for_running_under_load_differs_in_its_tiles_and_splits_only():
    """GraphBuilder(under_load=True) takes the tile choices measured with several clients on the
    device where the table has them (tuned.TUNED_UNDER_LOAD): same kernels in the same order on
    the same storages with the same parameters, a different tile or split of K on the shapes listed."""
    from reef_amd.modelgen import nets, tiling, tuned
    for key, (tile, split) in tuned.TUNED_UNDER_LOAD.items():
        # a finer split of K folded inside the launch, or another tile
        assert key in tuned.TUNED and (tile, split) != tuned.TUNED[key][:2]
        assert (split < 0 and abs(split) > abs(tuned.TUNED[key][1])) or tile != tuned.TUNED[key][0]
    M, N, K = 32, 196, 1152
    alone = tiling.choose(M, N, K, fused=False, taps=9, direct=True, rows=True, image=(14, 14))
    loaded = tiling.choose(M, N, K, fused=False, taps=9, direct=True, rows=True, image=(14, 14), under_load=True)
    assert alone["tile"] == loaded["tile"] == "g1" and (alone["split_k"], loaded["split_k"]) == (2, 4)
    assert loaded["fused"]
    a, b = nets.densenet(blocks=(2, 2, 2, 2)), nets.densenet(blocks=(2, 2, 2, 2), under_load=True)
    # the same convolutions on the same parameters; a tile that has a pre-activated form (p1) takes
    # the BN + ReLU in front of it into its loads, so the model under load may have fewer launches
    convs = lambda g: [k["attrs"][:12] for k in g.kernels if k["name"].startswith("reef_conv2d_")]
    assert convs(a) == convs(b) and len(b.kernels) <= len(a.kernels)
    assert [p[0] for p in a.params] == [p[0] for p in b.params]
    assert [k["launch_params"] for k in a.kernels] != [k["launch_params"] for k in b.kernels]
    assert nets.BUILDERS["densenet201"]().under_load        # the benchmark's best-effort model
    # matrix products: BERT-base's FFN-down product splits K in four instead of two
    for (M, N, K), (tile, split) in tuned.GEMM_UNDER_LOAD.items():
        alone, loaded = tiling.choose_gemm(M, N, K, 1, True), tiling.choose_gemm(M, N, K, 1, True, under_load=True)
        assert (loaded["tile"], loaded["gemm_split"]) == (tile, split) != (alone["tile"], alone.get("gemm_split", 1))
        assert tiling.choose_gemm(M, N, K, 2, True, under_load=True)["tile"] == tiling.choose_gemm(M, N, K, 2, True)["tile"]
    a, b = nets.bert(layers=1), nets.bert(layers=1, under_load=True)
    assert [k["name"] for k in a.kernels] == [k["name"] for k in b.kernels]
    assert [p[0] for p in a.params] == [p[0] for p in b.params]
    assert sum(x["launch_params"] != y["launch_params"] for x, y in zip(a.kernels, b.kernels)) == 1


def test_stream_drained_falls_back_to_the_query_of_a_backend_without_counters(fake):
    """reef_hal_stream_drained is what the padding loop asks between two real-time launches (the
    reference asks its runtime, scheduler.cpp:655-672 via GPUStreamEmpty); a backend that has no
    call of its own answers through stream_query."""
    L = B.lib()
    s = ctypes.c_void_p()
    assert L.reef_hal_stream_create(4, ctypes.byref(s)) == 0
    drained = ctypes.c_int(-1)
    assert L.reef_hal_stream_drained(s, ctypes.byref(drained)) == 0 and drained.value == 1
    assert L.reef_hal_stream_destroy(s) == 0
