"""End-to-end and per-layer parity of whole models against the CPU oracle,
through all three kernel flavours (raw / DKP single-sided / preemptible), and
the bit-identity guarantees between flavours."""
import ctypes
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd.modelgen import nets
from tests.helpers import compare_storages, max_rel_err, write_model, REL_TOL

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def resnet18_dir(tmp_path_factory):
    g = nets.resnet(18)
    return g, write_model(g, tmp_path_factory.mktemp("r18"))


@pytest.fixture(scope="module")
def resnet18_oracle(resnet18_dir):
    g, d = resnet18_dir
    model = json.load(open(os.path.join(d, g.name + ".json")))
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    x = nets.image_input("resnet18", (3, 224, 224))
    orc.set_input("data", x)
    orc.run()
    return model, orc, x


@pytest.mark.parametrize("kind,preemptible", [(B.BASE, False), (B.TRANS, False), (B.HYBRID, False),
                                              (B.HYBRID, True)])
def test_resnet18_per_layer(resnet18_dir, resnet18_oracle, kind, preemptible):
    """ResNet-18, 3x224x224 (the reference's CPU-runnable configuration): every
    intermediate tensor within 1e-4 of the oracle, in every flavour."""
    g, d = resnet18_dir
    model, orc, x = resnet18_oracle
    exe = B.Executor.from_dir(d, g.name, kind)
    exe.set_input_checked("data", x)
    if preemptible:
        exe.execute_preemptable()
    else:
        exe.execute()
    worst = compare_storages(exe, orc, model, what="resnet18 kind=%d" % kind)
    out = exe.get_output()
    assert out.shape == (1000,) and abs(out.sum() - 1.0) < 1e-4
    print("worst rel err %.2e at storage %s" % worst)


def test_flavours_bit_identical(resnet18_dir, resnet18_oracle):
    """raw, DKP and preemptible flavours run the same arithmetic per task: outputs
    must be bit-identical (the DKP co-run == solo guarantee starts here)."""
    g, d = resnet18_dir
    _, _, x = resnet18_oracle
    outs = []
    last = []
    for kind, pre in ((B.BASE, False), (B.TRANS, False), (B.HYBRID, True)):
        exe = B.Executor.from_dir(d, g.name, kind)
        exe.set_input_checked("data", x)
        exe.execute_preemptable() if pre else exe.execute()
        outs.append(exe.get_output())
        # logits (input of the softmax) are a more sensitive probe than the softmax output
        model = exe  # keep alive
        last.append(exe.get_data(json.load(open(os.path.join(d, g.name + ".json")))["kernels"][-1]["args"][0], 1000))
    for o, l in zip(outs[1:], last[1:]):
        np.testing.assert_array_equal(o, outs[0])
        np.testing.assert_array_equal(l, last[0])


def test_resnet152_end_to_end(tmp_path):
    """ResNet-152 at the benchmark shape: per-layer and end-to-end parity."""
    g = nets.resnet(152)
    d = write_model(g, tmp_path)
    model = json.load(open(os.path.join(d, g.name + ".json")))
    x = nets.image_input("resnet152", (3, 224, 224))
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe.set_input_checked("data", x)
    exe.execute()
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    orc.set_input("data", x)
    orc.run()
    worst = compare_storages(exe, orc, model, what="resnet152")
    print("resnet152 worst per-layer rel err %.2e (storage %s)" % worst)
    logits_idx = model["kernels"][-1]["args"][0]
    assert max_rel_err(exe.get_data(logits_idx, 1000), orc.storage[logits_idx]) < REL_TOL
    assert int(np.argmax(exe.get_output())) == int(np.argmax(orc.get("output")))
    # rerun: same bits (no state left behind by split-K workspaces)
    first = exe.get_data(logits_idx, 1000)
    exe.execute()
    np.testing.assert_array_equal(exe.get_data(logits_idx, 1000), first)


def test_preempt_flag_stops_and_restart_is_bit_identical(resnet18_dir, resnet18_oracle):
    """Flag set before launch: every workgroup leaves at once, no completion is
    counted and the output stays untouched; after clearing the flag a rerun gives
    the same bits as an uninterrupted run (idempotence, src/reef/test/test.cpp:448-489)."""
    g, d = resnet18_dir
    _, _, x = resnet18_oracle
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe.set_input_checked("data", x)
    exe.execute_preemptable()
    ref = exe.get_output()
    slots = exe.read_task_slots()
    blocks = [exe.kernel_info(i)["block_num"] for i in range(exe.num_kernels())]
    assert slots == blocks, "every workgroup of every kernel completed once"

    exe2 = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe2.set_input_checked("data", x)
    exe2.poke_preempt_flag(1)
    exe2.execute_preemptable()
    assert exe2.read_task_slots() == [0] * exe2.num_kernels()
    assert (exe2.get_output() == 0).all(), "storages stay zero-filled"
    exe2.poke_preempt_flag(0)
    exe2.execute_preemptable()
    np.testing.assert_array_equal(exe2.get_output(), ref)


MODEL_INPUTS = {
    "mobilenetv2": lambda: {"data": nets.image_input("mobilenetv2", (3, 224, 224))},
    "densenet201": lambda: {"data": nets.image_input("densenet201", (3, 224, 224))},
    "inceptionv3": lambda: {"data": nets.image_input("inceptionv3", (3, 299, 299))},
    "bert_base": lambda: {"input0": nets.token_input("bert_base", 128, 30522)},
}


@pytest.mark.parametrize("name,preemptible", [("mobilenetv2", False), ("mobilenetv2", True),
                                              ("densenet201", True), ("inceptionv3", False),
                                              ("bert_base", True)])
def test_benchmark_models_per_layer(tmp_path, name, preemptible):
    """The other networks of the benchmark configurations at their full shapes
    (MobileNetV2 1.0, DenseNet-201, Inception-v3 @299, BERT-base seq 128): every
    intermediate tensor within 1e-4 of the CPU oracle."""
    g = nets.BUILDERS[name]()
    d = write_model(g, tmp_path)
    model = json.load(open(os.path.join(d, g.name + ".json")))
    inputs = MODEL_INPUTS[name]()
    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    for k, v in inputs.items():
        exe.set_input_checked(k, v)
        orc.set_input(k, v)
    exe.execute_preemptable() if preemptible else exe.execute()
    orc.run()
    worst = compare_storages(exe, orc, model, what=name)
    print("%s: %d kernels, worst per-layer rel err %.2e (storage %s)" % ((name, len(g.kernels)) + worst))
    assert np.isfinite(exe.get_output()).all()


@pytest.mark.parametrize("kind", [B.BASE, B.HYBRID])
def test_recorded_submission_replays_bit_identical(tmp_path, kind):
    """A whole-model run replays a recorded launch sequence.  Several replays, with new inputs
    copied in and other kernels run eagerly in between, each give exactly the output of the same
    model launched one kernel at a time."""
    g = nets.resnet(18)
    d = write_model(g, tmp_path)
    rec = B.Executor.from_dir(d, g.name, kind)
    rec.set_graph_launch(True)
    one = B.Executor.from_dir(d, g.name, kind)
    one.set_graph_launch(False)
    rng = np.random.default_rng(5)
    for rep in range(4):
        x = (nets.image_input("resnet18", (3, 224, 224)) * (1.0 + 0.25 * rep)
             + rng.standard_normal((3, 224, 224)).astype(np.float32) * 0.1).astype(np.float32)
        rec.set_input_checked("data", x)
        one.set_input_checked("data", x)
        rec.execute()
        one.execute()
        a, b = rec.get_output(), one.get_output()
        assert np.isfinite(a).all()
        np.testing.assert_array_equal(a, b, err_msg="replay %d" % rep)
        rec.execute_to(7)          # eager partial run between replays
    assert not np.array_equal(a, np.zeros_like(a))


def test_split_of_two_meets_in_the_pair_slots_or_on_the_counters_with_the_same_bits(tmp_path):
    """A split of two folded inside the launch has two protocols (REEF_F_PAIR_FOLD): launches
    that run to completion (raw flavour, real-time side of the padding flavour) meet in the pair
    slots with one atomic exchange per element, preemptible launches on the arrival counters.
    Same sums in the same order: all three flavours hold the same bits, run after run and in any
    order on ONE executor (shared buffers), the pair slots and the counters are empty at rest,
    and a preemptible run that was cut short (flag raised) leaves the pair slots alone."""
    g = nets.resnet(152)          # the benchmark network: 71 of its convolutions are such splits
    pair = [k for k in g.kernels if k["name"].startswith("reef_conv2d") and k["attrs"][12] & 64]
    assert len(pair) >= 60, "the network must contain splits of two in the direct family"
    d = write_model(g, tmp_path)
    model = json.load(open(os.path.join(d, g.name + ".json")))
    x = nets.image_input("resnet152", (3, 224, 224))
    logits = model["kernels"][-1]["args"][0]
    n_log = model["storage"][logits]["size"]

    def slots_and_counters(exe):
        for k in model["kernels"]:
            a = k["attrs"]
            if k["name"].startswith("reef_conv2d") and a[12] & 64:
                n_args = a[23] if a[23] else len(k["args"])
                ws = k["args"][n_args - 2]
                mn = a[3] * a[4] * a[5]
                words = exe.get_data(ws, model["storage"][ws]["size"] // 4, np.int32)
                assert words.size == 3 * mn and not words[2 * mn:].any(), k["name"]
        for i, s in enumerate(model["storage"]):
            if s["name"] == "reef_sync":
                assert not exe.get_data(i, s["size"], np.int32).any()

    exe = B.Executor.from_dir(d, g.name, B.HYBRID)
    exe.set_input_checked("data", x)
    exe.execute()
    want = exe.get_data(logits, n_log)
    slots_and_counters(exe)
    for run in ("preemptible", "raw", "cut short", "raw", "preemptible"):
        zero = np.zeros(n_log, np.float32)
        assert B.lib().reef_executor_set_input_idx(exe.h, logits, ctypes.c_void_p(zero.ctypes.data),
                                                   ctypes.c_size_t(zero.nbytes)) == 0
        if run == "cut short":
            exe.poke_preempt_flag(1)
            exe.execute_preemptable()          # every workgroup leaves at once
            exe.poke_preempt_flag(0)
            slots_and_counters(exe)
            continue
        exe.execute_preemptable() if run == "preemptible" else exe.execute()
        np.testing.assert_array_equal(exe.get_data(logits, n_log), want, err_msg=run)
        slots_and_counters(exe)
    exe.close()
    # the padding flavour, single-sided (real-time side): pair slots again
    t = B.Executor.from_dir(d, g.name, B.TRANS)
    t.set_input_checked("data", x)
    for _ in range(2):
        t.execute()
        np.testing.assert_array_equal(t.get_data(logits, n_log), want)
        slots_and_counters(t)
    t.close()
