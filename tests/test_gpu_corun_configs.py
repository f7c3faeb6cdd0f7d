"""The co-location workloads of the benchmark configurations, checked for the two guarantees
the reference's scheduler tests assert on ResNet-18 (src/reef/test/test.cpp:448-536):

  * a best-effort task that was preempted and restarted, or that rode along in real-time
    kernels (dynamic kernel padding), ends with exactly the bits of an uninterrupted solo run;
  * the real-time model's result is bit-identical to its solo run whatever shared its launches.

Here at the model pairs the configurations name: 4 x DenseNet-201 under ResNet-152 (reset-based
preemption), MobileNetV2 under ResNet-152 (dynamic kernel padding, measured profiles), and
2 x BERT-base under Inception-v3.  After each co-run EVERY float storage a kernel writes (all
activations, the logits, split-K partial tensors) is compared with the solo run bit for bit,
and the logits with the CPU oracle within 1e-4 of the tensor's largest magnitude.
The last test does the same with two of the reference's OWN model directories, imported
(reef_amd/legacy.py): resource/resnet18 real-time over two resource/mobilenet best-effort clients.
"""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd import legacy
from reef_amd import profiler
from reef_amd.modelgen import builder as MB
from reef_amd.modelgen import nets
from tests.helpers import max_rel_err, write_model, REL_TOL

pytestmark = pytest.mark.gpu

NAMES = ("resnet152", "densenet201", "mobilenetv2", "inceptionv3", "bert_base")


IMPORTED = {"resnet18": 224, "mobilenet": 224}      # reference model directory -> image side
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def write_imported(name, root):
    """tests/golden/<name>.json (the reference's graph file) imported onto this build's kernels,
    with seeded parameters in the reference's own format converted the way a `.param` file is."""
    ref_json = os.path.join(GOLDEN, name + ".json")
    g = legacy.import_model(ref_json)
    d = str(root)
    g.write(d)
    MB.write_params(os.path.join(d, name + ".param"), legacy.convert_params(g, legacy.seeded_params(ref_json)))
    return g, d


def model_input(name):
    if name in IMPORTED:
        return "data", nets.image_input(name, (3, IMPORTED[name], IMPORTED[name]))
    if name == "bert_base":
        return "input0", nets.token_input(name, 128, 30522)
    side = 299 if name == "inceptionv3" else 224
    return "data", nets.image_input(name, (3, side, side))


def written_float_storages(model):
    idx = set()
    for k in model["kernels"]:
        idx.update(k["args"])
    out = []
    for i in sorted(idx):
        s = model["storage"][i]
        if s["name"] in ("data", "input0", "reef_sync") or s["name"].startswith("p"):
            continue
        # not the split-K workspaces (temp_arg): scratch whose content depends on how the kernel
        # was launched (a best-effort launch leaves its partial tiles there, a launch that runs
        # to completion folds a split of two through the pair slots and leaves nothing)
        if s["stype"] == "float32":
            out.append(i)
    return out


class Solo:
    """One model: its directory with a measured profile, the state of every written storage
    after an uninterrupted solo run, and the oracle's result."""

    def __init__(self, name, root):
        self.name = name
        if name in IMPORTED:
            self.g, self.dir = write_imported(name, root)
        else:
            self.g = nets.BUILDERS[name]()
            self.dir = write_model(self.g, root)
        profiler.write_profile(self.dir, name, iters=5, warmup=1)
        self.model = json.load(open(os.path.join(self.dir, name + ".json")))
        self.key, self.x = model_input(name)
        exe = B.Executor.from_dir(self.dir, name, B.HYBRID)
        exe.set_input_checked(self.key, self.x)
        exe.execute()
        self.idx = written_float_storages(self.model)
        self.state = {i: exe.get_data(i, self.n_floats(i)) for i in self.idx}
        self.out_size = exe.get_data_size("output") // 4
        exe.close()
        # the tensor the last kernel reads (logits of the classifiers) and the model output
        self.probe = [self.model["kernels"][-1]["args"][0],
                      [i for i, s in enumerate(self.model["storage"]) if s["name"] == "output"][0]]
        orc = O.GraphOracle(self.model, os.path.join(self.dir, name + ".param"))
        orc.set_input(self.key, self.x)
        orc.run()
        for i in self.probe:
            if self.model["storage"][i]["stype"] != "float32":
                continue
            err = max_rel_err(self.state[i], orc.storage[i])
            assert err <= REL_TOL, "%s solo storage %d: rel err %.2e vs the oracle" % (name, i, err)

    def n_floats(self, i):
        s = self.model["storage"][i]
        return s["size"] // 4 if s["stype"] == "byte" else s["size"]

    def check(self, sched, mid, what):
        """Every written storage of model `mid` of a scheduler equals the solo run's bits.
        The arrival counters of folded split-K kernels are int32 and must be back at zero."""
        for i in self.idx:
            got = sched.get_data(mid, i, self.n_floats(i))
            if not np.array_equal(got, self.state[i]):
                bad = int(np.flatnonzero(got != self.state[i])[0])
                raise AssertionError("%s: storage %d (%s) differs from the solo run at element %d: %r vs %r"
                                     % (what, i, self.model["storage"][i]["name"], bad, got[bad],
                                        self.state[i][bad]))
        for i, s in enumerate(self.model["storage"]):
            if s["name"] == "reef_sync":
                cnt = sched.get_data(mid, i, s["size"], np.int32)
                assert not cnt.any(), "%s: split-K arrival counters left non-zero" % what
        # the pair slots of a split of two (REEF_F_PAIR_FOLD = 64) are empty at rest
        for k in self.model["kernels"]:
            a = k.get("attrs", [])
            if k["name"].startswith("reef_conv2d") and len(a) >= 24 and a[12] & 64:
                n_args = a[23] if a[23] else len(k["args"])
                ws = k["args"][n_args - 2]
                mn = a[3] * a[4] * a[5]
                slots = sched.get_data(mid, ws, self.n_floats(ws), np.int32)[2 * mn:3 * mn]
                assert slots.size == mn and not slots.any(), "%s: pair slots of %s left non-zero" % (what, k["name"])


@pytest.fixture(scope="module")
def solos(tmp_path_factory):
    cache = {}

    def get(name):
        if name not in cache:
            cache[name] = Solo(name, tmp_path_factory.mktemp(name))
        return cache[name]
    return get


def corun(solos, rt_name, be_name, n_be, mode, requests, interval_us, slack=None):
    rt_s, be_s = solos(rt_name), solos(be_name)
    s = B.Scheduler(mode)
    s.set_wait_sync(True)
    if slack is not None:
        s.set_dkp_slack_percent(slack)
    rt = s.load_model(rt_s.dir, rt_name)
    s.bind_model_queue(s.create_queue(B.QUEUE_RT), rt)
    assert s.set_input(rt, rt_s.x, rt_s.key) == 0
    bes = []
    for _ in range(n_be):
        m = s.load_model(be_s.dir, be_name)
        s.bind_model_queue(s.create_queue(B.QUEUE_BE), m)
        assert s.set_input(m, be_s.x, be_s.key) == 0
        bes.append(m)
    s.run()
    r = s.run_load(rt, bes, requests=requests, warmup=5, mean_interval_us=interval_us, seed=0x5EEF)
    # the clients stop after their current task; every best-effort model then completes one more
    # uninterrupted inference so that its final state is that of a whole run
    r2 = s.run_load(rt, bes, requests=0, be_only_ms=40)
    assert (r2["be_completed"] > 0).all()
    rt_s.check(s, rt, "%s real-time under %d x %s" % (rt_name, n_be, be_name))
    for j, m in enumerate(bes):
        be_s.check(s, m, "%s best-effort client %d under %s" % (be_name, j, rt_name))
    stats = {"preempt_times": s.preempt_times(), "padded_kernels": s.padded_kernels(),
             "padded_by_op": s.padded_by_op(),
             "be_preempted": r["be_preempted"], "be_completed": r["be_completed"],
             "be_padded": r["be_padded"], "preempt_us": s.preempt_samples(),
             "rt_p50_us": float(np.percentile(r["rt_latency_us"], 50))}
    s.shutdown()
    s.close()
    return stats


def test_cfg3_four_densenet201_under_resnet152_reset_preemption(solos):
    """4 best-effort DenseNet-201 clients, real-time ResNet-152 every 3 ms on average: at least
    30 real-time requests and 10 preemptions; afterwards all five models hold solo bits."""
    st = corun(solos, "resnet152", "densenet201", 4, B.MODE_REEF, requests=40, interval_us=3000.0)
    print("cfg3:", {k: (v.tolist() if hasattr(v, "tolist") and k != "preempt_us" else v)
                    for k, v in st.items() if k != "preempt_us"},
          "preempt mean %.1f us max %d" % (st["preempt_us"].mean(), st["preempt_us"].max()))
    assert st["preempt_times"] >= 10
    assert st["be_preempted"].sum() >= 10 and st["be_completed"].sum() > 0


def test_cfg4_mobilenetv2_padded_into_resnet152(solos):
    """Dynamic kernel padding with measured profiles: MobileNetV2 (whole-block, expansion + depthwise
    and pointwise launches, all of the convolution class) rides in ResNet-152's launches.  Real-time requests back to back on average every 2 ms keep the
    device mostly in real-time mode, so padding is where the best-effort model makes progress."""
    st = corun(solos, "resnet152", "mobilenetv2", 1, B.MODE_REEF, requests=60, interval_us=2000.0,
               slack=100)
    print("cfg4:", {k: (v.tolist() if hasattr(v, "tolist") else v) for k, v in st.items() if k != "preempt_us"})
    assert st["padded_kernels"] > 0
    # the generated MobileNetV2 has no depthwise launch of its own any more: its depthwise stages are
    # inside convolution launches (REEF_OP_CONV2D), and nothing else may have been merged
    assert st["padded_by_op"][1] > 0, "no merged launch carried a convolution of the best-effort model"
    assert sum(st["padded_by_op"]) == st["padded_by_op"][1] + st["padded_by_op"][7] + st["padded_by_op"][8]
    assert st["be_completed"].sum() > 0


def test_cfg5_two_bert_base_under_inceptionv3(solos):
    """2 best-effort BERT-base encoders (GEMM, LayerNorm, GELU, softmax kernels) preempted by a
    real-time Inception-v3."""
    st = corun(solos, "inceptionv3", "bert_base", 2, B.MODE_REEF, requests=40, interval_us=3000.0)
    print("cfg5:", {k: (v.tolist() if hasattr(v, "tolist") else v) for k, v in st.items() if k != "preempt_us"})
    assert st["preempt_times"] >= 10
    assert st["be_preempted"].sum() >= 5 and st["be_completed"].sum() > 0


def test_imported_reference_directories_corun(solos):
    """The reference's resource/resnet18 (its Winograd triples as direct convolutions) as the
    real-time model over two clients of its resource/mobilenet (depthwise kernels), both imported:
    preemptions and padded kernels happen, and all three models end with solo bits."""
    st = corun(solos, "resnet18", "mobilenet", 2, B.MODE_REEF, requests=60, interval_us=1500.0, slack=100)
    print("imported:", {k: (v.tolist() if hasattr(v, "tolist") else v) for k, v in st.items() if k != "preempt_us"})
    assert st["preempt_times"] >= 10 and st["be_completed"].sum() > 0
    assert st["padded_kernels"] > 0
