"""rpc.resnet18_param of the reference (src/reef/test/test.cpp:34-57) on the device: client ->
gRPC -> scheduler -> GPU -> shared memory, with a best-effort client loading the device beside it."""
import json
import os
import threading

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import rpc
from reef_amd.modelgen import nets
from tests.helpers import REL_TOL, max_rel_err, write_model

pytestmark = pytest.mark.gpu


def test_rpc_round_trip_on_the_device(tmp_path_factory):
    g = nets.resnet(18, image=(3, 64, 64), classes=100, name="resnet18_rpc")
    d = write_model(g, tmp_path_factory.mktemp("rpc18"))
    x = nets.image_input("rpc", (3, 64, 64))
    model = json.load(open(os.path.join(d, g.name + ".json")))
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    orc.set_input("data", x)
    want = orc.run().copy()

    server = rpc.REEFServer("127.0.0.1:0")
    server.run()
    addr = "127.0.0.1:%d" % server.port
    try:
        stop = threading.Event()
        be_done = []

        def best_effort():
            c = rpc.REEFClient(addr)
            c.init(False)
            m = c.load_model(d, g.name)
            m.get_input_blob("data").array()[:] = x.ravel()
            m.load_input()
            while not stop.is_set():
                m.infer()
                be_done.append(1)
            ob = m.get_output_blob("output")
            m.get_output()
            be_done.append(ob.array()[:want.size].copy())
            c.close()

        t = threading.Thread(target=best_effort)
        t.start()
        c = rpc.REEFClient(addr)
        c.init(True)
        m = c.load_model(d, g.name)
        m.get_input_blob("data").array()[:] = x.ravel()
        m.load_input()
        out = m.get_output_blob("output")
        lats = []
        for _ in range(20):
            lats.append(m.infer()[1])
            m.get_output()
            got = out.array()[:want.size]
            assert np.isfinite(got).all() and max_rel_err(got, want) <= REL_TOL
        first = out.array()[:want.size].copy()
        stop.set()
        t.join(timeout=30)
        assert not t.is_alive() and len(be_done) >= 2
        # the preempted best-effort client holds the same bits as the real-time one
        np.testing.assert_array_equal(be_done[-1], first)
        print("rpc round trip: median %.2f ms over %d requests, %d best-effort inferences beside them"
              % (sorted(lats)[len(lats) // 2] * 1e3, len(lats), len(be_done) - 1))
        c.close()
    finally:
        server.shutdown()


def test_rpc_load_model_takes_a_directory_of_the_reference(tmp_path):
    """The reference's resource/resnet18 as its pipeline wrote it (graph with TVM's kernel names, a
    parameter file holding the Winograd weights transformed) sent to LoadModel as it is: the
    server imports it, times its kernels for the profile, and the client's inference through
    shared memory gives the probabilities the oracle gives for the imported graph."""
    import shutil
    from reef_amd import legacy
    from reef_amd.modelgen import builder as MB
    name = "resnet18"
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name + ".json")
    ref_dir = tmp_path / "resource" / name
    ref_dir.mkdir(parents=True)
    shutil.copyfile(golden, ref_dir / (name + ".json"))
    MB.write_params(str(ref_dir / (name + ".param")), legacy.seeded_params(golden))
    x = nets.image_input("rpc", (3, 224, 224))
    server = rpc.REEFServer("127.0.0.1:0")
    server.run()
    try:
        c = rpc.REEFClient("127.0.0.1:%d" % server.port)
        c.init(True)
        m = c.load_model(str(ref_dir), name)
        import glob
        (imported,) = glob.glob(os.path.join(server.import_root, "*", name))   # keyed by its source
        prof = json.load(open(os.path.join(imported, name + ".profile.json")))
        assert prof["model_latency"] > 0 and len(prof["kernel_latency"]) == 31
        orc = O.GraphOracle(json.load(open(os.path.join(imported, name + ".json"))), os.path.join(imported, name + ".param"))
        orc.set_input("data", x)
        want = orc.run().copy()
        m.get_input_blob("data").array()[:] = x.ravel()
        m.load_input()
        _, lat = m.infer()
        out = m.get_output_blob("output")
        m.get_output()
        got = out.array()[:1000]
        assert abs(float(got.sum()) - 1.0) < 1e-4 and max_rel_err(got, want[:1000]) <= REL_TOL
        print("imported resnet18 over rpc: %.2f ms" % (lat * 1e3))
        c.close()
    finally:
        server.shutdown()
