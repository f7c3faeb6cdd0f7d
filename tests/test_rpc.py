"""The RPC front-end (reef_amd/rpc.py) against the reference's contract: src/reef/protos/reef.proto:5-79
on the wire, handlers as src/reef/server/server.cpp:34-188, blobs in POSIX shared memory named
"<mid>_<name>".  The round trip is the reference's own rpc test (src/reef/test/test.cpp:34-57: client
-> server -> device -> shared memory), here over the recording backend with the oracle as the device."""
import json
import os

import grpc
import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd import rpc
from reef_amd.modelgen import nets
from tests.fakehal import FakeHal
from tests.helpers import write_model


@pytest.fixture()
def served(tmp_path_factory):
    fake = FakeHal().install()
    fake.lib.fake_hal_set_auto_progress(4)
    server = rpc.REEFServer("127.0.0.1:0", measure_imported=False)    # no device to time kernels on here
    server.run()
    dirs = {}
    for g in (nets.mocked_kernel(), nets.resnet(18, image=(3, 32, 32), classes=16, name="tiny18")):
        dirs[g.name] = (g, write_model(g, tmp_path_factory.mktemp(g.name)))
    yield server, "127.0.0.1:%d" % server.port, dirs
    server.shutdown()
    fake.remove()


def test_messages_have_the_reference_wire_format():
    """Field numbers and types of reef.proto:25-79, pinned by hand-encoded bytes."""
    m = rpc.MSG["LoadModelRequest"](dir="a", name="bc", qid=3)
    assert m.SerializeToString() == b"\x0a\x01a\x12\x02bc\x18\x03"
    assert rpc.MSG["SetPriorityRequest"](rt=True).SerializeToString() == b"\x08\x01"
    r = rpc.MSG["RegisterBlobReply"].FromString(b"\x08\x01\x12\x06" + b"7_data" + b"\x18\x80\x60")
    assert (r.succ, r.key, r.size) == (True, "7_data", 12288)
    assert rpc.MSG["InferRequest"](mid=5, **{"async": True}).SerializeToString() == b"\x08\x05\x10\x01"
    r = rpc.MSG["InferReply"].FromString(b"\x08\x01\x10\x09")
    assert (r.succ, r.tid) == (True, 9)
    assert rpc.MSG["GetBlobRequest"](key="k").SerializeToString() == b"\x0a\x01k"
    assert rpc.MSG["SetBlobReply"](succ=True).SerializeToString() == b"\x08\x01"
    assert rpc.MSG["LoadModelReply"].FromString(b"\x08\x01\x10\x02").mid == 2
    assert rpc.MSG["SetPriorityReply"].FromString(b"\x08\x01\x10\x20").qid == 32
    assert rpc.DEFAULT_REEF_ADDR == "localhost:34543"


def test_round_trip_through_shared_memory(served):
    server, addr, dirs = served
    g, d = dirs["tiny18"]
    x = nets.image_input("rpc", (3, 32, 32))
    model = json.load(open(os.path.join(d, g.name + ".json")))
    orc = O.GraphOracle(model, os.path.join(d, g.name + ".param"))
    orc.set_input("data", x)
    want = orc.run().copy()

    client = rpc.REEFClient(addr)
    assert client.init(True) and client.qid == 32          # all real-time clients share queue 32 (scheduler.h:147-148)
    m = client.load_model(d, g.name)
    inp = m.get_input_blob("data")
    assert m.input_blob_key == "%d_data" % m.mid and inp.size == x.nbytes
    assert os.path.exists("/dev/shm/" + m.input_blob_key)   # what a C++ client would shm_open
    inp.array()[:] = x.ravel()
    m.load_input()
    tid, lat = m.infer()
    out = m.get_output_blob("output")
    m.get_output()
    np.testing.assert_array_equal(out.array()[:want.size], want)
    tid2, _ = m.infer()
    assert tid2 != tid and lat > 0

    # a best-effort client beside it gets a queue of its own
    be = rpc.REEFClient(addr)
    be.init(False)
    assert be.qid != 32
    gm, dm = dirs["mocked_kernel"]
    mm = be.load_model(dm, gm.name)
    for name in "abc":
        blob, key = mm.register_blob(name)
        blob.array()[:] = 3.0
        assert be.calls["SetBlob"](rpc.MSG["SetBlobRequest"](key=key)).succ
        blob.close()
    mm.infer()
    ob = mm.get_output_blob("output")
    mm.get_output()
    np.testing.assert_array_equal(ob.array(), np.full(8192, 18.0, np.float32))   # test.cpp:105-115
    key = m.input_blob_key
    client.close()
    be.close()
    server_side = server.shms[key][2]
    assert server_side.create           # the server made the blob and unlinks it (shared_memory.cpp:29-33)


def test_failures_answer_succ_false_with_status_ok(served):
    server, addr, dirs = served
    ch = grpc.insecure_channel(addr)
    call = lambda meth, req: ch.unary_unary("/reef.rpc.REEFService/" + meth,
                                            request_serializer=lambda b: b,
                                            response_deserializer=rpc.MSG[meth + "Reply"].FromString)(req)
    # hand-encoded requests, as a foreign client would send them
    assert call("LoadModel", b"\x0a\x04/nop\x12\x01x\x18\x20").succ is False        # no such directory
    assert call("RegisterBlob", b"\x08\x63\x12\x04data").succ is False               # model 99 does not exist
    assert call("SetBlob", b"\x0a\x05no_me").succ is False
    assert call("GetBlob", b"\x0a\x05no_me").succ is False
    assert call("Infer", b"\x08\x63").succ is False
    r = call("SetPriority", b"")                                                     # rt = false
    assert r.succ and r.qid == 0
    ch.close()


def test_load_model_imports_a_directory_of_the_reference(served, tmp_path):
    """A client sends the path of a directory as the reference's pipeline wrote it (mobilenet.json with
    TVM's kernel names, mobilenet.param with its keys; the code objects there are for another GPU and
    are never opened): LoadModel imports it and the inference gives what the table's
    interpretation of the reference graph gives."""
    import shutil
    from reef_amd import legacy
    from reef_amd.modelgen import builder as MB
    from tests.test_legacy_import import golden, interpret_reference_graph
    server, addr, _ = served
    name = "mobilenet"
    ref_dir = tmp_path / "resource" / name
    ref_dir.mkdir(parents=True)
    shutil.copyfile(golden(name), ref_dir / (name + ".json"))
    params = legacy.seeded_params(golden(name))
    MB.write_params(str(ref_dir / (name + ".param")), params)
    (ref_dir / (name + ".trans.co")).write_bytes(b"not for this GPU")
    x = nets.image_input("rpc", (3, 224, 224))
    ref = json.load(open(golden(name)))
    want = interpret_reference_graph(ref, legacy.load_table(name), dict(params), x)
    out_idx = [i for i, s in enumerate(ref["storage"]) if s["name"] == "output"][0]

    client = rpc.REEFClient(addr)
    client.init(True)
    m = client.load_model(str(ref_dir), name)
    # imported once, into a directory keyed by where the source lies and the state of its files
    import glob
    first = glob.glob(os.path.join(server.import_root, "*", name, name + ".be.co"))
    assert server.import_root and len(first) == 1
    inp = m.get_input_blob("data")
    inp.array()[:] = x.ravel()
    m.load_input()
    m.infer()
    out = m.get_output_blob("output")
    m.get_output()
    got = out.array()[:1000]
    assert abs(float(got.sum()) - 1.0) < 1e-4
    np.testing.assert_allclose(got, want[out_idx][:1000], rtol=0, atol=1e-6)
    # a directory of the reference without a packaged table is answered like any other failure
    other = tmp_path / "resource" / "nonet"
    other.mkdir()
    shutil.copyfile(golden(name), other / "nonet.json")
    reply = client.calls["LoadModel"](rpc.MSG["LoadModelRequest"](dir=str(other), name="nonet", qid=client.qid))
    assert reply.succ is False
    # the same directory again is served from the first import; a model of the same name in ANOTHER
    # directory (other parameters) is imported on its own instead of being answered with the first
    client.load_model(str(ref_dir), name)
    assert len(glob.glob(os.path.join(server.import_root, "*", name, name + ".json"))) == 1
    second = tmp_path / "elsewhere" / name
    second.mkdir(parents=True)
    shutil.copyfile(golden(name), second / (name + ".json"))
    MB.write_params(str(second / (name + ".param")), [(k, np.asarray(v) * 0.5) for k, v in params])
    client.load_model(str(second), name)
    assert len(glob.glob(os.path.join(server.import_root, "*", name, name + ".json"))) == 2
    client.close()
