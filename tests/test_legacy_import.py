"""The importer for the reference's own model directories (reef_amd/legacy.py) on the reference's
resource/resnet152, resource/mobilenet, resource/alexnet, resource/vgg, resource/resnet18 and
resource/inception graphs
(tests/golden/<model>.json, data fixtures): same storages, same call
order, and the imported graph computes what the reference's kernels compute according to the
table of shapes that was derived by running those kernels (tests/golden/make_resnet152_shapes.py,
make_graph_shapes.py).

The CPU check interprets the reference graph DIRECTLY from the table with the oracle's ops and
compares that with the imported model run through the executor (fake backend) -- two code paths
from the same table, so a wrong role, attribute order or epilogue flag in the importer shows."""
import ctypes
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd import legacy
from reef_amd.modelgen import builder as MB
from reef_amd.modelgen import nets
from tests.fakehal import FakeHal

HERE = os.path.dirname(os.path.abspath(__file__))
REF_JSON = os.path.join(HERE, "golden", "resnet152.json")
TABLE = os.path.join(HERE, "golden", "resnet152_kernel_shapes.json")


def interpret_reference_graph(ref, table, params, x, upto=None):
    """The reference graph evaluated from the table with the oracle's ops.  Returns the storages."""
    st = {i: np.zeros(s["size"], np.float32) for i, s in enumerate(ref["storage"])}
    for i, s in enumerate(ref["storage"]):
        if s["name"] in params:
            st[i][:] = params[s["name"]]
    st[0][:] = x.ravel()
    wino = {}
    for n, k in enumerate(ref["kernels"]):
        if upto is not None and n >= upto:
            break
        e, a = table[k["name"]], k["args"]
        if e["op"] == "winograd_data":
            wino[a[1]] = (a[0], None)
        elif e["op"] == "winograd_gemm":
            wino[a[2]] = (wino.pop(a[1])[0], a[0])
        elif e["op"] == "conv2d":
            cin, H, W, cout, s = e["cin"], e["h"], e["w"], e["cout"], e["stride"]
            (kh, kwid), (ph, pw) = legacy.pair(e["k"]), legacy.pair(e["pad"])
            Ho, Wo = (H + 2 * ph - kh) // s + 1, (W + 2 * pw - kwid) // s + 1
            if e.get("winograd_tile"):
                # three calls of the reference = one direct convolution on the un-transformed filter
                alpha = e["winograd_tile"] + 2
                src, u = wino.pop(a[0])
                ws = legacy.winograd_untransform(st[u].reshape(alpha, alpha, cin, cout), e["winograd_tile"])
                a = [src, u, a[1]] + list(a[2:])
            else:
                ws = st[a[1]].reshape(cout, cin, kh, kwid)
            xs = st[a[0]][:cin * H * W].reshape(cin, H, W)
            full = lambda i: st[i][:cout * Ho * Wo].reshape(cout, Ho, Wo)
            kw = dict(stride=(s, s), pad=(ph, pw))
            ep = e["epilogue"]
            if ep == "none":
                y = O.conv2d(xs, ws, act=0, **kw)
            elif ep == "relu":
                y = O.conv2d(xs, ws, act=1, **kw)
            elif ep == "residual":
                y = O.conv2d(xs, ws, residual=full(a[3]), act=0, **kw)
            elif ep == "bias_relu":
                y = O.conv2d(xs, ws, bias=st[a[3]], act=1, **kw)
            elif ep == "residual_bias_relu":
                y = O.conv2d(xs, ws, residual=full(a[3]), bias=st[a[4]], act=1, **kw)
            else:
                y = O.conv2d(xs, ws, residual=full(a[3]), scale=st[a[4]], shift=st[a[5]], act=1, **kw)
            st[a[2]][:y.size] = y.ravel()
        elif e["op"] == "dwconv2d":
            C, H, W, kk, sd, p = e["c"], e["h"], e["w"], e["k"], e["stride"], e["pad"]
            y = O.conv2d(st[a[0]][:C * H * W].reshape(C, H, W), st[a[1]].reshape(C, 1, kk, kk), bias=st[a[3]],
                         stride=(sd, sd), pad=(p, p), groups=C, act=e["act"])
            st[a[2]][:y.size] = y.ravel()
        elif e["op"] == "eltwise":
            C, inner = e["c"], e["inner"]
            y = O.eltwise(st[a[1]][:C * inner].reshape(C, inner), shift=st[a[2]], act=e["act"])
            st[a[0]][:y.size] = y.ravel()
        elif e["op"] == "pool2d":
            C, H, W = e["c"], e["h"], e["w"]
            y = O.pool2d(st[a[0]][:C * H * W].reshape(C, H, W), (e["k"], e["k"]), (e["stride"], e["stride"]),
                         (e["pad"], e["pad"]), 0 if e["mode"] == "max" else 1, bias=st[a[2]] if e.get("bias") else None,
                         act=e.get("act", 0), count_include_pad=bool(e.get("count_include_pad")))
            st[a[1]][:y.size] = y.ravel()
        elif e["op"] == "concat":
            hw = e["h"] * e["w"]
            y = np.concatenate([st[a[1 + j]][:c * hw] for c, j in zip(e["parts"], e["operand"])])
            st[a[0]][:y.size] = y
        elif e["op"] == "global_avgpool":
            C, hw = e["c"], e["hw"]
            st[a[1]][:C] = O.global_avgpool(st[a[0]][:C * hw].reshape(C, hw)).ravel()
        elif e["op"] == "copy":
            st[a[0]][:e["n"]] = st[a[1]][:e["n"]]
        elif e["op"] == "dense":
            y = O.dense(st[a[0]][:e["in"]].reshape(1, e["in"]), st[a[1]].reshape(e["out"], e["in"]), bias=st[a[3]],
                        act=e.get("act", 0))
            st[a[2]][:e["out"]] = y.ravel()
        elif e["op"] == "softmax":
            st[a[1]][:e["cols"]] = O.softmax(st[a[0]][:e["cols"]].reshape(1, e["cols"])).ravel()
        else:
            raise AssertionError(e["op"])
    return st


@pytest.fixture(scope="module")
def imported(tmp_path_factory):
    d = str(tmp_path_factory.mktemp("legacy152"))
    g = legacy.import_model(REF_JSON, table=TABLE)
    g.write(d)
    params = legacy.seeded_params(REF_JSON, table=TABLE)
    MB.write_params(os.path.join(d, g.name + ".param"), params)
    return g, d, dict(params)


def test_import_keeps_storages_order_and_parameter_keys(imported):
    g, d, params = imported
    ref = json.load(open(REF_JSON))
    out = json.load(open(os.path.join(d, "resnet152.json")))
    n = len(ref["storage"])
    assert out["storage"][:n] == ref["storage"]                # same indices, names, sizes
    assert all(s["name"] in ("temp_arg", "reef_sync") for s in out["storage"][n:])
    assert out["args"] == ref["args"]
    assert len(out["kernels"]) == len(ref["kernels"]) == 207   # one launch per reference launch
    assert g.imported_from == [k["name"] for k in ref["kernels"]]
    for ko, kr in zip(out["kernels"], ref["kernels"]):
        assert ko["name"].startswith("reef_") and ko["launch_params"][3:] == [256, 1, 1]
        # every storage the reference kernel touches is bound to the replacement, and the
        # replacement binds nothing else of the reference's storages
        assert sorted(set(x for x in ko["args"] if x < n)) == sorted(set(kr["args"])), (ko, kr)
    assert len(params) == sum(1 for s in ref["storage"] if s["name"].startswith("p"))


def test_imported_graph_equals_the_table_interpretation_through_the_executor(imported):
    g, d, params = imported
    ref = json.load(open(REF_JSON))
    table = json.load(open(TABLE))
    x = nets.image_input("legacy", (3, 64, 64))
    want = interpret_reference_graph(ref, table, params, x)
    fake = FakeHal().install()
    exe = None
    try:
        exe = B.Executor.from_dir(d, "resnet152", B.HYBRID)
        exe.set_input_checked("data", x)
        exe.execute()
        got = exe.get_output()      # the whole `output` storage: a shared buffer, the classes come first
        out_idx = [i for i, s in enumerate(ref["storage"]) if s["name"] == "output"][0]
        np.testing.assert_allclose(got, want[out_idx][:got.size], rtol=0, atol=1e-6)
        assert abs(float(got[:1000].sum()) - 1.0) < 1e-4
        # every intermediate buffer of the reference graph, as the last writer left it
        for i, s in enumerate(ref["storage"]):
            if s["name"] == "null":
                have = exe.get_data(i, s["size"])
                scale = max(np.abs(want[i]).max(), 1e-6)
                assert np.abs(have - want[i]).max() <= 1e-5 * scale, i
    finally:
        if exe is not None:
            exe.close()
        fake.remove()


def test_import_refuses_a_table_that_does_not_fit_the_graph():
    table = json.load(open(TABLE))
    bad = json.loads(json.dumps(table))
    bad["fused_nn_conv2d_add_nn_relu_9_kernel0"]["h"] = 8
    with pytest.raises(legacy.ImportError_, match="fused_nn_conv2d_add_nn_relu_9_kernel0"):
        legacy.import_model(REF_JSON, table=bad)
    del bad["fused_nn_softmax_kernel0"]
    bad["fused_nn_conv2d_add_nn_relu_9_kernel0"]["h"] = 16
    with pytest.raises(legacy.ImportError_, match="not in the table"):
        legacy.import_model(REF_JSON, table=bad)
    # the packaged table is the fixture
    assert legacy.load_table("resnet152") == table


# ---- the directories whose tables come from a walk of the graph: MobileNet v1 (depthwise
# ---- convolutions), AlexNet, and `vgg` (in fact a pre-activation ResNet-50 at 64 x 64) ---------
def golden(name, what=""):
    return os.path.join(HERE, "golden", name + what + ".json")


@pytest.mark.parametrize("name,calls,ops", [
    ("mobilenet", 31, {"reef_dwconv2d": 13, "reef_global_avgpool": 1, "reef_copy": 1, "reef_dense": 1, "reef_softmax": 1}),
    ("alexnet", 13, {"reef_pool2d": 3, "reef_copy": 1, "reef_dense": 3, "reef_softmax": 1}),
    ("vgg", 71, {"reef_eltwise": 13, "reef_pool2d": 1, "reef_global_avgpool": 1, "reef_copy": 1, "reef_dense": 1,
                 "reef_softmax": 1}),
])
def test_walked_models_import_with_storages_order_and_keys(name, calls, ops, tmp_path):
    ref = json.load(open(golden(name)))
    g = legacy.import_model(golden(name))
    g.write(str(tmp_path))
    out = json.load(open(os.path.join(str(tmp_path), name + ".json")))
    n = len(ref["storage"])
    assert out["storage"][:n] == ref["storage"] and out["args"] == ref["args"]
    assert all(s["name"] in ("temp_arg", "reef_sync") for s in out["storage"][n:])
    assert len(out["kernels"]) == len(ref["kernels"]) == calls
    count = {}
    for ko, kr in zip(out["kernels"], ref["kernels"]):
        sym = ko["name"].split("#")[0]
        count[sym] = count.get(sym, 0) + 1
        assert sorted(set(x for x in ko["args"] if x < n)) == sorted(set(kr["args"])), (ko, kr)
    for sym, c in ops.items():
        assert count.get(sym) == c, (sym, count)
    assert sum(c for sym, c in count.items() if sym.startswith("reef_conv2d")) == calls - sum(ops.values())
    assert legacy.load_table(name) == json.load(open(golden(name, "_kernel_shapes")))
    # every entry but the softmax was reproduced by the oracle from the reference's own kernel
    assert [k.replace("tvmgen_default_", "") for k, e in legacy.load_table(name).items()
            if not e["witness"]] == ["fused_nn_softmax_kernel0"]


def test_winograd_filter_transform():
    """F(2x2, 3x3) is the textbook transform (Lavin & Gray) up to the order of its points; both
    tile sizes: transform then least-squares inverse gives the filter back, and the transform of a
    filter that is 1 at the centre is the outer product of G's middle column with itself."""
    G2 = legacy.winograd_G(2)
    textbook = [[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]]
    assert sorted(map(tuple, G2.tolist())) == sorted(map(tuple, textbook))
    rs = np.random.default_rng(3)
    for tile in (2, 4):
        G = legacy.winograd_G(tile)
        assert G.shape == (tile + 2, 3) and np.linalg.matrix_rank(G) == 3
        g = rs.standard_normal((5, 3, 3, 3)).astype(np.float32)
        U = legacy.winograd_transform(g, tile)
        assert U.shape == (tile + 2, tile + 2, 3, 5)
        np.testing.assert_allclose(legacy.winograd_untransform(U, tile), g, rtol=0, atol=1e-6)
        centre = np.zeros((1, 1, 3, 3), np.float32)
        centre[0, 0, 1, 1] = 1
        np.testing.assert_allclose(legacy.winograd_transform(centre, tile)[:, :, 0, 0], np.outer(G[:, 1], G[:, 1]),
                                   rtol=0, atol=1e-7)


def test_resnet18_import_replaces_winograd_triples_by_direct_convolutions(tmp_path):
    """resource/resnet18: 57 calls, 13 of its convolutions as three calls each on transformed
    weights (p4: 36 x 64 x 64 values for a 3x3 64 -> 64 filter).  Imported: 31 kernels, a storage
    `<key>_direct` per transformed weight, the reference's storages untouched."""
    name = "resnet18"
    ref = json.load(open(golden(name)))
    g = legacy.import_model(golden(name))
    g.write(str(tmp_path))
    out = json.load(open(os.path.join(str(tmp_path), name + ".json")))
    n = len(ref["storage"])
    assert out["storage"][:n] == ref["storage"]
    added = [s for s in out["storage"][n:] if s["name"] not in ("temp_arg", "reef_sync")]
    assert len(added) == 13 and all(s["name"].endswith("_direct") for s in added)
    assert len(ref["kernels"]) == 57 and len(out["kernels"]) == 57 - 2 * 13 == len(g.imported_calls)
    table = legacy.load_table(name)
    skipped = [i for i, k in enumerate(ref["kernels"]) if table[k["name"]]["op"].startswith("winograd_")]
    assert sorted(set(range(57)) - set(skipped)) == g.imported_calls
    assert g.direct_weights["p4"] == ("p4_direct", 4, 64, 64)
    assert sum(1 for e in table.values() if e.get("winograd_tile") == 2) == 9       # 28x28 and smaller
    # parameters: a transformed weight of the reference's file comes back as the filter it was made from
    params = legacy.seeded_params(golden(name))
    MB.write_params(os.path.join(str(tmp_path), "ref.param"), params)
    back = legacy.read_params(os.path.join(str(tmp_path), "ref.param"))
    assert [k for k, _ in back] == [k for k, _ in params]
    conv = dict(legacy.convert_params(g, back))
    assert "p4" not in conv and conv["p4_direct"].size == 64 * 64 * 9 and dict(back)["p4"].size == 36 * 64 * 64
    np.testing.assert_allclose(legacy.winograd_transform(conv["p4_direct"].reshape(64, 64, 3, 3), 4).ravel(),
                               dict(back)["p4"], rtol=0, atol=1e-6)
    with pytest.raises(legacy.ImportError_, match="p4"):
        legacy.convert_params(g, [("p4", np.zeros(9 * 64 * 64, np.float32))])
    assert legacy.load_table(name) == json.load(open(golden(name, "_kernel_shapes")))


def test_inception_import_has_asymmetric_filters_padded_pools_and_concatenations(tmp_path):
    """resource/inception (Inception-v3 at 299 x 299, 146 calls): 1x7 / 7x1 / 1x3 / 3x1 / 5x5 filters,
    twelve Winograd triples of six kinds (two of them unpadded), 3x3 stride-1 average pools that count the padding,
    and concatenations whose operands TVM lists in the REVERSE of their channel order."""
    name = "inception"
    ref = json.load(open(golden(name)))
    table = legacy.load_table(name)
    assert table == json.load(open(golden(name, "_kernel_shapes")))
    g = legacy.import_model(golden(name))
    g.write(str(tmp_path))
    out = json.load(open(os.path.join(str(tmp_path), name + ".json")))
    n = len(ref["storage"])
    assert out["storage"][:n] == ref["storage"] and len(ref["kernels"]) == 146
    concat_parts = sum(len(table[k["name"]]["parts"]) for k in ref["kernels"] if table[k["name"]]["op"] == "concat")
    concats = sum(1 for k in ref["kernels"] if table[k["name"]]["op"] == "concat")
    triples = sum(1 for k in ref["kernels"] if table[k["name"]].get("winograd_tile"))
    assert (concats, concat_parts, triples) == (11, 46, 12)
    assert len(out["kernels"]) == 146 - 2 * triples + concat_parts - concats
    assert sorted(set(g.imported_calls)) == [i for i, k in enumerate(ref["kernels"])
                                              if not table[k["name"]]["op"].startswith("winograd_")]
    assert all(e["operand"] == list(range(len(e["parts"])))[::-1] for e in table.values() if e["op"] == "concat")
    assert {tuple(e["k"]) for e in table.values() if e["op"] == "conv2d" and not isinstance(e["k"], int)} \
        == {(1, 7), (7, 1), (1, 3), (3, 1)}
    assert sum(1 for e in table.values() if e.get("winograd_tile") and e["pad"] == 0) == 2
    assert all(e.get("count_include_pad") for e in table.values() if e["op"] == "pool2d" and e["mode"] == "avg" and e["pad"])
    assert abs(g.flops / 1e9 - 11.426) < 0.01        # Inception-v3's convolutions + classifier
    with pytest.raises(legacy.ImportError_, match="fused_concatenate_11_kernel0"):
        bad = json.loads(json.dumps(table))
        bad["fused_concatenate_11_kernel0"]["operand"] = [0, 1, 2, 3]
        legacy.import_model(golden(name), table=bad)


def test_import_model_dir_converts_a_parameter_file_with_transformed_weights(tmp_path):
    """A directory laid out like the reference's (resnet18.json + resnet18.param holding the
    Winograd weights transformed) -> a directory of this build: graph, profile, code objects, and
    a parameter file in which every transformed weight has become its direct filter; a directory
    without Winograd kernels keeps its parameter file byte for byte."""
    import shutil
    for name in ("resnet18", "mobilenet"):
        src, dst = tmp_path / (name + "_ref"), tmp_path / (name + "_out")
        src.mkdir()
        shutil.copyfile(golden(name), src / (name + ".json"))
        params = legacy.seeded_params(golden(name))
        MB.write_params(str(src / (name + ".param")), params)
        g = legacy.import_model_dir(str(src), name, str(dst))
        for ext in (".json", ".profile.json", ".param", ".raw.co", ".be.co", ".trans.co"):
            assert (dst / (name + ext)).exists(), ext
        got = legacy.read_params(str(dst / (name + ".param")))
        if name == "mobilenet":
            assert not g.direct_weights
            assert (dst / (name + ".param")).read_bytes() == (src / (name + ".param")).read_bytes()
            continue
        keys = [k for k, _ in got]
        assert len(g.direct_weights) == 13 and all(k + "_direct" in keys and k not in keys for k in g.direct_weights)
        assert len(keys) == len(params)
        storages = {s_["name"]: s_["size"] for s_ in json.load(open(dst / (name + ".json")))["storage"]}
        assert all(storages[k] == a.size for k, a in got)          # every parameter fits the storage of its name


@pytest.mark.parametrize("name,side", [("mobilenet", 224), ("vgg", 64), ("resnet18", 224), ("inception", 299)])
def test_imported_walked_model_equals_the_table_interpretation_through_the_executor(name, side, tmp_path):
    d = str(tmp_path)
    g = legacy.import_model(golden(name))
    g.write(d)
    params = legacy.seeded_params(golden(name))
    MB.write_params(os.path.join(d, name + ".param"), legacy.convert_params(g, params))
    ref = json.load(open(golden(name)))
    x = nets.image_input("legacy", (3, side, side))
    want = interpret_reference_graph(ref, legacy.load_table(name), dict(params), x)
    fake = FakeHal().install()
    exe = None
    try:
        exe = B.Executor.from_dir(d, name, B.HYBRID)
        exe.set_input_checked("data", x)
        exe.execute()
        for i, s in enumerate(ref["storage"]):
            if s["name"] in ("null", "output"):
                have = exe.get_data(i, s["size"])
                scale = max(np.abs(want[i]).max(), 1e-6)
                assert np.abs(have - want[i]).max() <= 1e-5 * scale, (i, s)
        out_idx = [i for i, s in enumerate(ref["storage"]) if s["name"] == "output"][0]
        assert abs(float(exe.get_data(out_idx, ref["storage"][out_idx]["size"])[:1000].sum()) - 1.0) < 1e-4
    finally:
        if exe is not None:
            exe.close()
        fake.remove()


# ---- the transformer directory --------------------------------------------------------------
def interpret_bert_graph(ref, table, params, ids, position_ids):
    """resource/bert evaluated call by call from the table with the oracle's ops: every call of a
    LayerNorm / softmax chain is computed as its own step (mean, variance, ...), the way the
    reference runs it.  Returns the storages."""
    dt = {"int64": np.int64, "uint1": np.uint8, "byte": np.uint8}
    st = {i: np.zeros(s["size"], dt.get(s["stype"], np.float32)) for i, s in enumerate(ref["storage"])}
    for i, s in enumerate(ref["storage"]):
        if s["name"] in params:
            st[i][:] = params[s["name"]]
    st[0][:] = ids
    st[ref["kernels"][1]["args"][4]][:] = position_ids
    f32 = lambda i: st[i].view(np.float32) if st[i].dtype != np.float32 else st[i]   # byte scratch holds floats
    for k in ref["kernels"]:
        name, a = k["name"], k["args"]
        e = table[name]
        if name.startswith("fused_full_equal"):
            st[a[0]][:e["n"]] = 0
        elif e["op"] == "embedding":
            S, H = e["seq"], e["hidden"]
            y = st[a[1]].reshape(-1, H)[st[a[2]][:S]] + st[a[3]].reshape(-1, H)[st[a[4]][:S]]
            st[a[0]][:S * H] = y.ravel()
        elif name.startswith("fused_mean_1_kernel0"):
            f32(a[1])[:480] = st[a[0]][:480 * 480].reshape(480, 480).sum(1, dtype=np.float64)
        elif name.startswith("fused_mean_1_kernel1"):
            st[a[0]][:480] = f32(a[1])[:480] / 480
        elif name.startswith("fused_variance_1_kernel0"):
            x = st[a[0]][:480 * 480].reshape(480, 480).astype(np.float64)
            f32(a[2])[:480] = ((x - st[a[1]][:480, None]) ** 2).sum(1)
        elif name.startswith("fused_variance_1_kernel1"):
            st[a[0]][:480] = f32(a[1])[:480] / 480
        elif e["op"] == "layernorm":
            R, C = e["rows"], e["cols"]
            x = st[a[1]][:R * C].reshape(R, C).astype(np.float64)
            y = (x - st[a[2]][:R, None]) / np.sqrt(st[a[3]][:R, None].astype(np.float64) + e["eps"]) * st[a[4]][:C] + st[a[5]][:C]
            st[a[0]][:R * C] = y.ravel()
        elif e["op"] == "copy":
            st[a[0]][:e["n"]] = st[a[1]][:e["n"]]
        elif e["op"] == "gemm_nt":
            bt, M, N, K = e["batch"], e["m"], e["n"], e["k"]
            y = O.batch_matmul(st[a[0]][:bt * M * K].reshape(bt, M, K), st[a[1]][:bt * N * K].reshape(bt, N, K), True, 1.0)
            st[a[2]][:y.size] = y.ravel()
        elif e["op"] == "rowbias_heads":
            R, Hh, D = e["rows"], e["heads"], e["d"]
            x = st[a[1]][:R * Hh * D].reshape(R, Hh, D) + st[a[2]][:R, None, None]
            st[a[0]][:x.size] = (x.transpose(1, 0, 2) * np.float32(e.get("scale", 1.0))).ravel()
        elif e["op"] == "rowbias_transpose":
            R, C = e["rows"], e["cols"]
            st[a[0]][:R * C] = (st[a[1]][:R * C].reshape(R, C) + st[a[2]][:R, None]).T.ravel()
        elif e["op"] == "heads_merge":
            Hh, R, D = e["heads"], e["rows"], e["d"]
            st[a[0]][:Hh * R * D] = st[a[1]][:Hh * R * D].reshape(Hh, R, D).transpose(1, 0, 2).ravel()
        elif name.startswith("fused_reshape_cast_broadcast_to_like_where"):
            n = e["copy"]
            x = st[a[2]][:n].reshape(-1, 480)
            st[a[0]][:n] = np.where(st[a[1]][:480][None, :] != 0, -np.inf, x).ravel()
        elif name.startswith("fused_nn_softmax_1_kernel0"):              # row maxima
            f32(a[0])[:12 * 480] = st[a[1]][:12 * 480 * 480].reshape(-1, 480).max(1)
        elif name.startswith("fused_nn_softmax_1_kernel1"):              # exp(x - max)
            x = st[a[1]][:12 * 480 * 480].reshape(-1, 480)
            f32(a[0])[:x.size] = np.exp(x - f32(a[2])[:12 * 480, None]).ravel()
        elif name.startswith("fused_nn_softmax_1_kernel2"):              # row sums
            f32(a[0])[:12 * 480] = f32(a[1])[:12 * 480 * 480].reshape(-1, 480).sum(1, dtype=np.float64)
        elif e["op"] == "masked_softmax":
            R, C = e["rows"], e["cols"]
            st[a[0]][:R * C] = (f32(a[1])[:R * C].reshape(R, C) / f32(a[2])[:R, None]).ravel()
        elif e["op"] == "rowbias_add":
            R, C = e["rows"], e["cols"]
            st[a[0]][:R * C] = ((st[a[1]][:R * C].reshape(R, C) + st[a[2]][:R, None]) + st[a[3]][:R * C].reshape(R, C)).ravel()
        elif e["op"] == "rowbias_gelu":
            R, C = e["rows"], e["cols"]
            st[a[0]][:R * C] = O.bias_gelu((st[a[1]][:R * C].reshape(R, C) + st[a[2]][:R, None]).astype(np.float32)).ravel()
        else:
            raise AssertionError(name)
    return st


def test_imported_bert_equals_the_call_by_call_interpretation(tmp_path):
    """resource/bert: 205 calls -> 160 kernels (a LayerNorm's five calls and a softmax's five become
    one kernel each, a row-bias call two); the imported graph through the executor (recording
    backend) gives what the reference's call sequence gives when every call is evaluated as its
    own step."""
    name = "bert"
    ref = json.load(open(golden(name)))
    table = legacy.load_table(name)
    assert table == json.load(open(golden(name, "_kernel_shapes"))) and all(e["witness"] for e in table.values())
    g = legacy.import_model(golden(name))
    d = str(tmp_path)
    g.write(d)
    out = json.load(open(os.path.join(d, name + ".json")))
    n = len(ref["storage"])
    assert out["storage"][:n] == ref["storage"] and len(ref["kernels"]) == 205 and len(out["kernels"]) == 160
    skipped = [i for i, k in enumerate(ref["kernels"]) if i not in g.imported_calls]
    assert len(skipped) == 1 + 13 * 4 + 6 * 3 and all(table[ref["kernels"][i]["name"]]["op"] in ("chain_stage", "mask_fill")
                                                      for i in skipped)
    params = legacy.seeded_params(golden(name))
    assert len(params) == 100 and "p2" not in dict(params)      # the int64 position ids are not a float parameter
    MB.write_params(os.path.join(d, name + ".param"), legacy.convert_params(g, params))
    ids = nets.token_input("legacy", 480, 30522)
    pos = np.arange(480, dtype=np.int64)
    want = interpret_bert_graph(ref, table, dict(params), ids, pos)
    fake = FakeHal().install()
    exe = None
    try:
        exe = B.Executor.from_dir(d, name, B.HYBRID)
        for idx, arr in ((0, ids), (ref["kernels"][1]["args"][4], pos)):
            arr = np.ascontiguousarray(arr, np.int64)
            assert B.lib().reef_executor_set_input_idx(exe.h, idx, ctypes.c_void_p(arr.ctypes.data),
                                                       ctypes.c_size_t(arr.nbytes)) == 0
        exe.execute()
        out_idx = [i for i, s in enumerate(ref["storage"]) if s["name"] == "output"][0]
        got = exe.get_data(out_idx, 480 * 480)
        assert np.isfinite(got).all()
        assert np.abs(got - want[out_idx][:got.size]).max() <= 1e-4 * np.abs(want[out_idx]).max()
        rows = got.reshape(480, 480)
        assert np.abs(rows.mean(1)).max() < 0.2     # the last call is a LayerNorm with gamma ~ 1, beta ~ 0
    finally:
        if exe is not None:
            exe.close()
        fake.remove()
