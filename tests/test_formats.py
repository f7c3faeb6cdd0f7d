"""Model resource formats: the product's parsers on the files the reference's own
parser tests use (src/reef/test/test.cpp:59-91), the oracle's Python reader on the
same files, and round trips through both writers."""
import array
import ctypes
import json
import os
import re
import struct

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from reef_amd.modelgen import builder as MB

L = B.lib()
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def model_summary(path):
    v = [ctypes.c_int() for _ in range(4)]
    st = L.reef_model_parse_summary(path.encode(), *[ctypes.byref(x) for x in v])
    return st, [x.value for x in v]


def profile_summary(path):
    v = [ctypes.c_int() for _ in range(4)]
    st = L.reef_profile_parse_summary(path.encode(), *[ctypes.byref(x) for x in v])
    return st, [x.value for x in v]


@pytest.mark.parametrize("name,n_storage,n_kernels", [("mocked_kernel", 5, 2), ("resnet152", 317, 207),
                                                      ("resnet18", None, None), ("bert", None, None)])
def test_parse_reference_graph_json(golden_dir, name, n_storage, n_kernels):
    path = os.path.join(golden_dir, name + ".json")
    ref = json.load(open(path))
    st, (ns, nk, na, nsh) = model_summary(path)
    assert st == 0
    assert (ns, nk, na, nsh) == (len(ref["storage"]), len(ref["kernels"]), len(ref["args"]),
                                 len(ref["shared_memory"]))
    assert nk > 0                                  # parser.parse_model, test.cpp:59-65
    if n_storage is not None:
        assert (ns, nk) == (n_storage, n_kernels)
    # the oracle's graph loader accepts the same file
    orc = O.GraphOracle(ref)
    assert len(orc.storage) == ns
    if name == "resnet152":
        assert orc.storage[0].size == 12288        # 3 x 64 x 64 input
    if name == "bert":
        assert orc.storage[0].dtype == np.int64 and ref["storage"][0]["stype"] == "int64"


def test_parse_reference_profiles(golden_dir):
    st, (ml, nk, mn, cnt) = profile_summary(os.path.join(golden_dir, "resnet18.profile.json"))
    assert st == 0 and nk == 54 and mn > 0 and cnt > 0          # parser.parse_profile, test.cpp:79-91
    st, (ml, nk, mn, cnt) = profile_summary(os.path.join(golden_dir, "mocked_kernel.profile.json"))
    assert (st, ml, nk, mn, cnt) == (0, 30, 2, 14, 32)
    st, (ml, nk, _, _) = profile_summary(os.path.join(golden_dir, "resnet152.profile.json"))
    assert (st, ml) == (0, 13233) and nk == len(json.load(open(os.path.join(golden_dir, "resnet152.profile.json")))["kernel_latency"])


def test_profile_to_json_round_trip(golden_dir, tmp_path):
    for name in ("mocked_kernel", "resnet18", "resnet152"):
        path = os.path.join(golden_dir, name + ".profile.json")
        buf = ctypes.create_string_buffer(1 << 16)
        assert L.reef_profile_roundtrip(path.encode(), buf, ctypes.c_size_t(len(buf))) == 0
        assert json.loads(buf.value.decode()) == json.load(open(path))
        # what to_json writes parses again to the same summary
        p2 = tmp_path / (name + ".json")
        p2.write_bytes(buf.value)
        assert profile_summary(str(p2)) == profile_summary(path)


def reference_style_param_file(path, params):
    """Byte-for-byte what script/tvm_generate_model.py:66-76 (dump_params) writes."""
    with open(path, "wb") as f:
        f.write(bytes("TVM_MODEL_PARAMS\0", "ascii"))
        f.write(array.array('Q', [len(params)]).tobytes())
        for k, v in params.items():
            p = array.array('f', v.flatten().tolist())
            f.write(bytes(k, "ascii"))
            f.write(bytes("\0", "ascii"))
            f.write(array.array('Q', [len(p)]).tobytes())
            f.write(p.tobytes())


def param_summary(path, key):
    n, klen = ctypes.c_uint64(), ctypes.c_uint64()
    first, last = ctypes.c_float(), ctypes.c_float()
    st = L.reef_param_parse_summary(path.encode(), key.encode(), ctypes.byref(n), ctypes.byref(klen),
                                    ctypes.byref(first), ctypes.byref(last))
    return st, n.value, klen.value, first.value, last.value


def test_param_format_both_writers_both_readers(tmp_path):
    rng = np.random.default_rng(3)
    params = {"p0": rng.standard_normal((8, 3, 3, 3)).astype(np.float32),
              "p22": rng.standard_normal(294912).astype(np.float32),   # the size test.cpp:76 expects of p22
              "a_rather_long_parameter_name_1": np.arange(5, dtype=np.float32)}
    ref_file, own_file = str(tmp_path / "ref.param"), str(tmp_path / "own.param")
    reference_style_param_file(ref_file, params)
    MB.write_params(own_file, [(k, v) for k, v in params.items()])
    assert open(ref_file, "rb").read() == open(own_file, "rb").read()
    for key, arr in params.items():
        st, n, klen, first, last = param_summary(ref_file, key)
        assert (st, n, klen) == (0, 3, arr.size)
        assert first == arr.reshape(-1)[0] and last == arr.reshape(-1)[-1]
    got = O.read_params(ref_file)
    assert set(got) == set(params)
    for k in params:
        np.testing.assert_array_equal(got[k], params[k].reshape(-1))
    assert param_summary(ref_file, "nope")[0] == 2


def test_param_parser_rejects_malformed(tmp_path):
    bad = tmp_path / "bad.param"
    bad.write_bytes(b"NOT_A_PARAM_FILE\0" + struct.pack("<Q", 1))
    assert param_summary(str(bad), "p0")[0] == 2
    trunc = tmp_path / "trunc.param"
    trunc.write_bytes(b"TVM_MODEL_PARAMS\0" + struct.pack("<Q", 1) + b"p0\0" + struct.pack("<Q", 10) + b"\0" * 8)
    assert param_summary(str(trunc), "p0")[0] == 2
    empty = tmp_path / "empty.param"
    empty.write_bytes(b"TVM_MODEL_PARAMS\0" + struct.pack("<Q", 0))   # the reference asserts count != 0
    assert param_summary(str(empty), "p0")[0] == 2
    assert param_summary(str(tmp_path / "missing.param"), "p0")[0] == 2


def test_json_subset_and_superset(tmp_path):
    """Single-quoted strings and bare decimals as the reference's tokenizer takes them
    (src/reef/util/json.cpp:39-74), plus standard JSON it rejects (true/false/null, exponents)."""
    p = tmp_path / "m.json"
    p.write_text("{'storage': [{'name': 'a', 'size': 4, 'stype': 'float32'}],\n"
                 " \"kernels\": [{\"name\": \"add\", \"launch_params\": [1,1,1,4,8,4], \"args\": [0, 0, 0],"
                 "  \"attrs\": [-3, 7], \"extra\": true, \"f\": 1.5e3, \"n\": null}],\n"
                 " \"args\": [0], \"shared_memory\": {\"add\": 1024}}")
    assert model_summary(str(p)) == (0, [1, 1, 1, 1])
    for text in ("{", "{\"storage\": [}", "{\"storage\": [], \"kernels\": [{\"name\": \"k\", \"launch_params\": [1,2], \"args\": []}]}",
                 "{\"storage\": [], \"kernels\": [{\"name\": \"k\", \"launch_params\": [1,1,1,1,1,1], \"args\": [3]}]}", "bogus"):
        p.write_text(text)
        assert model_summary(str(p))[0] == 2, text
    assert model_summary(str(tmp_path / "missing.json"))[0] == 2


def test_arg_offsets_are_checked_against_their_storages(tmp_path):
    """The added key `arg_offsets` (bytes into each operand's storage): one entry per argument,
    multiples of 16, inside the storage; the reference's reader never looks at the key."""
    p = tmp_path / "m.json"
    body = ("{\"storage\": [{\"name\": \"a\", \"size\": 64, \"stype\": \"float32\"}, {\"name\": \"b\", \"size\": 8, "
            "\"stype\": \"float32\"}], \"kernels\": [{\"name\": \"add\", \"launch_params\": [1,1,1,4,8,4], "
            "\"args\": [0, 0, 1], \"arg_offsets\": %s}], \"args\": [0], \"shared_memory\": {}}")
    for offs, ok in (("[0, 128, 16]", True), ("[0, 240, 0]", True), ("[0, 0, 0]", True),
                     ("[0, 128]", False),          # one entry per argument
                     ("[0, 8, 0]", False),         # 16-byte steps
                     ("[0, 256, 0]", False),       # a holds 256 bytes
                     ("[0, 0, 32]", False),        # b holds 32 bytes
                     ("[0, -16, 0]", False)):
        p.write_text(body % offs)
        assert (model_summary(str(p))[0] == 0) == ok, offs


def test_generated_model_is_reference_parsable_subset(tmp_path):
    """Generated graph JSON holds only ints, strings, lists and dicts (what the reference's
    parser accepts) and keeps its four top-level keys."""
    from reef_amd.modelgen import nets
    g = nets.resnet(18, image=(3, 32, 32), classes=8, name="t")
    g.write(str(tmp_path), link_code_objects=False)
    m = json.load(open(tmp_path / "t.json"))
    assert set(m) == {"storage", "kernels", "args", "shared_memory"}

    def walk(v):
        if isinstance(v, dict):
            assert all(isinstance(k, str) for k in v)
            for x in v.values():
                walk(x)
        elif isinstance(v, list):
            for x in v:
                walk(x)
        else:
            assert isinstance(v, (int, str)) and not isinstance(v, bool), v
    walk(m)
    assert all(len(k["launch_params"]) == 6 for k in m["kernels"])
    assert {s["stype"] for s in m["storage"]} <= {"float32", "int64", "byte", "uint1", "int32"}
    st, (ns, nk, _, _) = model_summary(str(tmp_path / "t.json"))
    assert (st, ns, nk) == (0, len(m["storage"]), len(m["kernels"]))
    prof = json.load(open(tmp_path / "t.profile.json"))
    assert set(prof["kernel_latency"]) == {k["name"] for k in m["kernels"]}


def test_library_exports_every_declared_symbol():
    """Every function declared in include/*.h is exported by libreef_amd.so."""
    lib = B.lib()
    declared = []
    for h in ("reef_hal.h", "reef_c.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"typedef struct reef_hal_backend \{.*?\} reef_hal_backend;", "", text, flags=re.S)
        declared += re.findall(r"\b(reef_[a-z0-9_]+)\s*\(", text)
    declared = sorted(set(declared))
    assert len(declared) > 80
    missing = [n for n in declared if not hasattr(lib, n)]
    assert not missing, missing


def test_code_object_metadata_reader():
    """Kernel resources come from the code object's metadata note (host-only parse)."""
    from reef_amd.paths import code_object
    out = (ctypes.c_int * 6)()
    for fl in ("raw", "be", "trans"):
        co = code_object(fl).encode()
        assert L.reef_code_object_kernel_meta(co, b"reef_conv2d_128x128", out) == 0
        vg, ag, sg, lds, scratch, kernarg = list(out)
        assert ag >= 64 and 73744 <= lds <= 73744 + 16 and scratch == 0 and 64 + 40 <= vg <= 512
        assert L.reef_code_object_kernel_meta(co, b"reef_eltwise", out) == 0
        assert out[3] <= 16 and out[4] == 0
        assert L.reef_code_object_kernel_meta(co, b"no_such_kernel", out) == 2
    # kernarg block sizes: raw = ReefOpDesc (160 B), be = two pointers + desc
    assert L.reef_code_object_kernel_meta(code_object("raw").encode(), b"reef_pool2d", out) == 0
    assert out[5] == 176
    assert L.reef_code_object_kernel_meta(code_object("be").encode(), b"reef_pool2d", out) == 0
    assert out[5] >= 192           # + the compiler's hidden arguments
    assert L.reef_code_object_kernel_meta(code_object("trans").encode(), b"reef_pool2d", out) == 0
    assert out[5] == 424           # sizeof(ReefDkpArgs)
    # the proxies claim exactly the register ranges of their class: (arch VGPRs, accumulation registers)
    for cls, (arch, acc) in {"8": (64, 0), "5": (96, 0), "4": (96, 32), "3": (136, 32), "3b": (152, 16),
                             "2": (192, 64), "2b": (224, 32), "2c": (128, 128), "1": (256, 256)}.items():
        assert L.reef_code_object_kernel_meta(code_object("trans").encode(),
                                              ("merge_framework_" + cls).encode(), out) == 0
        assert out[4] == 0 and out[3] == 0 and out[5] == 424, "proxy %s: no scratch, no LDS of its own" % cls
        assert (out[0] - out[1], out[1]) == (arch, acc), (cls, list(out))
        assert 512 // ((out[0] + 7) // 8 * 8) == int(cls[0]), "proxy %s: wavefronts per SIMD" % cls
    # no kernel of any flavour spills
    for fl in ("raw", "be", "trans"):
        for k in ("reef_conv2d_128x128", "reef_conv2d_pw_64x64", "reef_conv2d_u_64x128", "reef_gemm_nt_128x128",
                  "reef_gemm_nn_64x64", "reef_dense", "reef_layernorm", "add"):
            assert L.reef_code_object_kernel_meta(code_object(fl).encode(), k.encode(), out) == 0
            assert out[4] == 0, (fl, k)


def test_benchmark_models_name_only_compiled_kernels_without_scratch():
    """Every kernel symbol the generator emits for the four CNNs and BERT exists in all three
    code objects, uses no scratch memory, and has a proxy whose register ranges hold it."""
    import ctypes
    from reef_amd.modelgen import nets
    from reef_amd.paths import code_object
    L = B.lib()
    out = (ctypes.c_int * 6)()
    symbols = set()
    for name in ("resnet152", "densenet201", "inceptionv3", "mobilenetv2", "bert_base"):
        g = nets.BUILDERS[name]()
        symbols |= {k["name"].split("#")[0] for k in g.kernels}
    assert any(s.startswith("reef_conv2d_d") for s in symbols)      # the direct family is in use
    for fl in ("raw", "be", "trans"):
        co = code_object(fl).encode()
        for sym in sorted(symbols):
            assert L.reef_code_object_kernel_meta(co, sym.encode(), out) == 0, (fl, sym)
            assert out[4] == 0, "%s in %s.co uses %d bytes of scratch" % (sym, fl, out[4])
    co = code_object("trans").encode()
    # every one of those kernels fits the register ranges of some proxy with any other
    proxies = []
    for n in ("8", "5", "4", "3", "3b", "2", "2b", "2c", "1"):
        assert L.reef_code_object_kernel_meta(co, ("merge_framework_" + n).encode(), out) == 0
        assert out[4] == 0
        proxies.append((out[0] - out[1], out[1], out[2]))
    for sym in sorted(symbols):
        assert L.reef_code_object_kernel_meta(co, sym.encode(), out) == 0
        assert any(out[0] - out[1] <= v and out[1] <= a and out[2] <= s for v, a, s in proxies), (sym, list(out))


def test_direct_tile_geometry():
    """Launch geometry of the direct family: K is split on channel boundaries, in whole steps
    (16 channels of a filter with several taps, 128 channels of a 1x1 filter)."""
    from reef_amd.modelgen import tiling
    f = tiling.forced("16x16k4", 256, 196, 2304, 1, 9)
    assert (f["m_tiles"], f["n_tiles"], f["split_k"], f["k_chunk"], f["tasks"]) == (16, 13, 1, 2304, 208)
    f = tiling.forced("16x16k4", 88, 169, 72 * 9, 2, 9)
    assert f["k_chunk"] % (16 * 9) == 0 and f["split_k"] == 2 and f["k_chunk"] * 2 >= 72 * 9
    f = tiling.forced("16x16k4", 512, 49, 1024, 3, 1)
    assert f["k_chunk"] % 128 == 0 and f["split_k"] * f["k_chunk"] >= 1024
    assert tiling.direct_ok(256, 3, 3) and tiling.direct_ok(64, 1, 1) and tiling.direct_ok(24, 1, 7)
    assert tiling.direct_ok(24, 1, 7, "16x32k4") and not tiling.direct_ok(24, 1, 7, "16x64k4")
    f = tiling.forced("32x32d4", 256, 196, 2304, 4, 9)
    assert (f["m_tiles"], f["n_tiles"], f["split_k"], f["tasks"]) == (8, 7, 4, 224)
    assert tiling.lds_bytes("32x32d4") == 4 * 4 * 320 * 4 + 16
    assert not tiling.direct_ok(3, 7, 7) and not tiling.direct_ok(20, 1, 1) and not tiling.direct_ok(16, 4, 4)
    assert tiling.direct_ok(48, 5, 5) and tiling.direct_ok(48, 5, 5, "16x32k4") and not tiling.direct_ok(48, 5, 5, "32x32d4")
    # the analytic model never picks the direct tile; only the measured table may, and only
    # when the caller vouches for the filter
    t = tiling.choose(256, 196, 2304, fused=False, pointwise=False, taps=9, direct=False)
    assert t["tile"] != "16x16k4"
    assert tiling.lds_bytes("16x16k4") == 4 * 320 * 4 + 16


def test_gemm_tile_choice_follows_the_line_rule():
    """BERT-base's products: the generator takes a direct tile where a workgroup's stream of
    cache lines, (BM + BN) K / 32 times the workgroups queued per CU, is shorter than the staged
    tile's, and never without K-contiguous, 16-byte aligned operands."""
    from reef_amd.modelgen import tiling
    t = tiling.choose_gemm(128, 768, 768, 1, True)                               # projections
    assert (t["tile"], t["gemm_split"]) == ("16x32k4", 1)
    t = tiling.choose_gemm(128, 768, 3072, 1, True)              # FFN down: the long K split in two
    assert (t["tile"], t["gemm_split"]) == ("32x32d4", 2)
    assert tiling.choose_gemm(12 * 128, 128, 3072, 12, True).get("gemm_split", 1) == 1    # a batch never splits
    assert tiling.choose_gemm(128, 3072, 768, 1, True)["tile"] == "32x32k4"      # FFN up: staged
    assert tiling.choose_gemm(128, 768, 768, 1, False)["tile"] in tiling.GEMM_TILES
    for t in tiling.GEMM_DIRECT_TILES:
        f = tiling.forced(t, 128, 768, 768, 1)
        assert f["split_k"] == 1 and f["tasks"] == f["m_tiles"] * f["n_tiles"]


def _kernel_descriptors(path):
    """name -> 64-byte kernel descriptor, from the code object's dynamic symbols <name>.kd."""
    import struct
    blob = open(path, "rb").read()
    magic = b"__CLANG_OFFLOAD_BUNDLE__"
    if blob.startswith(magic):          # hipcc --genco wraps the ELF in an offload bundle
        n, = struct.unpack_from("<Q", blob, len(magic))
        pos = len(magic) + 8
        for _ in range(n):
            off, size, tlen = struct.unpack_from("<QQQ", blob, pos)
            triple = blob[pos + 24:pos + 24 + tlen]
            pos += 24 + tlen
            if b"gfx950" in triple:
                blob = blob[off:off + size]
                break
    assert blob[:4] == b"\x7fELF" and blob[4] == 2
    shoff, = struct.unpack_from("<Q", blob, 0x28)
    shentsize, shnum, _ = struct.unpack_from("<HHH", blob, 0x3A)
    secs = [struct.unpack_from("<IIQQQQIIQQ", blob, shoff + i * shentsize) for i in range(shnum)]
    out = {}
    for (_, typ, _, _, off, size, link, _, _, entsize) in secs:
        if typ not in (2, 11):      # SHT_SYMTAB, SHT_DYNSYM
            continue
        stroff = secs[link][4]
        for k in range(size // entsize):
            st_name, _, _, shndx, value, _ = struct.unpack_from("<IBBHQQ", blob, off + k * entsize)
            end = blob.index(b"\0", stroff + st_name)
            name = blob[stroff + st_name:end].decode()
            if not name.endswith(".kd") or shndx == 0 or shndx >= shnum:
                continue
            sec = secs[shndx]
            fo = sec[4] + (value - sec[3])
            out[name[:-3]] = blob[fo:fo + 64]
    return out


def test_every_padding_kernel_starts_its_wavefronts_in_the_same_state():
    """A merge_framework_<n> proxy jumps to the first instruction of another kernel of the code
    object, so all of them must ask the hardware for the same initial wavefront state: the same
    preloaded scalar registers (argument block address only, then the workgroup id x), no scratch,
    no hidden arguments, the same floating-point mode bits."""
    import struct
    from reef_amd.paths import code_object
    kds = _kernel_descriptors(code_object("trans"))
    assert len(kds) > 80 and "merge_framework_3" in kds and "reef_conv2d_d9_16x32k4" in kds
    ref = None
    for name, kd in sorted(kds.items()):
        group_seg, private_seg, kernarg = struct.unpack_from("<III", kd, 0)
        rsrc3, rsrc1, rsrc2 = struct.unpack_from("<III", kd, 44)
        props, preload = struct.unpack_from("<HH", kd, 56)
        state = {
            "private_segment": private_seg,
            "kernarg_size": kernarg,
            "float_mode_dx10_ieee": (rsrc1 >> 12) & 0xFFF & ~0x100,      # rounding, denormals, priv=0, dx10 clamp, debug, ieee
            "enable_private_segment": rsrc2 & 1,
            "user_sgpr_count": (rsrc2 >> 1) & 0x1F,
            "workgroup_id_xyz_info": (rsrc2 >> 7) & 0xF,
            "exceptions": rsrc2 >> 13,
            "kernel_code_properties": props,
            "kernarg_preload": preload,
            "tg_split": (rsrc3 >> 16) & 1,
        }
        if ref is None:
            ref = state
            # argument block address in s[0:1] is the only user register; workgroup id x follows in s2
            assert state["user_sgpr_count"] == 2 and state["kernel_code_properties"] == 0x8
            assert state["workgroup_id_xyz_info"] == 1 and state["private_segment"] == 0
            assert state["kernarg_size"] == 424 and state["kernarg_preload"] == 0
        assert state == ref, (name, state, ref)
        if name.startswith("merge_framework_"):
            assert group_seg == 0, name     # LDS of a merged launch is all dynamic, from offset 0


def check_kernels(path):
    ok, why = B.check_model(path)
    return (0 if ok else 1), why


def test_every_generated_kernel_fits_its_storages(tmp_path):
    """What the executors check at load time: the shape attributes of each kernel against the
    storages it is given and its grid.  Every network of the generator passes, views included."""
    from reef_amd.modelgen import nets
    graphs = [nets.resnet(50, image=(3, 64, 64), classes=16, name="r50"),
              nets.densenet(image=(3, 64, 64), classes=16, name="d"),
              nets.mobilenet_v2(image=(3, 64, 64), classes=16, name="mb"),
              nets.inception_v3(image=(3, 107, 107), classes=16, name="inc"),
              nets.bert(layers=2, hidden=128, heads=2, seq=48, ffn=256, vocab=100, name="bert", attention_mask=True),
              nets.bert(layers=1, hidden=128, heads=2, seq=48, ffn=256, vocab=100, name="bert3",
                        fused_attention=False),
              nets.mocked_kernel(name="mock")]
    for g in graphs:
        g.write(str(tmp_path), link_code_objects=False)
        st, why = check_kernels(tmp_path / (g.name + ".json"))
        assert st == 0, (g.name, why)


def test_kernels_that_do_not_fit_are_refused(tmp_path):
    """A graph file whose attributes ask for more than its storages hold, for another number of
    operands or for another grid is refused with a reason, by the check and by an executor that
    loads it (no launch is ever made from it)."""
    from reef_amd.modelgen import nets
    from tests.fakehal import FakeHal
    g = nets.bert(layers=1, hidden=128, heads=2, seq=48, ffn=256, vocab=100, name="b", attention_mask=True)
    g.write(str(tmp_path))
    good = json.load(open(tmp_path / "b.json"))
    by_symbol = {}
    for i, k in enumerate(good["kernels"]):
        by_symbol.setdefault(k["name"].split("#")[0].rsplit("_", 1)[0] if k["name"].startswith("reef_gemm") else
                             k["name"].split("#")[0], i)
    at, ln, gm = by_symbol["reef_attention"], by_symbol["reef_layernorm"], by_symbol["reef_gemm_ntd"]

    def broken(edit):
        m = json.loads(json.dumps(good))
        edit(m)
        p = tmp_path / "x.json"
        p.write_text(json.dumps(m))
        return p

    def shrink(m):       # the output of the attention loses its last element
        m["storage"][m["kernels"][at]["args"][1]]["size"] -= 1

    def longer(m):       # more key positions than the kernel can stage
        m["kernels"][at]["attrs"][0] = 129

    def grid(m):         # one workgroup too many
        m["kernels"][ln]["launch_params"][0] += 1

    def operand(m):      # the residual flag without a residual operand
        k = m["kernels"][ln]
        k["attrs"][2] ^= 1
        if not k["attrs"][2] & 1:
            k["args"].append(k["args"][0])

    def offset(m):       # a matrix that starts so late that its last row leaves the storage
        m["kernels"][gm]["attrs"][17] += 4

    def view(m):         # the same through an operand view
        k = m["kernels"][ln]
        k["arg_offsets"] = [16] + [0] * (len(k["args"]) - 1)

    for edit, word in ((shrink, "context"), (longer, "staging"), (grid, "workgroups"), (operand, "operands"),
                       (offset, "needs"), (view, "input")):
        p = broken(edit)
        st, why = check_kernels(p)
        assert st != 0 and word in why, (edit.__name__, st, why)
    # a convolution under a symbol that was compiled for another filter, and splits that stop short
    r = nets.resnet(18, image=(3, 32, 32), classes=8, name="r")
    r.write(str(tmp_path), link_code_objects=False)
    good_b, good = good, json.load(open(tmp_path / "r.json"))
    ci = next(i for i, k in enumerate(good["kernels"]) if k["name"].startswith("reef_conv2d_d1_"))

    def family(m):
        k = m["kernels"][ci]
        k["name"] = k["name"].replace("reef_conv2d_d1_", "reef_conv2d_d9_")

    def chunk(m):
        a = m["kernels"][ci]["attrs"]
        a[16] = a[0] * a[6] * a[7] // (2 * a[15])       # each split takes half of its share of K

    for edit, word in ((family, "loader family"), (chunk, "cover")):
        st, why = check_kernels(broken(edit))
        assert st != 0 and word in why, (edit.__name__, st, why)
    good = good_b
    # and the executor refuses the file
    fake = FakeHal().install()
    try:
        exe = B.Executor(B.BASE)
        exe.load(str(tmp_path / "b.json"), str(tmp_path / "b.raw.co"))      # the file as generated loads
        del exe
        with pytest.raises(B.ReefError, match="OutOfRange"):
            B.Executor(B.BASE).load(str(broken(shrink)), str(tmp_path / "b.raw.co"))
    finally:
        fake.remove()


def test_a_pointwise_plus_depthwise_kernel_is_checked_against_its_storages(tmp_path):
    """reef_conv2d_xdw_<tile>: operand list, sizes and tile counts follow from the attributes; a graph
    file that disagrees is refused with the reason."""
    from reef_amd import binding as B
    g = MB.GraphBuilder("xdwfmt")
    x = g.input("data", (24, 20, 30))
    g.mark_output(g.conv2d_dw(x, 48))
    base = g.write(str(tmp_path / "ok"), link_code_objects=False)
    assert B.check_model(base + ".json") == (True, "")
    model = json.load(open(base + ".json"))
    k = model["kernels"][0]
    assert k["name"].startswith("reef_conv2d_xdw_g2") and len(k["args"]) == 6

    def broken(change, reason):
        m = json.loads(json.dumps(model))
        change(m)
        p = str(tmp_path / "broken.json")
        json.dump(m, open(p, "w"))
        ok, why = B.check_model(p)
        assert not ok and reason in why, why

    broken(lambda m: m["kernels"][0]["args"].pop(), "operands")                         # no depthwise bias
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(18, 7), "loader family")      # wrong tile count
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(12, 1), "loader family")      # flag missing
    broken(lambda m: m["storage"][m["kernels"][0]["args"][4]].__setitem__("size", 48 * 8), "depthwise weights")
    broken(lambda m: m["kernels"][0]["launch_params"].__setitem__(0, 5), "workgroups")


def test_a_whole_block_kernel_is_checked_against_its_storages(tmp_path):
    """reef_conv2d_sdp_<tile> / reef_conv2d_xdp2_<tile>: eight operands, the output sized by the
    projection's channels (carried in the counter slot, which such a launch does not use), the
    limits of the two forms; a graph file that disagrees is refused with the reason."""
    from reef_amd import binding as B
    g = MB.GraphBuilder("blkfmt")
    x = g.input("data", (3, 30, 44))
    y = g.conv2d_block(x, 32, 16, front="stem")
    g.mark_output(g.conv2d_block(y, 96, 24, front="expand"))
    base = g.write(str(tmp_path / "ok"), link_code_objects=False)
    assert B.check_model(base + ".json") == (True, "")
    model = json.load(open(base + ".json"))
    k0, k1 = model["kernels"]
    assert k0["name"].startswith("reef_conv2d_sdp_g4") and k1["name"].startswith("reef_conv2d_xdp2_g1")
    assert len(k0["args"]) == 8 and k0["attrs"][20] == 16 and k1["attrs"][20] == 24
    assert model["storage"][k1["args"][2]]["size"] == 24 * 8 * 11
    assert not MB.GraphBuilder.block_fits("expand", 16, 96, 24, 45)         # odd width
    assert not MB.GraphBuilder.block_fits("expand", 24, 144, 32, 56)        # too many channels for one workgroup
    assert not MB.GraphBuilder.block_fits("stem", 3, 30, 16, 224)           # middle channels not in fours

    def broken(change, reason):
        m = json.loads(json.dumps(model))
        change(m)
        p = str(tmp_path / "broken.json")
        json.dump(m, open(p, "w"))
        ok, why = B.check_model(p)
        assert not ok and reason in why, why

    broken(lambda m: m["kernels"][0]["args"].pop(), "operands")                         # no projection bias
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(20, 40), "loader family")     # more than 32 output channels
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(12, 1 | 128), "loader family")  # projection flag missing
    broken(lambda m: m["kernels"][1]["attrs"].__setitem__(17, 6), "loader family")      # a workgroup holds every channel
    broken(lambda m: m["storage"][m["kernels"][1]["args"][6]].__setitem__("size", 24 * 90), "projection weights")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][2]].__setitem__("size", 15 * 15 * 22), "output")
    broken(lambda m: m["kernels"][1]["launch_params"].__setitem__(0, 5), "workgroups")


def test_a_product_behind_a_layernorm_is_checked_against_its_storages(tmp_path):
    """reef_gemm_ntl_<tile> and the residual of a matrix product: operand list and sizes follow from
    the flags; the LayerNorm flag belongs to the kernels named ntl and to no other."""
    from reef_amd import binding as B
    g = MB.GraphBuilder("ntlfmt")
    x = g.input("x", (40, 200))
    r = g.input("r", (40, 96))
    w = g.param((96, 200), 0.05)
    b = g.param((96,), 0.05)
    gamma, beta = g.layernorm_params(200)
    normed = g.temp((40, 200))
    y = g.gemm(x, w, 40, 96, 200, trans_b=True, bias=b, res=r, ln=dict(gamma=gamma, beta=beta, out=normed))
    g.mark_output(y)
    base = g.write(str(tmp_path / "ok"), link_code_objects=False)
    assert B.check_model(base + ".json") == (True, "")
    model = json.load(open(base + ".json"))
    k = model["kernels"][0]
    # A, W gamma, C, bias, residual, c1, c2, gamma, beta, A'
    assert k["name"].startswith("reef_gemm_ntl_32x32k4") and len(k["args"]) == 10 and k["attrs"][5] == 1 | 2 | 4 | 8
    # the three derived tensors are what their definitions say
    par = dict(g.params)
    gm, bt = (par[model["storage"][k["args"][i]]["name"]].astype(np.float64) for i in (7, 8))
    W = par[model["storage"][k["args"][1]]["name"][:-2]].astype(np.float64).reshape(96, 200)
    Wg, c1, c2 = (par[model["storage"][k["args"][i]]["name"]] for i in (1, 5, 6))
    np.testing.assert_array_equal(Wg.reshape(96, 200), (W * gm[None, :]).astype(np.float32))
    np.testing.assert_allclose(c1, (W * gm[None, :]).sum(1), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(c2, W @ bt, rtol=1e-6, atol=1e-7)
    assert all(model["storage"][k["args"][i]]["name"].endswith("k") for i in (1, 5, 6))

    def broken(change, reason):
        m = json.loads(json.dumps(model))
        change(m)
        p = str(tmp_path / "broken.json")
        json.dump(m, open(p, "w"))
        ok, why = B.check_model(p)
        assert not ok and reason in why, why

    broken(lambda m: m["kernels"][0]["args"].pop(), "operands")                               # no A'
    broken(lambda m: m["kernels"][0]["attrs"].pop(), "epsilon")
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(5, 1 | 8), "contradict")            # ntl without the flag
    broken(lambda m: m["kernels"][0].__setitem__("name", "reef_gemm_nt_32x32k4#0"), "contradict")
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(17, 4), "without offset")           # offA
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(3, 1 << 17), "65536")               # K
    broken(lambda m: m["storage"][m["kernels"][0]["args"][4]].__setitem__("size", 40 * 95), "residual")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][5]].__setitem__("size", 95), "column sums")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][7]].__setitem__("size", 199), "gamma")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][9]].__setitem__("size", 39 * 200), "normalised A")



def test_a_matrix_product_with_k_split_across_workgroups_is_checked(tmp_path):
    """reef_gemm_ntd_<tile> with split_k: two more operands (workspace, counters), split_k times
    the workgroups, chunks that are multiples of 128 and cover K."""
    from reef_amd import binding as B
    g = MB.GraphBuilder("splitfmt")
    x = g.input("x", (40, 520))
    w = g.param((96, 520), 0.05)
    g.mark_output(g.gemm(x, w, 40, 96, 520, trans_b=True, force_tile="16x32k4", split_k=2))
    base = g.write(str(tmp_path / "ok"), link_code_objects=False)
    assert B.check_model(base + ".json") == (True, "")
    model = json.load(open(base + ".json"))
    k = model["kernels"][0]
    assert k["attrs"][20:] == [0, 2, 384, 0] and k["attrs"][5] == 16 and len(k["args"]) == 5
    assert k["launch_params"][0] == 2 * 3 * 3

    def broken(change, reason):
        m = json.loads(json.dumps(model))
        change(m)
        p = str(tmp_path / "broken.json")
        json.dump(m, open(p, "w"))
        ok, why = B.check_model(p)
        assert not ok and reason in why, why

    broken(lambda m: m["kernels"][0]["args"].pop(), "operands")
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(22, 256), "cover K")
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(22, 300), "multiples of 128")
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(21, 3), "pair fold")
    broken(lambda m: m["kernels"][0].__setitem__("name", "reef_gemm_nt_32x32k4#0"), "only the direct kernels")
    broken(lambda m: m["kernels"][0]["launch_params"].__setitem__(0, 9), "workgroups")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][3]].__setitem__("size", 2 * 40 * 96 * 4), "workspace")


def test_a_stem_kernel_is_checked_against_its_storages(tmp_path):
    """reef_conv2d_sp7_g2: the output sizes are the pooled ones, the operand list follows the flags,
    and the kernel is only for 7x7 / stride 2 / padding 3 filters on at most three channels."""
    from reef_amd import binding as B
    g = MB.GraphBuilder("sp7fmt")
    x = g.input("data", (3, 37, 45))
    g.mark_output(g.conv2d_pool(x, 24, in_shift=True, pool_shift=True, pool_act=MB.ACT_RELU))
    base = g.write(str(tmp_path / "ok"), link_code_objects=False)
    assert B.check_model(base + ".json") == (True, "")
    model = json.load(open(base + ".json"))
    k = model["kernels"][0]
    a = k["attrs"]
    assert k["name"].startswith("reef_conv2d_sp7_g2") and len(k["args"]) == 6
    assert a[4:6] == [10, 12] and a[12] == 1 | 256 | 512 | 1024 and a[17:19] == [2, 5] and k["launch_params"][0] == 10

    def broken(change, reason):
        m = json.loads(json.dumps(model))
        change(m)
        p = str(tmp_path / "broken.json")
        json.dump(m, open(p, "w"))
        ok, why = B.check_model(p)
        assert not ok and reason in why, why

    broken(lambda m: m["kernels"][0]["args"].pop(), "operands")                              # no pool shift
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(4, 19), "output size")             # the convolution's rows, not the pooled
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(8, 1), "output size")              # stride 1
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(12, 1 | 256 | 2), "loader family") # a residual is not supported
    broken(lambda m: m["kernels"][0]["attrs"].__setitem__(18, 4), "loader family")           # wrong tile count
    broken(lambda m: m["kernels"][0].__setitem__("name", "reef_conv2d_u_64x32k2#0"), "loader family")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][2]].__setitem__("size", 24 * 10 * 11), "output")
    broken(lambda m: m["storage"][m["kernels"][0]["args"][4]].__setitem__("size", 2), "input shift")
