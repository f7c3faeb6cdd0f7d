"""Writes <model>_kernel_shapes.json for model directories of the reference whose graph can be
walked from the input with every kernel witnessed on the way:

  mobilenet  MobileNet v1 with depthwise convolutions, 224 x 224
  alexnet    11x11 / 5x5 / 3x3 convolutions without bias, plain max-pools, three dense layers
  vgg        despite its name a pre-activation ResNet-50 at 64 x 64 (kernel names carry TVM's
             `tvmgen_default_` prefix): the residual families of resnet152
  resnet18   pre-activation ResNet-18 at 224 x 224 whose 3x3 stride-1 convolutions are Winograd
             triples (kernel0: input transform, kernel1: GEMMs, kernel2: inverse transform +
             epilogue) on TRANSFORMED weights
  inception  Inception-v3 at 299 x 299: 1x7 / 7x1 / 1x3 / 3x1 / 5x5 filters, Winograd triples with
             and without padding, average pools, channel concatenations
  bert       a 6-layer transformer encoder (hidden 480, 12 heads of 40, sequence 480).  Its shapes
             follow from the storage sizes; what each kernel computes is witnessed by
             tests/test_gpu_reference_kernels.py::test_reference_bert_kernels_match_oracle, which
             this script runs before it writes the table (LayerNorm and softmax are chains of
             five calls each there; the table marks the calls that only carry a chain forward)

For every kernel name: what it computes -- op, shape, filter, stride, padding, epilogue.  The
shapes are baked into the generated source and the graph JSON only holds shared, maximal buffer
sizes, so every entry has a witness: the graph is walked from the input, each distinct kernel of
oracle/_ref/<model>.raw.co (the reference's own <model>.cu compiled for gfx950, `make -C oracle
ref`) is run once on random operands on the GPU, and of the hypotheses that are consistent with
its operand sizes and with the number of elements it writes (groups 1 or depthwise, square
filters 1..11 and 1xk / kx1, stride 1/2/4, every padding up to half the filter) exactly one must make the CPU oracle reproduce
its output.  The epilogue follows from the family name (resnet152.cu:315-363, 376-713, 2662: add =
residual when the operand is a tensor of the graph, bias when it is a parameter).  Dense kernels
are run on small non-negative integers and softmax has no witness, for the reason given in the
module docstring of tests/test_gpu_reference_kernels.py.

A Winograd triple is witnessed as one: a random direct filter g is transformed with
reef_amd.legacy.winograd_transform (output tile 4 or 2, weight layout [e][n][Cin][Cout] or
[e][n][Cout][Cin]), the reference's three kernels run on it, and exactly one hypothesis must give
what the oracle's DIRECT convolution of g gives (to 1e-4 of the largest output: two summation
orders and the transform's own rounding).  That pins the transform matrix the importer inverts.

Needs a GPU:  python tests/golden/make_graph_shapes.py mobilenet|alexnet|vgg|resnet18|inception|bert
The result is committed as tests/golden/<model>_kernel_shapes.json (fixture) and as
reef_amd/legacy_tables/<model>.json (the importer's table for that model directory)."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import oracle as O                                   # noqa: E402
from reef_amd import binding as B                                # noqa: E402
from reef_amd import legacy                                      # noqa: E402
from tests import test_gpu_reference_kernels as T                # noqa: E402

WINO = "fused_nn_contrib_conv2d_winograd_without_weight_transform"
EPILOGUE = {"fused_nn_conv2d": "none", "fused_nn_conv2d_nn_relu": "relu",
            "fused_nn_conv2d_add": "residual", "fused_nn_conv2d_add_nn_relu": "bias_relu",
            "fused_nn_conv2d_add_add_nn_relu": "residual_bias_relu",
            "fused_nn_conv2d_add_multiply_add_nn_relu": "residual_scale_shift_relu"}


def plain(name):
    return name[len("tvmgen_default_"):] if name.startswith("tvmgen_default_") else name


def family(name):
    return plain(name).split("_kernel0")[0].rstrip("0123456789").rstrip("_")


def winograd_family(name):
    """Epilogue family of a Winograd kernel2 name, as the direct convolutions spell it.  TVM cuts
    long names and appends a hash (`..._add_multiply_add_nn_re_<digits>__kernel2`)."""
    rest = plain(name)[len(WINO):].split("_kernel")[0].rstrip("_")
    if rest.startswith("_add_multiply_add_nn_re"):
        return "fused_nn_conv2d_add_multiply_add_nn_relu"
    return "fused_nn_conv2d" + rest.rstrip("0123456789").rstrip("_")


def witness_winograd(exe, model, roles, params, src, kidx, cin, H, W, rng):
    """Runs the triple (src["k0"], src["k1"], kidx) under every hypothesis; returns the table entry."""
    k = model["kernels"][kidx]
    kname, a = k["name"], k["args"]
    size = lambda i: model["storage"][i]["size"]
    ep = EPILOGUE[winograd_family(kname)]
    relu = ep.endswith("relu")
    names = roles[kname]
    assert names[0] == "bgemm" and names[1].startswith("T_") and all(n.startswith("placeholder") for n in names[2:]), names
    hits = []
    for tile in (4, 2):
        alpha = tile + 2
        if size(src["U"]) % (alpha * alpha * cin):
            continue
        cout = size(src["U"]) // (alpha * alpha * cin)
        for layout, pad in (("enio", 1), ("enoi", 1), ("enio", 0), ("enoi", 0)):
            Ho, Wo = H + 2 * pad - 2, W + 2 * pad - 2
            g = (rng.standard_normal((cout, cin, 3, 3)) * np.sqrt(2.0 / (cin * 9))).astype(np.float32)
            U = legacy.winograd_transform(g, tile)
            T._set(exe, model, src["U"], U if layout == "enio" else U.transpose(0, 1, 3, 2))
            x = T._set(exe, model, src["in"], rng.standard_normal(size(src["in"])).astype(np.float32))
            small, full = [], []
            for s_idx in a[2:]:
                v = T._set(exe, model, s_idx, rng.standard_normal(size(s_idx)).astype(np.float32))
                (small if s_idx in params else full).append(v)
            T._set(exe, model, a[1], np.full(size(a[1]), T.SENTINEL, np.float32))
            for i in (src["k0"], src["k1"], kidx):
                exe.execute_kernel(i)
            out = exe.get_data(a[1], size(a[1]))
            written = np.nonzero(out != T.SENTINEL)[0]
            n = int(written.max()) + 1 if written.size else 0
            if n != cout * Ho * Wo or written.size != n or (small and small[0].size != cout):
                continue
            kw = dict(stride=(1, 1), pad=(pad, pad), act=1 if relu else 0, acc64=True)
            if full:
                kw["residual"] = full[0][:n].reshape(cout, Ho, Wo)
            if ep == "residual_scale_shift_relu":
                kw.update(scale=small[0], shift=small[1])
            elif small:
                kw["bias"] = small[0]
            want = O.conv2d(x[:cin * H * W].reshape(cin, H, W), g, **kw)
            dev = float(np.abs(out[:n] - want.ravel()).max()) / max(float(np.abs(want).max()), 1.0)
            print("    tile %d layout %s pad %d: deviation %.2e" % (tile, layout, pad, dev), flush=True)
            if dev <= 1e-4:
                hits.append((tile, layout, cout, pad))
    assert len(hits) == 1, (kname, hits)
    tile, layout, cout, pad = hits[0]
    assert layout == "enio", "the importer assumes [e][n][Cin][Cout]"
    return {"op": "conv2d", "cin": cin, "h": H, "w": W, "cout": cout, "k": 3, "stride": 1, "pad": pad,
            "epilogue": ep, "winograd_tile": tile, "witness": True}


FILTERS = [(1, 1), (3, 3), (5, 5), (7, 7), (11, 11), (1, 3), (3, 1), (1, 7), (7, 1)]


def conv_hypotheses(cin, H, W, w_size, cout_known, n_written):
    seen = set()
    for groups in (1, cin):
        for kh, kw in FILTERS:
            per = (cin // groups) * kh * kw
            if w_size % per:
                continue
            cout = w_size // per
            if (cout_known and cout != cout_known) or (groups > 1 and cout != cin):
                continue
            for s in (1, 2, 4):
                for ph in range(kh // 2 + 1):
                    for pw in range(kw // 2 + 1):
                        if kh == kw and ph != pw:
                            continue
                        Ho, Wo = (H + 2 * ph - kh) // s + 1, (W + 2 * pw - kw) // s + 1
                        h = (cout, groups, (kh, kw), s, (ph, pw))
                        if Ho >= 1 and Wo >= 1 and cout * Ho * Wo == n_written and h not in seen:
                            seen.add(h)
                            yield h


def one_or_two(v):
    return v[0] if v[0] == v[1] else list(v)


def derive(name):
    path = os.path.join(HERE, name + ".json")
    model = json.load(open(path))
    roles = json.load(open(os.path.join(HERE, name + "_kernel_roles.json")))
    params = set(legacy.param_storages(model).values())
    exe = B.Executor(B.BASE)
    exe.load(path, os.path.join(ROOT, "oracle", "_ref", name + ".raw.co"))
    rng = np.random.default_rng(224)
    size = lambda i: model["storage"][i]["size"]
    side = int(round((size(0) // 3) ** 0.5))
    shape = {0: (3, side, side)}
    table = {}
    wino = {}
    for kidx, k in enumerate(model["kernels"]):
        kname, a = k["name"], k["args"]
        pname = plain(kname)
        new = kname not in table
        if pname.startswith(WINO) and pname.endswith("_kernel0"):      # (in, V)
            wino[a[1]] = {"in": a[0], "k0": kidx}
            table.setdefault(kname, {"op": "winograd_data", "witness": True})
        elif pname.startswith(WINO) and pname.endswith("_kernel1"):    # (U, V, M)
            wino[a[2]] = dict(wino.pop(a[1]), U=a[0], k1=kidx)
            table.setdefault(kname, {"op": "winograd_gemm", "witness": True})
        elif pname.startswith(WINO):                                    # (M, out, epilogue operands)
            src = wino.pop(a[0])
            cin, H, W = shape[src["in"]]
            if new:
                print(kname, flush=True)
                table[kname] = witness_winograd(exe, model, roles, params, src, kidx, cin, H, W, rng)
                print("%-60s %s" % (kname, table[kname]), flush=True)
            e = table[kname]
            assert (e["cin"], e["h"], e["w"]) == (cin, H, W), kname
            shape[a[1]] = (e["cout"], H + 2 * e["pad"] - 2, W + 2 * e["pad"] - 2)
        elif pname.startswith("fused_nn_conv2d"):
            cin, H, W = shape[a[0]]
            if new:
                ep = EPILOGUE[family(kname)]
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                x, w = ops["placeholder"], ops["placeholder1"]
                extra = [(ops[r], s_idx in params) for r, s_idx in zip(roles[kname], a)
                         if r.startswith("placeholder") and r not in ("placeholder", "placeholder1")]
                small = [e for e, is_param in extra if is_param]
                full = [e for e, is_param in extra if not is_param]
                assert (len(full), len(small)) == {"none": (0, 0), "relu": (0, 0), "residual": (1, 0),
                                                   "bias_relu": (0, 1), "residual_bias_relu": (1, 1),
                                                   "residual_scale_shift_relu": (1, 2)}[ep], (kname, ep)
                relu = ep.endswith("relu")
                hits = []
                for cout, groups, (kh, kwid), s, (ph, pw) in conv_hypotheses(cin, H, W, w.size,
                                                                             small[0].size if small else 0, n):
                    Ho, Wo = (H + 2 * ph - kh) // s + 1, (W + 2 * pw - kwid) // s + 1
                    kw = dict(stride=(s, s), pad=(ph, pw), groups=groups, act=1 if relu else 0, acc64=True)
                    if full:
                        kw["residual"] = full[0][:cout * Ho * Wo].reshape(cout, Ho, Wo)
                    if ep == "residual_scale_shift_relu":
                        kw.update(scale=small[0], shift=small[1])
                    elif small:
                        kw["bias"] = small[0]
                    want = O.conv2d(x[:cin * H * W].reshape(cin, H, W), w.reshape(cout, cin // groups, kh, kwid), **kw)
                    if T.close(out[:n], want):
                        hits.append((cout, groups, one_or_two((kh, kwid)), s, one_or_two((ph, pw))))
                assert len(hits) == 1, (kname, hits)
                cout, groups, kk, s, p = hits[0]
                if groups > 1:
                    assert ep == "bias_relu", kname
                    table[kname] = {"op": "dwconv2d", "c": cin, "h": H, "w": W, "k": kk, "stride": s, "pad": p,
                                    "bias": True, "act": 1, "witness": True}
                else:
                    table[kname] = {"op": "conv2d", "cin": cin, "h": H, "w": W, "cout": cout, "k": kk, "stride": s,
                                    "pad": p, "epilogue": ep, "witness": True}
                print("%-60s %s" % (kname, table[kname]), flush=True)
            e = table[kname]
            C = e["c"] if e["op"] == "dwconv2d" else e["cout"]
            assert (e["h"], e["w"]) == (H, W) and (e.get("cin", e.get("c")) == cin), kname
            (kh, kwid), (ph, pw) = legacy.pair(e["k"]), legacy.pair(e["pad"])
            shape[a[2]] = (C, (H + 2 * ph - kh) // e["stride"] + 1, (W + 2 * pw - kwid) // e["stride"] + 1)
        elif pname.startswith("fused_add"):                         # (out, in, per-channel shift)
            C, H, W = shape[a[1]]
            assert size(a[2]) == C, kname
            if new:
                act = 1 if "nn_relu" in pname else 0
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                assert n == C * H * W, kname
                want = O.eltwise(ops["placeholder"][:n].reshape(C, H * W), shift=ops["placeholder1"], act=act)
                assert T.close(out[:n], want), kname
                table[kname] = {"op": "eltwise", "c": C, "inner": H * W, "shift": True, "act": act, "witness": True}
                print("%-60s %s" % (kname, table[kname]), flush=True)
            assert table[kname]["c"] == C and table[kname]["inner"] == H * W, kname
            shape[a[0]] = (C, H, W)
        elif pname.startswith(("fused_nn_max_pool2d", "fused_nn_avg_pool2d")):   # (in, out[, bias])
            C, H, W = shape[a[0]]
            if new:
                mode = 0 if "max_pool" in pname else 1
                with_bias = "_add_nn_relu" in pname
                assert len(a) == (3 if with_bias else 2) and (not with_bias or size(a[2]) == C), kname
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                x = ops["placeholder"][:C * H * W].reshape(C, H, W)
                hits = []
                for kk, s, p in ((3, 2, 0), (3, 2, 1), (2, 2, 0), (3, 1, 1), (H, 1, 0)):
                    Ho = (H + 2 * p - kk) // s + 1
                    for cip in ((False, True) if mode == 1 and p else (False,)):
                        if C * Ho * Ho != n or (kk, s, p, cip) in hits:
                            continue
                        want = O.pool2d(x, (kk, kk), (s, s), (p, p), mode, count_include_pad=cip,
                                        bias=ops["placeholder1"] if with_bias else None, act=1 if with_bias else 0)
                        if T.close(out[:n], want):
                            hits.append((kk, s, p, cip))
                assert len(hits) == 1, (kname, hits)
                kk, s, p, cip = hits[0]
                table[kname] = {"op": "pool2d", "c": C, "h": H, "w": W, "k": kk, "stride": s, "pad": p,
                                "mode": "max" if mode == 0 else "avg", "bias": with_bias,
                                "act": 1 if with_bias else 0, "witness": True}
                if cip:
                    table[kname]["count_include_pad"] = True
                print("%-60s %s" % (kname, table[kname]), flush=True)
            e = table[kname]
            Ho = (H + 2 * e["pad"] - e["k"]) // e["stride"] + 1
            shape[a[1]] = (C, Ho, Ho)
        elif pname.startswith("fused_concatenate"):                 # (out, parts in SOME order)
            parts = [shape[i] for i in a[1:]]
            assert len({p[1:] for p in parts}) == 1 and a[0] not in a[1:], (kname, parts)
            H, W = parts[0][1:]
            if new:
                # which operand lands where is found from the data: at every offset exactly one of
                # the remaining operands is what the kernel wrote there
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                assert n == sum(p[0] for p in parts) * H * W, kname
                order, off, left = [], 0, list(range(len(parts)))
                while left:
                    fits = [j for j in left if np.array_equal(out[off:off + parts[j][0] * H * W],
                                                              ops[roles[kname][1 + j]][:parts[j][0] * H * W])]
                    assert len(fits) == 1, (kname, off, fits)
                    order.append(fits[0])
                    left.remove(fits[0])
                    off += parts[fits[0]][0] * H * W
                table[kname] = {"op": "concat", "parts": [parts[j][0] for j in order], "operand": order,
                                "h": H, "w": W, "witness": True}
                print("%-60s %s" % (kname, table[kname]), flush=True)
            e = table[kname]
            assert e["parts"] == [parts[j][0] for j in e["operand"]] and (e["h"], e["w"]) == (H, W), kname
            shape[a[0]] = (sum(p[0] for p in parts), H, W)
        elif pname.startswith("fused_nn_global_avg_pool2d"):        # (in, out)
            C, H, W = shape[a[0]]
            if new:
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                assert n == C and T.close(out[:n], O.global_avgpool(ops["placeholder"][:C * H * W].reshape(C, H * W)))
                table[kname] = {"op": "global_avgpool", "c": C, "hw": H * W, "witness": True}
            shape[a[1]] = (C, 1, 1)
        elif pname.startswith("fused_nn_batch_flatten"):            # (out, in)
            C, H, W = shape[a[1]]
            if new:
                ops, out, n = T.run_reference_kernel(exe, model, roles, kidx, rng)
                assert n == C * H * W and np.array_equal(out[:n], ops["placeholder"][:n])
                table[kname] = {"op": "copy", "n": n, "witness": True}
            shape[a[0]] = (C * H * W, 1, 1)
        elif pname.startswith("fused_nn_dense_add"):                # (x, W, out, bias)
            in_f, out_f = shape[a[0]][0], size(a[3])
            assert size(a[1]) == in_f * out_f
            if new:
                relu = "nn_relu" in pname
                ints = {}
                for pn, s_idx in zip(roles[kname], a):
                    if pn.startswith("placeholder"):
                        ints[pn] = T._set(exe, model, s_idx, rng.integers(0, 4, size(s_idx)).astype(np.float32))
                exe.execute_kernel(kidx)
                got = exe.get_data(a[2], size(a[2]))[:out_f]
                want = O.dense(ints["placeholder"][:in_f].reshape(1, in_f), ints["placeholder1"].reshape(out_f, in_f),
                               bias=ints["placeholder2"], act=1 if relu else 0, acc64=True)
                np.testing.assert_array_equal(got, want.ravel(), err_msg=kname)
                table[kname] = {"op": "dense", "in": in_f, "out": out_f, "bias": True, "act": 1 if relu else 0,
                                "witness": True}
            shape[a[2]] = (out_f, 1, 1)
        elif pname.startswith("fused_nn_softmax"):                  # (in, out)
            table.setdefault(kname, {"op": "softmax", "rows": 1, "cols": shape[a[0]][0], "witness": False})
            shape[a[1]] = shape[a[0]]
        else:
            raise AssertionError("unexpected kernel " + kname)
    assert set(table) == {k["name"] for k in model["kernels"]}
    exe.close()
    return table


def derive_bert():
    model = json.load(open(os.path.join(HERE, "bert.json")))
    size = lambda i: model["storage"][i]["size"]
    first = {}
    for k in model["kernels"]:
        first.setdefault(k["name"], k["args"])
    emb = first["fused_cast_take_broadcast_to_like_cast_take_add_1_kernel0"]      # (out, table, ids, positions, position ids)
    S = size(emb[2])
    H = size(first["fused_subtract_add_sqrt_divide_multiply_add_1_kernel0"][4])     # gamma
    assert size(first["fused_nn_batch_matmul_3_kernel0"][1]) == H * H
    heads, d = 12, 40           # grid z of fused_nn_batch_matmul_5 and the `% 40` of the head split (bert.cu)
    assert heads * d == H and size(first["fused_nn_softmax_1_kernel3"][0]) == heads * S * S
    T.test_reference_bert_kernels_match_oracle()         # every family below, on random operands
    scale = float(np.float32(1.0) / np.sqrt(np.float32(d)))
    table = {
        "fused_full_equal_reshape_kernel0": {"op": "mask_fill", "n": S},
        "fused_cast_take_broadcast_to_like_cast_take_add_1_kernel0":
            {"op": "embedding", "vocab": size(emb[1]) // H, "positions": size(emb[3]) // H, "seq": S, "hidden": H},
        "fused_mean_1_kernel0": {"op": "chain_stage", "input": 0, "result": 1},
        "fused_mean_1_kernel1": {"op": "chain_stage", "result": 0},
        "fused_variance_1_kernel0": {"op": "chain_stage", "input": 0, "result": 2},
        "fused_variance_1_kernel1": {"op": "chain_stage", "result": 0},
        "fused_subtract_add_sqrt_divide_multiply_add_1_kernel0": {"op": "layernorm", "rows": S, "cols": H, "eps": 1e-12},
        "fused_reshape_4_kernel0": {"op": "copy", "n": S * H},
        "fused_reshape_5_kernel0": {"op": "copy", "n": heads * S * S},
        "fused_nn_batch_matmul_3_kernel0": {"op": "gemm_nt", "batch": 1, "m": S, "n": H, "k": H},
        "fused_nn_batch_matmul_5_kernel0": {"op": "gemm_nt", "batch": heads, "m": S, "n": S, "k": d},
        "fused_nn_batch_matmul_4_kernel0": {"op": "gemm_nt", "batch": heads, "m": S, "n": d, "k": S},
        "fused_reshape_add_reshape_transpose_divide_reshape_kernel0":
            {"op": "rowbias_heads", "rows": S, "heads": heads, "d": d, "scale": scale},
        "fused_reshape_add_reshape_transpose_transpose_reshape_transpose_kernel0":
            {"op": "rowbias_heads", "rows": S, "heads": heads, "d": d},
        "fused_reshape_add_reshape_transpose_reshape_transpose_kernel0": {"op": "rowbias_transpose", "rows": H, "cols": S},
        "fused_reshape_transpose_copy_reshape_1_kernel0": {"op": "heads_merge", "heads": heads, "rows": S, "d": d},
        "fused_reshape_cast_broadcast_to_like_where_kernel0":
            {"op": "chain_stage", "input": 2, "mask": 1, "result": 0, "copy": heads * S * S},
        "fused_nn_softmax_1_kernel0": {"op": "chain_stage", "result": 0},
        "fused_nn_softmax_1_kernel1": {"op": "chain_stage", "result": 0},
        "fused_nn_softmax_1_kernel2": {"op": "chain_stage", "result": 0},
        "fused_nn_softmax_1_kernel3": {"op": "masked_softmax", "rows": heads * S, "cols": S},
        "fused_reshape_add_add_kernel0": {"op": "rowbias_add", "rows": H, "cols": S},
        "fused_reshape_add_multiply_erf_multiply_add_multiply_reshape_kernel0": {"op": "rowbias_gelu", "rows": H, "cols": S},
    }
    assert set(table) == {k["name"] for k in model["kernels"]}
    for e in table.values():
        e["witness"] = True
    return table


def main():
    name = sys.argv[1]
    table = derive_bert() if name == "bert" else derive(name)
    outs = [os.path.join(HERE, name + "_kernel_shapes.json"),
            os.path.join(ROOT, "reef_amd", "legacy_tables", name + ".json")]
    if os.environ.get("REEF_SHAPES_COPY_DIR"):      # a third copy, e.g. where results of a remote run are collected
        outs.append(os.path.join(os.environ["REEF_SHAPES_COPY_DIR"], name + "_kernel_shapes.json"))
    for out in outs:
        os.makedirs(os.path.dirname(out), exist_ok=True)
        json.dump(table, open(out, "w"), indent=0, sort_keys=True)
    print(len(table), "kernels; without a witness:", [n for n, e in table.items() if not e["witness"]])


if __name__ == "__main__":
    main()
