"""Writes resnet152_kernel_shapes.json: for every kernel name of the reference's
resource/resnet152 model what it computes -- op, shape, stride, padding, epilogue.

The generated kernels have their shapes baked into the source and the graph JSON only holds
shared, maximal buffer sizes, so the shapes are found from what the kernels DO: each distinct
convolution kernel of oracle/_ref/resnet152.raw.co (the reference's own resnet152.cu compiled for
gfx950, `make -C oracle ref`) is run once on random operands on the GPU, and of the few
(Cout, Cin, k, H, stride) that are consistent with its operand sizes exactly the right one makes
the CPU oracle reproduce its output (the same search as tests/test_gpu_reference_kernels.py).
The remaining kernels follow from the operand sizes and from walking the graph with the shapes
found so far.  One kernel of the reference (fused_nn_conv2d_add_nn_relu_8_kernel0) is not a
convolution as checked in (see the module docstring of tests/test_gpu_reference_kernels.py); its
shape is taken from its place in the graph and the entry is marked "witness": false.

Needs a GPU:  python tests/golden/make_resnet152_shapes.py [out.json]
The result is committed as tests/golden/resnet152_kernel_shapes.json (fixture) and as
reef_amd/legacy_tables/resnet152.json (the importer's table for this model directory)."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import oracle as O                                   # noqa: E402
from reef_amd import binding as B                                # noqa: E402
from tests import test_gpu_reference_kernels as T                # noqa: E402

EPILOGUE = {"fused_nn_conv2d": "none", "fused_nn_conv2d_add": "residual",
            "fused_nn_conv2d_add_nn_relu": "bias_relu",
            "fused_nn_conv2d_add_add_nn_relu": "residual_bias_relu",
            "fused_nn_conv2d_add_multiply_add_nn_relu": "residual_scale_shift_relu"}


def family(name):
    return name.split("_kernel0")[0].rstrip("0123456789").rstrip("_")


def search_convs(model, roles, exe):
    rng = np.random.default_rng(152)
    found = {}
    for kidx in T.distinct_kernels(model, "fused_nn_conv2d"):
        name = model["kernels"][kidx]["name"]
        ops, out, n_written = T.run_reference_kernel(exe, model, roles, kidx, rng)
        x, w = ops["placeholder"], ops["placeholder1"]
        extras = [ops[n] for n in roles[name] if n.startswith("placeholder") and n not in ("placeholder", "placeholder1")]
        fam = family(name)
        small = [e for e in extras if e.size < n_written]
        for cout, cin, kk, H, s, p in T.conv_hypotheses(x.size, w.size, n_written, small[0].size if small else 0):
            Ho = (H + 2 * p - kk) // s + 1
            xs = x[:cin * H * H].reshape(cin, H, H)
            ws = w[:cout * cin * kk * kk].reshape(cout, cin, kk, kk)
            kw = dict(stride=(s, s), pad=(p, p), act=1 if fam.endswith("nn_relu") else 0, acc64=True)
            full = [e[:cout * Ho * Ho].reshape(cout, Ho, Ho) for e in extras if e.size >= n_written]
            ep = EPILOGUE[fam]
            if ep == "none":
                want = O.conv2d(xs, ws, **kw)
            elif ep == "residual":
                want = O.conv2d(xs, ws, residual=full[0], **kw)
            elif ep == "bias_relu":
                want = O.conv2d(xs, ws, bias=small[0], **kw)
            elif ep == "residual_bias_relu":
                want = O.conv2d(xs, ws, residual=full[0], bias=small[0], **kw)
            else:
                want = O.conv2d(xs, ws, residual=full[0], scale=small[0], shift=small[1], **kw)
            if T.close(out[:n_written], want):
                found[name] = {"op": "conv2d", "cin": cin, "h": H, "w": H, "cout": cout, "k": kk, "stride": s,
                               "pad": p, "epilogue": ep, "witness": True}
                break
    return found


def walk(model, table):
    """Shapes of the storages in execution order; fills what the search left open."""
    size = lambda i: model["storage"][i]["size"]
    shape = {0: (3, 64, 64)}
    pending = None          # (name, output storage) of a convolution whose stride is still open
    for k in model["kernels"]:
        name, a = k["name"], k["args"]
        if name.startswith("fused_nn_conv2d"):
            if pending and pending[1] == a[0]:
                # the consumer of the open convolution tells its output height
                e = table[pending[0]]
                e["stride"] = 1 if table[name]["h"] == e["h"] else 2
                Ho = (e["h"] + 2 * e["pad"] - e["k"]) // e["stride"] + 1
                assert Ho == table[name]["h"], (pending, name)
                shape[a[0]] = (e["cout"], Ho, Ho)
                pending = None
            cin, H, W = shape[a[0]]
            if name not in table:
                ep = EPILOGUE[family(name)]
                cout = size(a[3]) if ep == "bias_relu" else None
                assert cout, name
                kk = int(round((size(a[1]) // (cout * cin)) ** 0.5))
                assert cout * cin * kk * kk == size(a[1])
                table[name] = {"op": "conv2d", "cin": cin, "h": H, "w": W, "cout": cout, "k": kk, "stride": 0,
                               "pad": kk // 2, "epilogue": ep, "witness": False}
                pending = (name, a[2])
                shape[a[2]] = None
                continue
            e = table[name]
            assert (e["cin"], e["h"], e["w"]) == (cin, H, W), (name, e, shape[a[0]])
            Ho = (H + 2 * e["pad"] - e["k"]) // e["stride"] + 1
            shape[a[2]] = (e["cout"], Ho, Ho)
        elif name.startswith("fused_add"):                      # (out, in, per-channel shift)
            C, H, W = shape[a[1]]
            assert size(a[2]) == C
            table.setdefault(name, {"op": "eltwise", "c": C, "inner": H * W, "shift": True,
                                    "act": 1 if "nn_relu" in name else 0})
            assert table[name]["c"] == C and table[name]["inner"] == H * W, name
            shape[a[0]] = (C, H, W)
        elif name.startswith("fused_nn_max_pool2d_add_nn_relu"):   # (in, out, bias)
            C, H, W = shape[a[0]]
            table.setdefault(name, {"op": "pool2d", "c": C, "h": H, "w": W, "k": 3, "stride": 2, "pad": 1,
                                    "mode": "max", "bias": True, "act": 1})
            shape[a[1]] = (C, (H + 2 - 3) // 2 + 1, (W + 2 - 3) // 2 + 1)
        elif name.startswith("fused_nn_global_avg_pool2d"):        # (in, out)
            C, H, W = shape[a[0]]
            table.setdefault(name, {"op": "global_avgpool", "c": C, "hw": H * W})
            shape[a[1]] = (C, 1, 1)
        elif name.startswith("fused_nn_batch_flatten"):            # (out, in)
            C = shape[a[1]][0]
            table.setdefault(name, {"op": "copy", "n": C})
            shape[a[0]] = (C, 1, 1)
        elif name.startswith("fused_nn_dense_add"):                # (x, W, out, bias)
            in_f, out_f = shape[a[0]][0], size(a[3])
            assert size(a[1]) == in_f * out_f
            table.setdefault(name, {"op": "dense", "in": in_f, "out": out_f, "bias": True})
            shape[a[2]] = (out_f, 1, 1)
        elif name.startswith("fused_nn_softmax"):                  # (in, out)
            table.setdefault(name, {"op": "softmax", "rows": 1, "cols": shape[a[0]][0]})
            shape[a[1]] = shape[a[0]]
        else:
            raise AssertionError("unexpected kernel " + name)
    assert pending is None
    return table


def main():
    out_path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "resnet152_kernel_shapes.json")
    model = json.load(open(os.path.join(HERE, "resnet152.json")))
    roles = json.load(open(os.path.join(HERE, "resnet152_kernel_roles.json")))
    exe = B.Executor(B.BASE)
    exe.load(os.path.join(HERE, "resnet152.json"), T.REF_CO)
    table = walk(model, search_convs(model, roles, exe))
    names = {k["name"] for k in model["kernels"]}
    assert set(table) == names, names ^ set(table)
    json.dump(table, open(out_path, "w"), indent=0, sort_keys=True)
    print(len(table), "kernels ->", out_path, "; without a witness:",
          [n for n, e in table.items() if not e.get("witness", True)])


if __name__ == "__main__":
    main()
