"""Importer for the reference's own model directories.

A directory written by the reference's TVM pipeline (`resource/<model>/<model>.json`,
script/generate_final_schedule.py:109-144) names one generated kernel per call
(`fused_nn_conv2d_add_nn_relu_3_kernel0`) whose shape is baked into its source; the graph file
holds the storages, the call order, the argument bindings and nothing about what a kernel
computes.  This build's kernels are generic, so a graph for them says what every call computes
(op, shape, epilogue) in the added keys `op` and `attrs`, which the reference's reader ignores
(src/reef/executor/model.cpp:23-51).

`import_model` rewrites such a graph: same storages (same indices, names, sizes -- including the
buffers the reference shares between layers), same call order, same parameter keys (a `.param`
file of the reference loads unchanged), every call replaced by the `reef_*` kernel that computes
the same thing.  What a kernel name computes comes from a per-model table
(`legacy_tables/<model>.json`: name -> op, shape, stride, padding, epilogue); the argument roles
are those of the kernel families (convolution: in, W, out, then the epilogue operands in the
order the family name lists them; depthwise convolution: in, W, out, bias; elementwise add,
flatten and concatenation: out first (TVM lists a concatenation's operands in an order of its own;
the table says which operand comes first in the result); pooling: in, out; dense: x, W, out, bias).  Tables are packaged for the
reference's `resnet152`, `mobilenet`, `alexnet`, `vgg` (which holds a pre-activation ResNet-50 at
64 x 64 under TVM's `tvmgen_default_` kernel names), `resnet18`, `inception` and `bert` directories.
While it rewrites, the importer follows the tensor shapes through the graph and refuses a table
that does not fit the graph.

Winograd convolutions.  TVM compiles some 3x3 stride-1 convolutions as three calls
(`fused_nn_contrib_conv2d_winograd_without_weight_transform*_kernel0/1/2`: transform of the input
tiles, one GEMM per transform point, inverse transform + epilogue) through two scratch storages,
and stores their weights TRANSFORMED: U[e][n][ci][co] = sum_rs G[e][r] g[co][ci][r][s] G[n][s],
(t+2)^2 values per filter for output tiles of t x t.  The importer replaces such a triple by one
direct convolution on the first call's input (the calls 0 and 1 get no counterpart; the scratch
storages stay, unused), whose weights live in an added storage `<key>_direct`; `convert_params`
recovers g from a parameter file's U (least squares through G's pseudo-inverse: exact for a U
that is a transform).  G is the Cook-Toom matrix of TVM's interpolation points, which the
reference does not vendor; it is pinned by running the reference's three kernels on a U made with
it against the direct convolution (tests/golden/make_graph_shapes.py).

The transformer directory (`bert`: hidden 480, 12 heads, sequence 480).  TVM splits a LayerNorm
into five calls (two for the mean, two for the variance, one that normalises) and a softmax into
four behind a call that applies the attention mask; this build has one kernel for each, so the
leading calls of such a chain get no counterpart and the last one becomes the whole operation on
the chain's input.  The calls that add a bias along the ROWS of a [480][480] tensor before they
split heads, transpose or apply GELU become a per-row add followed by the transpose / GELU
kernel through an added scratch storage.  The 1/sqrt(d) that the query's head split applies is
moved into the product of queries and keys that follows it (alpha of that GEMM): the query buffer
holds unscaled values here, every other storage holds what the reference's call leaves there.
"""
import json
import os
import struct

import numpy as np

from .modelgen import builder as MB
from .modelgen.builder import Tensor

TABLE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "legacy_tables")

# interpolation points of F(t x t, 3 x 3), the point at infinity comes last
WINOGRAD_POINTS = {2: (0.0, -1.0, 1.0), 4: (0.0, -1.0, 1.0, 0.5, -2.0)}


class ImportError_(ValueError):
    pass


def pair(v):
    """Filter size / padding of a table entry: one number for a square one, [rows, columns] else."""
    return (v, v) if isinstance(v, int) else (int(v[0]), int(v[1]))


def winograd_G(tile):
    """(tile + 2) x 3 filter transform: row i = (1, a_i, a_i^2) / prod_{k != i} (a_i - a_k) for the
    finite points (the first row's sign made positive), (0, 0, 1) for the point at infinity."""
    a = WINOGRAD_POINTS[tile]
    alpha = tile + 2
    G = np.zeros((alpha, 3))
    for i in range(alpha - 1):
        f = 1.0
        for k in range(alpha - 1):
            if k != i:
                f *= a[i] - a[k]
        if i == 0 and f < 0:
            f = -f
        G[i] = [1.0 / f, a[i] / f, a[i] * a[i] / f]
    G[alpha - 1] = (0.0, 0.0, 1.0)
    return G


def winograd_transform(g, tile):
    """g [Cout][Cin][3][3] -> U [t+2][t+2][Cin][Cout], float32 (computed in float64)."""
    G = winograd_G(tile)
    return np.einsum("er,oirs,ns->enio", G, np.asarray(g, np.float64), G).astype(np.float32)


def winograd_untransform(U, tile):
    """U [t+2][t+2][Cin][Cout] -> g [Cout][Cin][3][3]: the least-squares solution of U = G g G^T."""
    P = np.linalg.pinv(winograd_G(tile))
    return np.einsum("re,enio,sn->oirs", P, np.asarray(U, np.float64), P).astype(np.float32)


def load_table(model_name):
    path = os.path.join(TABLE_DIR, model_name + ".json")
    if not os.path.exists(path):
        raise ImportError_("no kernel table for model '%s' (%s)" % (model_name, path))
    return json.load(open(path))


def import_model(ref_json_path, table=None, name=None, input_shape=None):
    """Reference graph file -> GraphBuilder holding the same graph on this build's kernels.
    `table`: dict or path (default: the packaged table named after the file).  `input_shape`:
    (C, H, W) of storage 0 (default: 3 x s x s with s from its size)."""
    ref = json.load(open(ref_json_path))
    model_name = name or os.path.splitext(os.path.basename(ref_json_path))[0]
    if table is None:
        table = load_table(model_name)
    elif isinstance(table, str):
        table = json.load(open(table))
    g = MB.GraphBuilder(model_name)
    g.unique_names = True
    g.fused_reduce = True
    g.storage = [dict(s) for s in ref["storage"]]
    g.graph_args = list(ref.get("args", []))
    n0 = ref["storage"][0]["size"]
    if ref["storage"][0]["stype"] != "float32":
        input_shape = ()                                # token ids: the table says every shape
    if input_shape is None:
        side = int(round((n0 // 3) ** 0.5))
        if 3 * side * side != n0:
            raise ImportError_("cannot tell the input shape from %d elements; pass input_shape" % n0)
        input_shape = (3, side, side)
    shape = {0: tuple(input_shape)}
    cnn = len(shape[0]) == 3
    wino = {}               # scratch storage -> {"in": input storage[, "U": transformed weights]}
    g.direct_weights = {}   # key of a transformed weight -> (key of its direct copy, tile, Cout, Cin)
    direct_idx = {}
    g.imported_calls = []   # per kernel of this graph: the index of the reference call it replaces
    chain = {}              # storage a skipped call of a LayerNorm / softmax chain wrote -> what it stands for
    alpha_of = {}           # storage holding unscaled queries -> the factor its consumer applies

    def size(i):
        return g.storage[i]["size"]

    def need(cond, kernel, what):
        if not cond:
            raise ImportError_("%s: %s" % (kernel["name"], what))

    def tensor(i, shp, kernel):
        n = 1
        for d in shp:
            n *= d
        need(n <= size(i), kernel, "storage %d holds %d elements, the table asks for %s" % (i, size(i), shp))
        return Tensor(i, shp)

    for call, k in enumerate(ref["kernels"]):
        kname, a = k["name"], k["args"]
        e = table.get(kname)
        need(e is not None, k, "not in the table")
        op = e["op"]
        first_new = len(g.kernels)
        if op == "winograd_data":                               # (in, V)
            need(len(a) == 2 and a[0] in shape, k, "input storage has no shape yet")
            wino[a[1]] = {"in": a[0]}
        elif op == "winograd_gemm":                             # (U, V, M)
            need(len(a) == 3 and a[1] in wino, k, "no transformed input reaches this call")
            wino[a[2]] = dict(wino.pop(a[1]), U=a[0])
        elif op == "conv2d":
            tile = e.get("winograd_tile")
            if tile:                                            # (M, out, epilogue operands)
                need(len(a) >= 2 and "U" in wino.get(a[0], ()), k, "no transformed operands reach this call")
                need((e["k"], e["stride"]) == (3, 1) and e["pad"] in (0, 1), k,
                     "a Winograd entry is a 3x3 stride-1 filter")
                src = wino.pop(a[0])
                alpha = tile + 2
                need(size(src["U"]) == alpha * alpha * e["cin"] * e["cout"], k, "transformed weight storage size")
                if src["U"] not in direct_idx:
                    key = ref["storage"][src["U"]]["name"]
                    direct_idx[src["U"]] = g._storage(key + "_direct", e["cout"] * e["cin"] * 9)
                    g.graph_args.append(direct_idx[src["U"]])
                    g.direct_weights[key] = (key + "_direct", tile, e["cout"], e["cin"])
                a = [src["in"], direct_idx[src["U"]], a[1]] + list(a[2:])
            need(len(a) >= 3 and a[0] in shape, k, "input storage has no shape yet")
            need(shape[a[0]] == (e["cin"], e["h"], e["w"]), k,
                 "table says input %s, the graph delivers %s" % ((e["cin"], e["h"], e["w"]), shape[a[0]]))
            (fh, fw), s, (ph, pw), cout = pair(e["k"]), e["stride"], pair(e["pad"]), e["cout"]
            Ho, Wo = (e["h"] + 2 * ph - fh) // s + 1, (e["w"] + 2 * pw - fw) // s + 1
            need(size(a[1]) == cout * e["cin"] * fh * fw, k, "weight storage size")
            ep = e["epilogue"]
            rest = a[3:]
            given = {"w": Tensor(a[1], (cout, e["cin"], fh, fw))}
            kw = dict(bias=False, act=MB.ACT_NONE, residual=None, affine=False)
            if ep == "bias_relu":
                need(len(rest) == 1 and size(rest[0]) == cout, k, "bias operand")
                given["bias"] = Tensor(rest[0], (cout,))
                kw.update(bias=True, act=MB.ACT_RELU)
            elif ep == "residual":
                need(len(rest) == 1 and shape.get(rest[0]) == (cout, Ho, Wo), k, "residual operand")
                kw.update(residual=Tensor(rest[0], (cout, Ho, Wo)))
            elif ep == "residual_bias_relu":
                need(len(rest) == 2 and shape.get(rest[0]) == (cout, Ho, Wo) and size(rest[1]) == cout, k,
                     "residual / bias operands")
                given["bias"] = Tensor(rest[1], (cout,))
                kw.update(residual=Tensor(rest[0], (cout, Ho, Wo)), bias=True, act=MB.ACT_RELU)
            elif ep == "residual_scale_shift_relu":
                need(len(rest) == 3 and shape.get(rest[0]) == (cout, Ho, Wo) and size(rest[1]) == cout
                     and size(rest[2]) == cout, k, "residual / scale / shift operands")
                given["scale"], given["shift"] = Tensor(rest[1], (cout,)), Tensor(rest[2], (cout,))
                kw.update(residual=Tensor(rest[0], (cout, Ho, Wo)), affine=True, act=MB.ACT_RELU)
            elif ep == "relu":
                need(not rest, k, "operands after the output")
                kw.update(act=MB.ACT_RELU)
            else:
                need(ep == "none" and not rest, k, "unknown epilogue " + ep)
            # a residual read from the buffer the result goes to would not survive a restart
            need(kw["residual"] is None or kw["residual"].idx != a[2], k, "in-place residual")
            g.conv2d(Tensor(a[0], shape[a[0]]), cout, (fh, fw), s, (ph, pw), out=tensor(a[2], (cout, Ho, Wo), k),
                     given=given, **kw)
            shape[a[2]] = (cout, Ho, Wo)
        elif op == "dwconv2d":                                  # (in, W, out, bias)
            need(len(a) == 4 and a[0] in shape and shape[a[0]] == (e["c"], e["h"], e["w"]), k, "shape")
            C, kk = e["c"], e["k"]
            need(size(a[1]) == C * kk * kk and size(a[3]) == C, k, "weight / bias operand")
            Ho = (e["h"] + 2 * e["pad"] - kk) // e["stride"] + 1
            Wo = (e["w"] + 2 * e["pad"] - kk) // e["stride"] + 1
            g.dwconv2d(Tensor(a[0], shape[a[0]]), kk, e["stride"], e["pad"], bias=True, act=e["act"],
                       out=tensor(a[2], (C, Ho, Wo), k),
                       given={"w": Tensor(a[1], (C, 1, kk, kk)), "bias": Tensor(a[3], (C,))})
            shape[a[2]] = (C, Ho, Wo)
        elif op == "eltwise":                                   # (out, in, per-channel shift)
            need(len(a) == 3 and a[1] in shape, k, "operands")
            C, H, W = shape[a[1]]
            need(C == e["c"] and H * W == e["inner"] and size(a[2]) == C, k, "shape")
            g.eltwise(Tensor(a[1], shape[a[1]]), shift=True, act=e["act"], out=tensor(a[0], shape[a[1]], k),
                      shift_t=Tensor(a[2], (C,)))
            shape[a[0]] = shape[a[1]]
        elif op == "pool2d":                                    # (in, out[, bias])
            need(a[0] in shape and shape[a[0]] == (e["c"], e["h"], e["w"]), k, "shape")
            out = g.pool2d(Tensor(a[0], shape[a[0]]), e["k"], e["stride"], e["pad"], mode=e["mode"],
                           bias=bool(e.get("bias")), act=e.get("act", 0), out=Tensor(a[1], (1,)),
                           count_include_pad=bool(e.get("count_include_pad")),
                           bias_t=Tensor(a[2], (e["c"],)) if e.get("bias") else None)
            need(out.size <= size(a[1]), k, "output storage too small")
            shape[a[1]] = out.shape
        elif op == "concat":                # (out, operands); `operand`: which of them comes first, second ...
            H, W, parts = e["h"], e["w"], e["parts"]
            need(len(a) == 1 + len(parts) and sorted(e["operand"]) == list(range(len(parts))), k,
                 "as many operands as parts")
            whole = tensor(a[0], (sum(parts), H, W), k)
            off = 0
            for c, i in zip(parts, [a[1 + j] for j in e["operand"]]):
                need(shape.get(i) == (c, H, W) and i != a[0], k, "part %d: the graph delivers %s" % (i, shape.get(i)))
                g.copy_into(Tensor(i, (c * H * W,)), whole, off)
                off += c * H * W
            shape[a[0]] = (sum(parts), H, W)
        elif op == "global_avgpool":                            # (in, out)
            C, H, W = shape[a[0]]
            need(C == e["c"] and H * W == e["hw"], k, "shape")
            g.global_avgpool(Tensor(a[0], shape[a[0]]), out=tensor(a[1], (C,), k))
            shape[a[1]] = (C, 1, 1)
        elif op == "copy":                                      # flatten: (out, in)
            n = e["n"]
            if cnn:         # the input's shape is known and must fit
                need(a[1] in shape and shape[a[1]][0] * shape[a[1]][1] * shape[a[1]][2] == n, k, "shape")
            need(len(a) == 2 and size(a[1]) >= n and a[0] != a[1], k, "operands")
            g.copy_into(Tensor(a[1], (n,)), tensor(a[0], (n,), k), 0)
            shape[a[0]] = (n, 1, 1)
        elif op == "dense":                                     # (x, W, out, bias)
            need(shape[a[0]][0] == e["in"] and size(a[1]) == e["in"] * e["out"], k, "shape")
            g.dense(Tensor(a[0], (e["in"],)), e["out"], bias=bool(e.get("bias")), act=e.get("act", 0),
                    out=tensor(a[2], (1, e["out"]), k),
                    w=Tensor(a[1], (e["out"], e["in"])), bias_t=Tensor(a[3], (e["out"],)) if e.get("bias") else None)
            shape[a[2]] = (e["out"], 1, 1)
        elif op == "chain_stage":
            # a call of a LayerNorm / softmax chain that has no counterpart: remember what its
            # result stands for.  `input`: position of the chain's input among the call's operands
            # (taken over from the stage before it when the call does not see the input itself),
            # `mask`: position of the attention mask; the call that applies the mask becomes a
            # copy of the scores (`copy`: elements), so that the softmax kernel, which applies the
            # mask itself, does not work in place and a restarted launch finds its input intact.
            src = None
            for j, i in enumerate(a):
                if j != e["result"] and i in chain:
                    src = dict(chain[i])
            if "input" in e:
                src = {"x": a[e["input"]]}
            need(src is not None, k, "a chain stage without its chain")
            if "mask" in e:
                src["mask"] = a[e["mask"]]
            if "copy" in e:
                need(src["x"] != a[e["result"]], k, "in-place mask")
                g.copy_into(Tensor(src["x"], (e["copy"],)), tensor(a[e["result"]], (e["copy"],), k), 0)
                src["x"] = a[e["result"]]
            chain[a[e["result"]]] = src
        elif op == "mask_fill":                                 # writes the all-zero mask: storages start as zeros
            pass
        elif op == "layernorm":                                 # (out, x, mean, variance, gamma, beta)
            need(len(a) == 6 and chain.get(a[2], {}).get("x") == a[1] and a[3] in chain, k, "not the end of a LayerNorm chain")
            g.layernorm(Tensor(a[1], (e["rows"], e["cols"])), e["rows"], e["cols"], eps=e["eps"],
                        out=tensor(a[0], (e["rows"], e["cols"]), k), gamma=Tensor(a[4], (e["cols"],)),
                        beta=Tensor(a[5], (e["cols"],)))
        elif op == "masked_softmax":                            # last call of the chain: (out, exp, sum)
            src = chain.get(a[1])
            need(src is not None and "mask" in src and src["x"] != a[0], k, "not the end of a softmax chain")
            g.softmax(Tensor(src["x"], (e["rows"], e["cols"])), e["rows"], e["cols"],
                      out=tensor(a[0], (e["rows"], e["cols"]), k), mask=Tensor(src["mask"], (e["cols"],)))
        elif op == "embedding":                                 # (out, table, ids, position table, position ids)
            seq, hid = e["seq"], e["hidden"]
            need(size(a[1]) == e["vocab"] * hid and size(a[3]) == e["positions"] * hid, k, "table sizes")
            t1 = g.embedding(Tensor(a[2], (seq,)), e["vocab"], seq, hid, pos=False, seg=False, tok=Tensor(a[1], (e["vocab"], hid)))
            t2 = g.embedding(Tensor(a[4], (seq,)), e["positions"], seq, hid, pos=False, seg=False,
                             tok=Tensor(a[3], (e["positions"], hid)))
            g.eltwise(t1, b=t2, out=tensor(a[0], (seq, hid), k))
        elif op == "gemm_nt":                                   # (A, B, C): C[b] = alpha A[b] B[b]^T
            bt, M, N, K = e["batch"], e["m"], e["n"], e["k"]
            need(size(a[0]) >= bt * M * K and size(a[1]) >= bt * N * K, k, "operand sizes")
            g.gemm(Tensor(a[0], (bt, M, K)), Tensor(a[1], (bt, N, K)), M, N, K, batch=bt, trans_b=True,
                   alpha=alpha_of.pop(a[0], 1.0), stride_a=M * K if bt > 1 else 0, stride_b=N * K if bt > 1 else 0,
                   stride_c=M * N if bt > 1 else 0, out=tensor(a[2], (bt, M, N), k))
        elif op == "rowbias_heads":                             # (out, x, bias): [row][head][d] -> [head][row][d] of x + bias[row]
            R, H, D = e["rows"], e["heads"], e["d"]
            t = g.eltwise(Tensor(a[1], (R, H * D)), shift=True, shift_t=Tensor(a[2], (R,)))
            g.transpose_102(t, R, H, D, out=tensor(a[0], (H, R, D), k))
            if e.get("scale", 1.0) != 1.0:
                alpha_of[a[0]] = e["scale"]
        elif op == "rowbias_transpose":                         # (out, x, bias): out[c][r] = x[r][c] + bias[r]
            R, C = e["rows"], e["cols"]
            t = g.eltwise(Tensor(a[1], (R, C)), shift=True, shift_t=Tensor(a[2], (R,)))
            g.transpose_102(t, R, C, 1, out=tensor(a[0], (C, R, 1), k))
        elif op == "heads_merge":                               # (out, x): [head][row][d] -> [row][head][d]
            H, R, D = e["heads"], e["rows"], e["d"]
            g.transpose_102(Tensor(a[1], (H, R, D)), H, R, D, out=tensor(a[0], (R, H, D), k))
        elif op == "rowbias_add":                               # (out, x, bias, res): (x + bias[row]) + res
            R, C = e["rows"], e["cols"]
            need(a[0] not in (a[1], a[3]), k, "in-place add")
            g.eltwise(Tensor(a[1], (R, C)), b=Tensor(a[3], (R, C)), shift=True, shift_t=Tensor(a[2], (R,)),
                      out=tensor(a[0], (R, C), k))
        elif op == "rowbias_gelu":                              # (out, x, bias): gelu(x + bias[row])
            R, C = e["rows"], e["cols"]
            t = g.eltwise(Tensor(a[1], (R, C)), shift=True, shift_t=Tensor(a[2], (R,)))
            g.bias_gelu(t, R, C, bias=False, out=tensor(a[0], (R, C), k))
        elif op == "softmax":                                   # (in, out)
            need(shape[a[0]][0] == e["cols"], k, "shape")
            g.softmax(Tensor(a[0], (e["rows"], e["cols"])), e["rows"], e["cols"],
                      out=tensor(a[1], (e["rows"], e["cols"]), k))
            shape[a[1]] = shape[a[0]]
        else:
            need(False, k, "unknown op " + op)
        g.imported_calls += [call] * (len(g.kernels) - first_new)
    need(not wino, ref["kernels"][-1], "a Winograd transform without its last call")
    g.imported_from = [k["name"] for k in ref["kernels"]]
    return g


def read_params(path):
    """[(key, float32 array)] of a `.param` file (reader src/reef/executor/model.cpp:82-121)."""
    with open(path, "rb") as f:
        blob = f.read()
    if blob[:17] != b"TVM_MODEL_PARAMS\0":
        raise ImportError_("%s is not a parameter file" % path)
    (count,), pos, out = struct.unpack_from("<Q", blob, 17), 25, []
    for _ in range(count):
        end = blob.index(b"\0", pos)
        key = blob[pos:end].decode("ascii")
        (n,) = struct.unpack_from("<Q", blob, end + 1)
        out.append((key, np.frombuffer(blob, "<f4", n, end + 9).copy()))
        pos = end + 9 + 4 * n
    return out


def convert_params(g, params):
    """Parameters of the reference graph -> parameters of the imported graph `g`: unchanged, except
    that a transformed Winograd weight is replaced by the direct weight recovered from it."""
    out = []
    for key, arr in params:
        if key in g.direct_weights:
            dkey, tile, cout, cin = g.direct_weights[key]
            alpha = tile + 2
            if arr.size != alpha * alpha * cin * cout:
                raise ImportError_("parameter %s holds %d values, the table asks for %d"
                                   % (key, arr.size, alpha * alpha * cin * cout))
            out.append((dkey, winograd_untransform(arr.reshape(alpha, alpha, cin, cout), tile).ravel()))
        else:
            out.append((key, arr))
    return out


def import_model_dir(ref_dir, model_name, out_dir, table=None, measured_profile=False):
    """<ref_dir>/<model>.json (+ .param if present) -> a model directory of this build in out_dir.
    Returns the GraphBuilder.  A `.param` file of the reference is taken over byte for byte (same
    keys, same storages) unless the graph has Winograd weights, which are converted
    (convert_params); the profile is the estimate unless measured_profile (needs a GPU)."""
    import shutil
    g = import_model(os.path.join(ref_dir, model_name + ".json"), table=table, name=model_name)
    g.write(out_dir)
    src = os.path.join(ref_dir, model_name + ".param")
    if os.path.exists(src):
        if g.direct_weights:
            MB.write_params(os.path.join(out_dir, model_name + ".param"), convert_params(g, read_params(src)))
        else:
            shutil.copyfile(src, os.path.join(out_dir, model_name + ".param"))
    if measured_profile:
        from . import profiler
        profiler.write_profile(out_dir, model_name)
    return g


def param_storages(ref):
    """{storage name: index} of the parameters of a reference graph: the storages its `args` list
    names (graph inputs and parameters, generate_final_schedule.py:109-144) other than the
    input.  TVM calls them p0..pN or by their relay names (conv_1_weight)."""
    return {ref["storage"][i]["name"]: i for i in ref.get("args", [])
            if i != 0 and ref["storage"][i]["name"] not in ("data", "null", "output", "temp_arg")}


def seeded_params(ref_json_path, table=None, seed=0x5EEF):
    """Seeded parameters for a reference graph that ships without a `.param` file (the checkout's
    resource/resnet152 does): He-normal weights, small biases / shifts, scales around 1 -- the
    distributions the generator of this build uses.  Returns [(key, float32 array)] in storage
    order, ready for modelgen.builder.write_params."""
    import math
    from .modelgen import rng
    ref = json.load(open(ref_json_path))
    model_name = os.path.splitext(os.path.basename(ref_json_path))[0]
    if table is None:
        table = load_table(model_name)
    elif isinstance(table, str):
        table = json.load(open(table))
    std = {}
    one_plus = set()
    params = set(param_storages(ref).values())
    transformed = {}                   # storage of a Winograd weight -> (tile, Cout, Cin)
    gemm_of = {}                       # scratch storage a Winograd GEMM wrote -> its weight storage
    for k in ref["kernels"]:
        e, a = table[k["name"]], k["args"]
        if e["op"] == "winograd_gemm":
            gemm_of[a[2]] = a[0]
        elif e["op"] == "conv2d" and e.get("winograd_tile"):
            transformed[gemm_of[a[0]]] = (e["winograd_tile"], e["cout"], e["cin"])
            if e["epilogue"] == "residual_scale_shift_relu":
                std[a[3]] = 0.1
                one_plus.add(a[3])
        elif e["op"] == "conv2d":
            std[a[1]] = math.sqrt(2.0 / (e["cin"] * pair(e["k"])[0] * pair(e["k"])[1]))
            if e["epilogue"] == "residual_scale_shift_relu":
                std[a[4]] = 0.1
                one_plus.add(a[4])
        elif e["op"] == "dwconv2d":
            std[a[1]] = math.sqrt(2.0 / (e["k"] * e["k"]))
        elif e["op"] == "dense":
            std[a[1]] = math.sqrt(2.0 / e["in"])
        elif e["op"] == "gemm_nt" and a[1] in params:
            std[a[1]] = math.sqrt(1.0 / e["k"])
        elif e["op"] == "layernorm":
            std[a[4]] = 0.1
            one_plus.add(a[4])
        elif e["op"] == "embedding":
            std[a[1]] = std[a[3]] = 0.5
    out = []
    for i, s in enumerate(ref["storage"]):
        name = s["name"]
        if i not in params or s["stype"] != "float32":      # a parameter file holds floats only
            continue
        if i in transformed:           # a seeded direct weight, stored the way the reference stores it
            tile, cout, cin = transformed[i]
            direct = rng.normal_f32(model_name + "/" + name, cout * cin * 9, math.sqrt(2.0 / (cin * 9)), seed)
            out.append((name, winograd_transform(direct.reshape(cout, cin, 3, 3), tile).ravel()))
            continue
        arr = rng.normal_f32(model_name + "/" + name, s["size"], std.get(i, 0.01), seed)
        if i in one_plus:
            arr = arr + 1.0
        out.append((name, arr.astype("float32")))
    return out
