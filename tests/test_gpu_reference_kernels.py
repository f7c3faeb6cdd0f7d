"""The CPU oracle against the reference's OWN device code.

`oracle/_ref/*.raw.co` are the reference's generated kernels (resource/resnet152/resnet152.cu,
resource/mocked_kernel/mocked_kernel.cu, resource/bert/bert.cu) compiled for gfx950 from where they lie in the reference
tree (`make -C oracle ref`); `tests/golden/*.json` are the reference's graph files for them.  The
executor of this build loads that pair like any model directory (kernel names resolve in the code
object, arguments are the storages in JSON order) and runs ONE reference kernel at a time on
random operands; the oracle has to reproduce its output.

The generated kernels have their shapes baked into the source and the graph JSON only holds
(shared, maximal) buffer sizes, so the shape of each kernel is found from what it does: the weight
and per-channel operand sizes give Cout and Cin*k*k, the number of output elements the kernel
writes gives Cout*Ho*Wo, and of the few (H, stride) that are consistent with those exactly the
right one makes the oracle's output equal the kernel's.  A wrong epilogue order, padding value or
stride rule in the oracle leaves no hypothesis that matches.

Two of the reference's kernels cannot serve as witnesses, and the tests say so explicitly:
  * fused_nn_conv2d_add_nn_relu_8_kernel0 stages its first 128 input channels with a row index
    `((threadIdx.x * 25) + 1) % 49 / 7` where every other load of the file has `+ i`
    (resource/resnet152/resnet152.cu:3399 against :3410): as checked in, it is not a convolution;
  * the dense and softmax kernels reduce across the wavefront with `__hip_ds_bpermute(int, float)`
    (resnet152.cu:14-26, 775-841); the HIP headers of ROCm 7.2 only declare the (int, int) form
    under that name, so the partial sums go through an integer and lose their fraction (and, as
    observed, their sign).  Dense is therefore checked on small non-negative integer operands
    (every partial sum is a non-negative integer, the detour is exact); softmax is not checked
    against the reference kernel.
"""
import ctypes
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
REF_CO = os.path.join(ROOT, "oracle", "_ref", "resnet152.raw.co")
MOCK_CO = os.path.join(ROOT, "oracle", "_ref", "mocked_kernel.raw.co")
SENTINEL = np.float32(-7.5e8)
TOL = 2e-5


def _need(path):
    if not os.path.exists(path):
        pytest.skip("%s not built (needs the reference tree at build time: make -C oracle ref)"
                    % os.path.relpath(path, ROOT))


@pytest.fixture(scope="module")
def ref152():
    _need(REF_CO)
    model = json.load(open(os.path.join(HERE, "golden", "resnet152.json")))
    roles = json.load(open(os.path.join(HERE, "golden", "resnet152_kernel_roles.json")))
    exe = B.Executor(B.BASE)
    exe.load(os.path.join(HERE, "golden", "resnet152.json"), REF_CO)
    return model, roles, exe


def _set(exe, model, idx, values):
    size = model["storage"][idx]["size"]
    buf = np.zeros(size, np.float32)
    v = np.asarray(values, np.float32).ravel()
    buf[:v.size] = v
    assert lib_ok(B.lib().reef_executor_set_input_idx(exe.h, idx, ctypes.c_void_p(buf.ctypes.data),
                                                      ctypes.c_size_t(buf.nbytes)))
    return buf


def lib_ok(st):
    return st == 0


def run_reference_kernel(exe, model, roles, kidx, rng):
    """Random operands in, sentinel in the output buffer, one launch.  Returns
    (operands by parameter name, raw output buffer, how many leading elements were written)."""
    k = model["kernels"][kidx]
    names = roles[k["name"]]
    assert len(names) == len(k["args"])
    out_pos = [i for i, n in enumerate(names) if not n.startswith("placeholder")]
    assert len(out_pos) == 1, names
    out_idx = k["args"][out_pos[0]]
    ops = {}
    for n, a in zip(names, k["args"]):
        size = model["storage"][a]["size"]
        if n.startswith("placeholder"):
            assert a != out_idx
            ops[n] = _set(exe, model, a, rng.standard_normal(size).astype(np.float32))
    _set(exe, model, out_idx, np.full(model["storage"][out_idx]["size"], SENTINEL, np.float32))
    exe.execute_kernel(kidx)
    out = exe.get_data(out_idx, model["storage"][out_idx]["size"])
    written = np.nonzero(out != SENTINEL)[0]
    n_written = int(written.max()) + 1 if written.size else 0
    assert written.size == n_written, "output is not one contiguous tensor"
    return ops, out, n_written


def close(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return a.shape == b.shape and np.abs(a - b).max() <= TOL * max(np.abs(b).max(), 1.0)


def conv_hypotheses(sx, sw, n_written, cout_known):
    for cout in ([cout_known] if cout_known else (64, 128, 256, 512, 1024, 2048)):
        if sw % cout or n_written % cout:
            continue
        q = sw // cout
        for k in (7, 3, 1):
            if q % (k * k):
                continue
            cin = q // (k * k)
            for H in (64, 32, 16, 8, 4, 2):
                if cin * H * H > sx:
                    continue
                for s in (1, 2):
                    p = k // 2
                    Ho = (H + 2 * p - k) // s + 1
                    if Ho >= 1 and cout * Ho * Ho == n_written:
                        yield cout, cin, k, H, s, p


def distinct_kernels(model, prefix):
    seen, out = set(), []
    for i, k in enumerate(model["kernels"]):
        if k["name"].startswith(prefix) and k["name"] not in seen:
            seen.add(k["name"])
            out.append(i)
    return out


def test_reference_conv_kernels_match_oracle(ref152):
    """The 25 generated convolution kernels of the reference's ResNet-152 (families
    fused_nn_conv2d[_add][_add][_multiply_add][_nn_relu], resnet152.cu:35-4786): 24 are
    reproduced by the oracle, one is known not to be a convolution."""
    model, roles, exe = ref152
    rng = np.random.default_rng(152)
    checked = 0
    failed = []
    for kidx in distinct_kernels(model, "fused_nn_conv2d"):
        k = model["kernels"][kidx]
        name = k["name"]
        ops, out, n_written = run_reference_kernel(exe, model, roles, kidx, rng)
        x, w = ops["placeholder"], ops["placeholder1"]
        extras = [ops[n] for n in roles[name] if n.startswith("placeholder") and n not in ("placeholder", "placeholder1")]
        fam = name.split("_kernel0")[0].rstrip("0123456789").rstrip("_")
        relu = fam.endswith("nn_relu")
        # per-channel operands are the small ones; a residual is as large as the output buffer
        small = [e for e in extras if e.size < n_written]
        cout_known = small[0].size if small else 0
        matches = []
        for cout, cin, kk, H, s, p in conv_hypotheses(x.size, w.size, n_written, cout_known):
            Ho = (H + 2 * p - kk) // s + 1
            xs = x[:cin * H * H].reshape(cin, H, H)
            ws = w[:cout * cin * kk * kk].reshape(cout, cin, kk, kk)
            kw = dict(stride=(s, s), pad=(p, p), act=1 if relu else 0, acc64=True)
            full = [e[:cout * Ho * Ho].reshape(cout, Ho, Ho) for e in extras if e.size >= n_written]
            if fam == "fused_nn_conv2d":
                want = O.conv2d(xs, ws, **kw)
            elif fam == "fused_nn_conv2d_add":                       # + residual (resnet152.cu:315-338)
                want = O.conv2d(xs, ws, residual=full[0], **kw)
            elif fam == "fused_nn_conv2d_add_nn_relu":               # relu(+ bias) (:376-713)
                want = O.conv2d(xs, ws, bias=small[0], **kw)
            elif fam == "fused_nn_conv2d_add_add_nn_relu":           # relu((+ residual) + bias) (:2662)
                want = O.conv2d(xs, ws, residual=full[0], bias=small[0], **kw)
            elif fam == "fused_nn_conv2d_add_multiply_add_nn_relu":  # relu(fma(+ residual, scale, shift)) (:340-363)
                want = O.conv2d(xs, ws, residual=full[0], scale=small[0], shift=small[1], **kw)
            else:
                raise AssertionError("unknown family " + fam)
            if close(out[:n_written], want):
                matches.append((cout, cin, kk, H, s, p))
        if not matches:
            failed.append((name, n_written))
            print("%-52s NO MATCH (wrote %d)" % (name, n_written))
            continue
        print("%-52s Cout %4d Cin %4d k %d H %2d stride %d pad %d" % ((name,) + matches[0]))
        checked += 1
    # the one kernel that is not a convolution as checked in (see the module docstring)
    assert [f[0] for f in failed] == ["fused_nn_conv2d_add_nn_relu_8_kernel0"], failed
    assert checked == 24


def test_reference_bandwidth_kernels_match_oracle(ref152):
    """Per-channel add (+ReLU), max-pool+add+ReLU, global average pool, flatten, dense+add,
    softmax (resnet152.cu:2-33,365-374,771-841,4056-4066,4390-4403,4472-4474,4782-4784)."""
    model, roles, exe = ref152
    rng = np.random.default_rng(7)
    done = set()
    for kidx, k in enumerate(model["kernels"]):
        name = k["name"]
        if name.startswith("fused_nn_conv2d") or name in done:
            continue
        done.add(name)
        ops, out, n = run_reference_kernel(exe, model, roles, kidx, rng)
        got = out[:n]
        if name.startswith("fused_add"):
            x, p = ops["placeholder"], ops["placeholder1"]
            C = p.size
            assert n % C == 0
            xs = x[:n].reshape(C, n // C)
            want = O.eltwise(xs, shift=p, act=1 if "nn_relu" in name else 0)
            assert close(got, want), name
        elif name.startswith("fused_nn_max_pool2d_add_nn_relu"):
            x, p = ops["placeholder"], ops["placeholder1"]
            C = p.size
            Ho = int(round((n // C) ** 0.5))
            H = 2 * Ho
            want = O.pool2d(x[:C * H * H].reshape(C, H, H), (3, 3), (2, 2), (1, 1), 0, bias=p, act=1)
            assert close(got, want), name
        elif name.startswith("fused_nn_global_avg_pool2d"):
            x = ops["placeholder"]
            ok = False
            for hw in (1, 4, 16, 49):
                if n * hw <= x.size and close(got, O.global_avgpool(x[:n * hw].reshape(n, hw))):
                    ok = True
            assert ok, name
        elif name.startswith("fused_nn_batch_flatten"):
            assert np.array_equal(got, ops["placeholder"][:n]), name
        elif name.startswith("fused_nn_dense_add"):
            # small non-negative integer operands: see the module docstring
            names = roles[name]
            ints = {}
            for pn, a in zip(names, k["args"]):
                if pn.startswith("placeholder"):
                    size = model["storage"][a]["size"]
                    ints[pn] = _set(exe, model, a, rng.integers(0, 4, size).astype(np.float32))
            out_idx = k["args"][[i for i, pn in enumerate(names) if not pn.startswith("placeholder")][0]]
            exe.execute_kernel(kidx)
            got = exe.get_data(out_idx, model["storage"][out_idx]["size"])[:n]
            x, w, b = ints["placeholder"], ints["placeholder1"], ints["placeholder2"]
            assert n == b.size and w.size % n == 0
            in_f = w.size // n
            want = O.dense(x[:in_f].reshape(1, in_f), w.reshape(n, in_f), bias=b, acc64=True)
            np.testing.assert_array_equal(got, want.ravel(), err_msg=name)
        elif name.startswith("fused_nn_softmax"):
            print("%-44s not a witness (float reduction through an int shuffle)" % name)
            continue
        else:
            raise AssertionError("unexpected kernel " + name)
        print("%-44s wrote %6d elements: oracle agrees" % (name, n))
    assert len(done) == 10


def _set_typed(exe, model, idx, values):
    """A storage of any element type (int64 ids, one-byte masks, float tensors), zero-extended."""
    st = model["storage"][idx]
    dt = {"int64": np.int64, "uint1": np.uint8, "byte": np.uint8}.get(st["stype"], np.float32)
    buf = np.zeros(st["size"], dt)
    v = np.asarray(values).astype(dt).ravel()
    buf[:v.size] = v
    assert lib_ok(B.lib().reef_executor_set_input_idx(exe.h, idx, ctypes.c_void_p(buf.ctypes.data),
                                                      ctypes.c_size_t(buf.nbytes)))
    return buf


def test_reference_bert_kernels_match_oracle():
    """The transformer kernels of the reference's BERT (resource/bert/bert.cu: hidden 480, 12 heads of
    40, sequence 480), each on random operands against the oracle's op: the five calls of a
    LayerNorm (mean, variance, normalise: bert.cu fused_mean_1 / fused_variance_1 /
    fused_subtract_add_sqrt_divide_multiply_add_1, eps 1e-12), the mask kernel + the four calls
    of a softmax (fused_reshape_cast_broadcast_to_like_where, fused_nn_softmax_1_kernel0-3), exact
    GELU with its bias, the embedding sum, the three batched products, the head split / merge
    transposes with their bias and scale, and the residual add.  These kernels reduce through
    shared memory, not through the shuffle that spoils the CNN directories' dense and softmax
    kernels, so all of them are witnesses.  (The reference lays activations out [feature][token]
    in places, hence the transposes around the oracle calls below.)"""
    co = os.path.join(ROOT, "oracle", "_ref", "bert.raw.co")
    _need(co)
    path = os.path.join(HERE, "golden", "bert.json")
    model = json.load(open(path))
    exe = B.Executor(B.BASE)
    exe.load(path, co)
    rng = np.random.default_rng(480)
    S = Hd = 480
    heads, hd = 12, 40
    calls = model["kernels"]
    first = {}
    for i, k in enumerate(calls):
        first.setdefault(k["name"], i)
    size = lambda i: model["storage"][i]["size"]
    rnd_into = lambda idx, n=None: _set_typed(exe, model, idx, rng.standard_normal(n or size(idx)))
    get = lambda idx, n: exe.get_data(idx, size(idx))[:n]

    # LayerNorm: calls mean k0, k1, variance k0, k1, normalise, as the graph wires them
    i0 = first["fused_mean_1_kernel0"]
    assert [c["name"] for c in calls[i0:i0 + 5]] == ["fused_mean_1_kernel0", "fused_mean_1_kernel1",
                                                      "fused_variance_1_kernel0", "fused_variance_1_kernel1",
                                                      "fused_subtract_add_sqrt_divide_multiply_add_1_kernel0"]
    a = calls[i0 + 4]["args"]                      # (out, x, mean, variance, gamma, beta)
    assert a[1] == calls[i0]["args"][0] and a[2] == calls[i0 + 1]["args"][0] and a[3] == calls[i0 + 3]["args"][0]
    x = rnd_into(a[1])[:S * Hd].reshape(S, Hd) * 3 + 0.5
    _set_typed(exe, model, a[1], x)
    gamma, beta = rnd_into(a[4])[:Hd], rnd_into(a[5])[:Hd]
    for i in range(i0, i0 + 5):
        exe.execute_kernel(i)
    assert close(get(a[0], S * Hd), O.layernorm(x, gamma, beta, None, 1e-12)), "layernorm"
    assert close(get(a[2], S), x.mean(1)) and close(get(a[3], S), x.var(1)), "mean / variance"

    # attention mask + softmax: where(mask, -inf, x), then max, exp, sum, divide
    i0 = first["fused_reshape_cast_broadcast_to_like_where_kernel0"]
    assert [c["name"][-20:] for c in calls[i0 + 1:i0 + 5]] == ["nn_softmax_1_kernel%d" % j for j in range(4)]
    w = calls[i0]["args"]                          # (out, mask, x)
    mask = (rng.random(S) < 0.3).astype(np.uint8)
    mask[:4] = 0
    _set_typed(exe, model, w[1], mask)
    x = rnd_into(w[2])[:heads * S * S].reshape(heads * S, S) * 4
    _set_typed(exe, model, w[2], x)
    for i in range(i0, i0 + 5):
        exe.execute_kernel(i)
    out = get(calls[i0 + 4]["args"][0], heads * S * S).reshape(heads * S, S)
    assert (out[:, mask != 0] == 0).all() and close(out, O.softmax(x, mask)), "masked softmax"

    # exact GELU of (x + bias[feature]) on a [feature][token] tensor
    i0 = first["fused_reshape_add_multiply_erf_multiply_add_multiply_reshape_kernel0"]
    a = calls[i0]["args"]                          # (out, x, bias)
    x, bias = rnd_into(a[1])[:Hd * S].reshape(Hd, S) * 2, rnd_into(a[2])[:Hd]
    _set_typed(exe, model, a[1], x)
    exe.execute_kernel(i0)
    assert close(get(a[0], Hd * S).reshape(Hd, S), O.bias_gelu(np.ascontiguousarray(x.T), bias).T), "gelu"

    # embedding: tok[ids] + pos[position ids]
    i0 = first["fused_cast_take_broadcast_to_like_cast_take_add_1_kernel0"]
    a = calls[i0]["args"]                          # (out, tok, ids, pos, position ids)
    vocab = size(a[1]) // Hd
    tok = rnd_into(a[1]).reshape(vocab, Hd)
    pos = rnd_into(a[3]).reshape(-1, Hd)
    ids = rng.integers(0, vocab, S)
    _set_typed(exe, model, a[2], ids)
    _set_typed(exe, model, a[4], np.arange(S))
    exe.execute_kernel(i0)
    np.testing.assert_array_equal(get(a[0], S * Hd).reshape(S, Hd), O.embedding(ids, tok, pos[:S]))

    # batched products (B stored [n][k] in all three)
    for name, (bt, M, N, K) in (("fused_nn_batch_matmul_3_kernel0", (1, S, Hd, Hd)),
                                 ("fused_nn_batch_matmul_5_kernel0", (heads, S, S, hd)),
                                 ("fused_nn_batch_matmul_4_kernel0", (heads, S, hd, S))):
        i0 = first[name]
        a = calls[i0]["args"]                      # (A, B, C)
        A = rnd_into(a[0])[:bt * M * K].reshape(bt, M, K)
        Bm = rnd_into(a[1])[:bt * N * K].reshape(bt, N, K)
        _set(exe, model, a[2], np.full(size(a[2]), SENTINEL, np.float32))
        exe.execute_kernel(i0)
        out = exe.get_data(a[2], size(a[2]))
        assert (out[:bt * M * N] != SENTINEL).all() and (out[bt * M * N:] == SENTINEL).all(), name
        assert close(out[:bt * M * N], O.batch_matmul(A, Bm, True, 1.0, True)), name

    # head split [row][head][d] -> [head][row][d] of (x + bias[row]) (and the 1/sqrt(d) of the queries)
    for name, scale in (("fused_reshape_add_reshape_transpose_divide_reshape_kernel0", 1.0 / np.sqrt(np.float32(hd))),
                        ("fused_reshape_add_reshape_transpose_transpose_reshape_transpose_kernel0", 1.0)):
        i0 = first[name]
        a = calls[i0]["args"]                      # (out, x, bias)
        x, bias = rnd_into(a[1])[:S * Hd].reshape(S, Hd), rnd_into(a[2])[:S]
        exe.execute_kernel(i0)
        want = O.transpose_102(O.eltwise(x, shift=bias).reshape(S, heads, hd)) * np.float32(scale)
        assert close(get(a[0], S * Hd), want), name
    # values: (x + bias[feature]) transposed, x stored [feature][token]
    i0 = first["fused_reshape_add_reshape_transpose_reshape_transpose_kernel0"]
    a = calls[i0]["args"]
    x, bias = rnd_into(a[1])[:Hd * S].reshape(Hd, S), rnd_into(a[2])[:Hd]
    exe.execute_kernel(i0)
    want = O.transpose_102(O.eltwise(x, shift=bias).reshape(Hd, S, 1))
    np.testing.assert_array_equal(get(a[0], S * Hd), want.ravel())
    # head merge [head][token][d] -> [token][head][d]
    i0 = first["fused_reshape_transpose_copy_reshape_1_kernel0"]
    a = calls[i0]["args"]
    x = rnd_into(a[1])[:S * Hd].reshape(heads, S, hd)
    exe.execute_kernel(i0)
    np.testing.assert_array_equal(get(a[0], S * Hd), O.transpose_102(x).ravel())
    # residual: (x + bias[feature]) + res
    i0 = first["fused_reshape_add_add_kernel0"]
    a = calls[i0]["args"]                          # (out, x, bias, res)
    x, bias, res = rnd_into(a[1])[:Hd * S].reshape(Hd, S), rnd_into(a[2])[:Hd], rnd_into(a[3])[:Hd * S].reshape(Hd, S)
    exe.execute_kernel(i0)
    assert close(get(a[0], Hd * S), O.eltwise(x, b=res, shift=bias)), "residual add"
    exe.close()


def test_reference_mocked_kernels_closed_form():
    """The reference's own mocked model on its own kernels: a = b = c = 3 -> (3 + 3) * 3 = 18
    (src/reef/test/test.cpp:105-115)."""
    _need(MOCK_CO)
    exe = B.Executor(B.BASE)
    exe.load(os.path.join(HERE, "golden", "mocked_kernel.json"), MOCK_CO)
    three = np.full(8192, 3.0, np.float32)
    for n in "abc":
        exe.set_input_checked(n, three)
    exe.execute()
    np.testing.assert_array_equal(exe.get_output(), np.full(8192, 18.0, np.float32))
