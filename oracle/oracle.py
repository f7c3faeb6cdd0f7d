"""CPU oracle for the REEF hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

ctypes front-end of ``libreef_oracle.so`` (``reef_oracle.c``) plus a graph
interpreter that executes a model directory's graph JSON kernel by kernel on
the CPU, the way the reference's ``ExecutorBase::execute`` walks
``model->kernels`` in order (src/reef/executor/executor_base.cpp:191-209),
binding ``args`` positionally to storages (executor_base.cpp:66-75).

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s
``cpu_baseline`` leg may import this module.  The attribute slots read here
follow ``include/reef_kernels.h`` and are typed in independently of the
product's model generator, so a slot mix-up on either side shows up as a
parity failure.
"""
import ctypes
import json
import os
import struct
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile libreef_oracle.so (and oracle/_ref when the reference tree exists)."""
    so = os.path.join(_HERE, "libreef_oracle.so")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(
            os.path.join(_HERE, "reef_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libreef_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libreef_oracle.so")
        if not os.path.exists(so):
            build()
        _LIB = ctypes.CDLL(so)
    return _LIB


def _p(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f32p)


def _f(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    """Limit the OpenMP team of the oracle (used by the timed cpu_baseline leg)."""
    os.environ["OMP_NUM_THREADS"] = str(n)


# --------------------------------------------------------------------------- ops
def conv2d(x, w, bias=None, residual=None, scale=None, shift=None, stride=(1, 1), pad=(0, 0),
           groups=1, act=0, act_max=6.0, acc64=False):
    x, w = _f(x), _f(w)
    Cin, H, W = x.shape
    Cout, _, kh, kw = w.shape
    Ho = (H + 2 * pad[0] - kh) // stride[0] + 1
    Wo = (W + 2 * pad[1] - kw) // stride[1] + 1
    out = np.empty((Cout, Ho, Wo), np.float32)
    bias, residual, scale, shift = _f(bias), _f(residual), _f(scale), _f(shift)
    lib().reef_oracle_conv2d(_p(x), _p(w), _p(bias), _p(residual), _p(scale), _p(shift), _p(out),
                             Cin, H, W, Cout, kh, kw, stride[0], stride[1], pad[0], pad[1],
                             groups, act, ctypes.c_float(act_max), int(acc64))
    return out


def dense(x, w, bias=None, act=0, acc64=False):
    x, w, bias = _f(x), _f(w), _f(bias)
    rows, in_f = x.shape
    out_f = w.shape[0]
    y = np.empty((rows, out_f), np.float32)
    lib().reef_oracle_dense(_p(x), _p(w), _p(bias), _p(y), rows, in_f, out_f, act, int(acc64))
    return y


def batch_matmul(a, b, trans_b=True, alpha=1.0, acc64=False):
    a, b = _f(a), _f(b)
    batch, M, K = a.shape
    N = b.shape[1] if trans_b else b.shape[2]
    c = np.empty((batch, M, N), np.float32)
    lib().reef_oracle_batch_matmul(_p(a), _p(b), _p(c), batch, M, N, K, int(trans_b),
                                   ctypes.c_float(alpha), int(acc64))
    return c


def pool2d(x, k, stride, pad, mode, bias=None, act=0, count_include_pad=False, out_hw=None):
    x, bias = _f(x), _f(bias)
    C, H, W = x.shape
    if out_hw is None:
        Ho = (H + 2 * pad[0] - k[0]) // stride[0] + 1
        Wo = (W + 2 * pad[1] - k[1]) // stride[1] + 1
    else:
        Ho, Wo = out_hw
    out = np.empty((C, Ho, Wo), np.float32)
    lib().reef_oracle_pool2d(_p(x), _p(bias), _p(out), C, H, W, k[0], k[1], stride[0], stride[1],
                             pad[0], pad[1], Ho, Wo, mode, int(count_include_pad), act)
    return out


def global_avgpool(x):
    x = _f(x)
    C = x.shape[0]
    out = np.empty((C,), np.float32)
    lib().reef_oracle_global_avgpool(_p(x), _p(out), C, int(x.size // C))
    return out


def eltwise(a, b=None, scale=None, shift=None, act=0, act_max=6.0):
    a, b, scale, shift = _f(a), _f(b), _f(scale), _f(shift)
    C = a.shape[0]
    inner = int(a.size // C)
    out = np.empty_like(a)
    lib().reef_oracle_eltwise(_p(a), _p(b), _p(scale), _p(shift), _p(out), C, inner, act,
                              ctypes.c_float(act_max))
    return out


def softmax(x, mask=None):
    """mask: one byte per column, non-zero = the column counts as -inf (bert.cu:381-388)."""
    x = _f(x)
    rows, cols = x.shape
    out = np.empty_like(x)
    if mask is None:
        lib().reef_oracle_softmax(_p(x), _p(out), rows, cols)
    else:
        mask = np.ascontiguousarray(mask, dtype=np.uint8)
        assert mask.size >= cols
        lib().reef_oracle_softmax_masked(_p(x), mask.ctypes.data_as(ctypes.c_void_p), _p(out), rows, cols)
    return out


def layernorm(x, gamma, beta, res=None, eps=1e-12):
    x, gamma, beta, res = _f(x), _f(gamma), _f(beta), _f(res)
    rows, cols = x.shape
    out = np.empty_like(x)
    lib().reef_oracle_layernorm(_p(x), _p(res), _p(gamma), _p(beta), _p(out), rows, cols,
                                ctypes.c_float(eps))
    return out


def bias_gelu(x, bias=None):
    x, bias = _f(x), _f(bias)
    rows, cols = x.shape
    out = np.empty_like(x)
    lib().reef_oracle_bias_gelu(_p(x), _p(bias), _p(out), rows, cols)
    return out


def embedding(ids, tok, pos=None, seg=None):
    ids = np.ascontiguousarray(ids, dtype=np.int64)
    tok, pos, seg = _f(tok), _f(pos), _f(seg)
    seq, hidden = ids.shape[0], tok.shape[1]
    out = np.empty((seq, hidden), np.float32)
    lib().reef_oracle_embedding(ids.ctypes.data_as(_i64p), _p(tok), _p(pos), _p(seg), _p(out), seq,
                                hidden)
    return out


def transpose_102(x, bias=None):
    x, bias = _f(x), _f(bias)
    d0, d1, d2 = x.shape
    out = np.empty((d1, d0, d2), np.float32)
    lib().reef_oracle_transpose_102(_p(x), _p(bias), _p(out), d0, d1, d2)
    return out


def mocked(a, b, is_multiply, blocks=64, threads=128):
    a, b = _f(a), _f(b)
    out = np.empty(blocks * threads, np.float32)
    lib().reef_oracle_mocked(_p(a), _p(b), _p(out), blocks, threads, int(is_multiply))
    return out


# ------------------------------------------------------------ model resource files
PARAM_MAGIC = b"TVM_MODEL_PARAMS\0"


def read_params(path):
    """``.param`` reader restating ModelParamParser::parse_from_file
    (src/reef/executor/model.cpp:82-121): 17-byte magic, u64 count, then per
    tensor a NUL-terminated key, u64 element count, that many little-endian f32."""
    out = {}
    with open(path, "rb") as f:
        data = f.read()
    assert data[:17] == PARAM_MAGIC, "bad magic"
    (n,) = struct.unpack_from("<Q", data, 17)
    assert n != 0
    off = 25
    for _ in range(n):
        end = data.index(b"\0", off)
        key = data[off:end].decode("ascii")
        off = end + 1
        (cnt,) = struct.unpack_from("<Q", data, off)
        off += 8
        assert cnt != 0
        out[key] = np.frombuffer(data, dtype="<f4", count=cnt, offset=off).copy()
        off += 4 * cnt
    return out


STYPE_SIZE = {"float32": 4, "int64": 8, "byte": 1, "uint1": 1, "int32": 4}  # model.cpp:147-156
STYPE_NP = {"float32": np.float32, "int64": np.int64, "byte": np.uint8, "uint1": np.uint8,
            "int32": np.int32}


def _bits_to_float(i):
    return struct.unpack("<f", struct.pack("<i", int(i)))[0]


def _opt(ptrs, pos, flags, bits):
    """Optional operands follow the fixed ones in flag-bit order."""
    out = []
    for b in bits:
        if flags & b:
            out.append(ptrs[pos])
            pos += 1
        else:
            out.append(None)
    return out


class GraphOracle:
    """Executes a graph JSON on the CPU.  Storages are zero-filled at load
    (executor_base.cpp:55-64); ``.param`` tensors are copied into the storage
    of the same name (executor_base.cpp:82-95)."""

    def __init__(self, model, params=None):
        if isinstance(model, str):
            with open(model) as f:
                model = json.load(f)
        self.model = model
        self.storage = [np.zeros(int(s["size"]), STYPE_NP[s["stype"]]) for s in model["storage"]]
        if params is not None:
            if isinstance(params, str):
                params = read_params(params)
            for i, s in enumerate(model["storage"]):
                if s["name"] in params:
                    arr = params[s["name"]]
                    self.storage[i][:arr.size] = arr

    def find(self, name):
        for i, s in enumerate(self.model["storage"]):
            if s["name"] == name:
                return i
        raise KeyError(name)

    def set_input(self, name, value):
        i = self.find(name)
        self.storage[i][:] = np.asarray(value).reshape(-1).astype(self.storage[i].dtype)

    def get(self, name="output"):
        return self.storage[self.find(name)]

    def run(self, upto=None, acc64=False):
        ks = self.model["kernels"]
        for k in ks[:len(ks) if upto is None else upto]:
            self.run_kernel(k, acc64)
        return self.get("output") if any(s["name"] == "output" for s in self.model["storage"]) \
            else None

    def run_kernel(self, k, acc64=False):
        name, a = k["name"].split("#")[0], k.get("attrs", [])
        # "arg_offsets": the byte at which an operand starts inside its storage (views, so results
        # land in the storage)
        offs = k.get("arg_offsets") or [0] * len(k["args"])
        P = [self.storage[i][o // self.storage[i].itemsize:] for i, o in zip(k["args"], offs)]
        if name.startswith("reef_conv2d"):
            Cin, H, W, Cout, Ho, Wo, kh, kw, sh, sw, ph, pw, flags, act, _tile, split_k = a[:16]
            act2 = a[19] if len(a) > 19 else 0   # a[20]: first sync counter (device detail)
            dst_off = a[22] if len(a) > 22 else 0  # a[21]: loader family (device detail)
            xin = P[0][:Cin * H * W].reshape(Cin, H, W)
            wgt = P[1][:Cout * Cin * kh * kw].reshape(Cout, Cin, kh, kw)
            if flags & 32:
                # pre-activation: the layer reads relu(in * scale[c] + shift[c]); the two vectors
                # follow the optional operands (a plain split-K launch has none)
                plain = split_k > 1 and not (flags & 16)
                pos = 3 if plain else 3 + bool(flags & 1) + bool(flags & 2) + 2 * bool(flags & 4) + 2 * bool(flags & 8)
                ps = P[pos][:Cin].astype(np.float64)[:, None, None]
                pt = P[pos + 1][:Cin].astype(np.float64)[:, None, None]
                xin = np.maximum(xin.astype(np.float64) * ps + pt, 0.0).astype(np.float32)
            if split_k > 1 and not (flags & 16):
                # Plain split-K: the partial sums are an implementation detail of the
                # device kernel; the oracle computes the whole convolution into slot 0
                # of the workspace and leaves the other slots zero, which the ordered
                # reduce then folds to the same mathematical result.
                ws = P[2].view(np.float32)
                ws[:split_k * Cout * Ho * Wo] = 0
                out = conv2d(xin, wgt, stride=(sh, sw), pad=(ph, pw), acc64=acc64)
                ws[:out.size] = out.reshape(-1)
                return
            # single pass, or split-K folded inside the kernel (workspace untouched here)
            bias, res, scale, shift, out2, shift2 = self._conv_opt(P, 3, flags)
            if flags & 128:
                # a depthwise 3x3 stage (padding 1, + bias, activation act2) behind the front filter, in
                # the same launch; its weights and bias follow the optional operands.  Behind a 1x1 front
                # filter the stride attributes are the depthwise stage's and the filter has stride 1;
                # behind a larger one they are the filter's and the depthwise stage has stride 1.
                pos = 3 + bool(flags & 1) + bool(flags & 2) + 2 * bool(flags & 4) + 2 * bool(flags & 8)
                front, behind = ((1, 1), (sh, sw)) if kh == 1 and kw == 1 else ((sh, sw), (1, 1))
                mid = conv2d(xin, wgt, bias, None, None, None, front, (ph, pw), 1, act, 6.0, acc64)
                out = conv2d(mid, P[pos][:Cout * 9].reshape(Cout, 1, 3, 3), P[pos + 1][:Cout], stride=behind,
                             pad=(1, 1), groups=Cout, act=act2, acc64=acc64)
                assert out.shape == (Cout, Ho, Wo)
                if flags & 4096:
                    # and a linear 1x1 projection (+ bias) behind that; such a launch has no counters and
                    # the slot of the first counter carries the projection's output channels
                    Pn = a[20]
                    out = conv2d(out, P[pos + 2][:Pn * Cout].reshape(Pn, Cout, 1, 1), P[pos + 3][:Pn], acc64=acc64)
            elif flags & 256:
                # a 3x3 / stride 2 / padding 1 max-pool behind the convolution in the same launch (Ho, Wo
                # are the pooled sizes); optionally a per-channel shift on the input -- inside the image,
                # the convolution's padding stays zero, as when the shift is a launch of its own -- and
                # one behind the pool, with the pool's activation act2
                pos = 3 + bool(flags & 1)
                if flags & 512:
                    xin = eltwise(xin.reshape(Cin, -1), shift=P[pos][:Cin]).reshape(Cin, H, W)
                    pos += 1
                mid = conv2d(xin, wgt, bias, None, None, None, (sh, sw), (ph, pw), 1, act, 6.0, acc64)
                out = pool2d(mid, (3, 3), (2, 2), (1, 1), 0, P[pos][:Cout] if flags & 1024 else None, act2)
                assert out.shape == (Cout, Ho, Wo)
            else:
                out = conv2d(xin, wgt, bias,
                             None if res is None else res[:Cout * Ho * Wo].reshape(Cout, Ho, Wo),
                             scale, shift, (sh, sw), (ph, pw), 1, act, 6.0, acc64)
            if flags & 2048:      # the global average of the layer's output instead of the output
                P[2][:Cout] = global_avgpool(out.reshape(Cout, -1))
                return
            P[2][dst_off:dst_off + out.size] = out.reshape(-1)
            if out2 is not None:
                out2[dst_off:dst_off + out.size] = eltwise(out.reshape(Cout, -1), shift=shift2[:Cout],
                                                           act=act2).reshape(-1)
        elif name == "reef_splitk_reduce":
            M, N, split_k, flags, act = a[:5]
            act2 = a[5] if len(a) > 5 else 0
            dst_off = a[6] if len(a) > 6 else 0
            bias, res, scale, shift, out2, shift2 = self._conv_opt(P, 2, flags)
            acc = np.zeros(M * N, np.float32)
            ws = P[0].view(np.float32)
            for s in range(split_k):
                acc = acc + ws[s * M * N:(s + 1) * M * N]
            v = acc.reshape(M, N)
            if res is not None:
                v = v + res[:M * N].reshape(M, N)
            if bias is not None:
                v = v + bias[:M, None]
            if scale is not None:
                v = (v.astype(np.float64) * scale[:M, None] + shift[:M, None]).astype(np.float32)
            if act == 1:
                v = np.maximum(v, 0)
            elif act == 2:
                v = np.minimum(np.maximum(v, 0), 6.0)
            v = v.astype(np.float32)
            P[1][dst_off:dst_off + M * N] = v.reshape(-1)
            if out2 is not None:
                out2[dst_off:dst_off + M * N] = eltwise(v, shift=shift2[:M], act=act2).reshape(-1)
        elif name == "reef_dwconv2d":
            C, H, W, Ho, Wo, kh, kw, sh, sw, ph, pw, flags, act = a[:13]
            bias = P[3] if flags & 1 else None
            out = conv2d(P[0][:C * H * W].reshape(C, H, W), P[1][:C * kh * kw].reshape(C, 1, kh, kw),
                         bias, stride=(sh, sw), pad=(ph, pw), groups=C, act=act, acc64=acc64)
            P[2][:out.size] = out.reshape(-1)
        elif name == "reef_pool2d":
            C, H, W, Ho, Wo, kh, kw, sh, sw, ph, pw, mode, cpad, flags, act = a[:15]
            bias = P[2] if flags & 1 else None
            xin = P[0][:C * H * W].reshape(C, H, W)
            if flags & 2:       # read through relu(in * scale[c] + shift[c])
                pp = 2 + (flags & 1)
                xin = eltwise(xin.reshape(C, -1), scale=P[pp][:C], shift=P[pp + 1][:C], act=1).reshape(C, H, W)
            out = pool2d(xin, (kh, kw), (sh, sw), (ph, pw), mode, bias,
                         act, bool(cpad), (Ho, Wo))
            P[1][:out.size] = out.reshape(-1)
        elif name == "reef_global_avgpool":
            C, HW = a[:2]
            xin = P[0][:C * HW].reshape(C, HW)
            if len(a) > 2 and a[2] & 1:       # read through relu(in * scale[c] + shift[c])
                xin = eltwise(xin, scale=P[2][:C], shift=P[3][:C], act=1)
            P[1][:C] = global_avgpool(xin)
        elif name == "reef_eltwise":
            C, inner, flags, act = a[:4]
            b, scale, shift = _opt(P, 2, flags, (1, 2, 4))
            n = C * inner
            out = eltwise(P[0][:n].reshape(C, inner), None if b is None else b[:n].reshape(C, inner),
                          scale, shift, act)
            P[1][:n] = out.reshape(-1)
        elif name == "reef_dense":
            rows, in_f, out_f, flags, act = a[:5]
            bias = P[3] if flags & 1 else None
            y = dense(P[0][:rows * in_f].reshape(rows, in_f), P[1][:out_f * in_f].reshape(out_f, in_f),
                      bias, act, acc64)
            P[2][:y.size] = y.reshape(-1)
        elif name == "reef_softmax":
            rows, cols = a[:2]
            mask = P[2].view(np.uint8)[:cols] if len(a) > 2 and a[2] & 1 else None
            P[1][:rows * cols] = softmax(P[0][:rows * cols].reshape(rows, cols), mask).reshape(-1)
        elif name == "reef_layernorm":
            rows, cols, flags, eps_bits = a[:4]
            res = P[4][:rows * cols].reshape(rows, cols) if flags & 1 else None
            y = layernorm(P[0][:rows * cols].reshape(rows, cols), P[1][:cols], P[2][:cols], res,
                          _bits_to_float(eps_bits))
            P[3][:y.size] = y.reshape(-1)
        elif name == "reef_bias_gelu":
            rows, cols, flags = a[:3]
            bias = P[2] if flags & 1 else None
            P[1][:rows * cols] = bias_gelu(P[0][:rows * cols].reshape(rows, cols), bias).reshape(-1)
        elif name == "reef_embedding":
            seq, hidden, flags, vocab = a[:4]
            pos, seg = _opt(P, 3, flags, (1, 2))
            y = embedding(P[0][:seq], P[1][:vocab * hidden].reshape(vocab, hidden),
                          None if pos is None else pos[:seq * hidden].reshape(seq, hidden), seg)
            P[2][:y.size] = y.reshape(-1)
        elif name == "reef_copy":
            count, dst_off = a[:2]
            P[1][dst_off:dst_off + count] = P[0][:count]
        elif name == "reef_transpose":
            d0, d1, d2, flags = a[:4]
            bias = P[2] if flags & 1 else None
            y = transpose_102(P[0][:d0 * d1 * d2].reshape(d0, d1, d2), bias)
            P[1][:y.size] = y.reshape(-1)
        elif name.startswith("reef_gemm"):
            (batch, M, N, K, trans_b, flags, act, alpha_bits, _t, _mt, _nt, lda, ldb, ldc, sA, sB,
             sC) = a[:17]
            oA, oB, oC = (list(a[17:20]) + [0, 0, 0])[:3]     # absent = 0 (include/reef_kernels.h)
            alpha = _bits_to_float(alpha_bits)
            bias = P[3] if flags & 1 else None
            A, B, C = P[0][oA:], P[1][oB:], P[2][oC:]
            p = 3 + (flags & 1)
            R = None
            if flags & 8:                                     # residual, laid out as C is
                R = P[p][oC:]
                p += 1
            if flags & 2:
                # reef_gemm_ntl_*: LayerNorm of the rows of A, then the product with W -- the weights as
                # the reference has them, which the model keeps under the name of the scaled copy
                # without its "gk"; the scaled copy and the two vectors the kernel works from
                # (include/reef_kernels.h) are not used here
                gamma, beta = P[p + 2][:K], P[p + 3][:K]
                rows = np.ascontiguousarray(np.lib.stride_tricks.as_strided(A, (M, K), (lda * 4, 4)))
                normed = layernorm(rows, gamma, beta, None, _bits_to_float(a[20]))
                if flags & 4:
                    np.lib.stride_tricks.as_strided(P[p + 4], (M, K), (lda * 4, 4))[:, :] = normed
                A, lda = normed.reshape(-1), K
                wname = self.model["storage"][k["args"][1]]["name"]
                assert wname.endswith("gk"), wname
                B = self.storage[[t["name"] for t in self.model["storage"]].index(wname[:-2])]
            for bi in range(batch):
                Am = np.lib.stride_tricks.as_strided(A[bi * sA:], (M, K), (lda * 4, 4))
                if trans_b:
                    Bm = np.lib.stride_tricks.as_strided(B[bi * sB:], (N, K), (ldb * 4, 4))
                else:
                    Bm = np.lib.stride_tricks.as_strided(B[bi * sB:], (K, N), (ldb * 4, 4))
                c = batch_matmul(np.ascontiguousarray(Am)[None], np.ascontiguousarray(Bm)[None],
                                 bool(trans_b), alpha, acc64)[0]
                if bias is not None:
                    c = c + bias[:N][None, :]
                if act == 1:
                    c = np.maximum(c, 0)
                elif act == 3:
                    c = bias_gelu(c)
                if R is not None:
                    c = c + np.lib.stride_tricks.as_strided(R[bi * sC:], (M, N), (ldc * 4, 4))
                Cm = np.lib.stride_tricks.as_strided(C[bi * sC:], (M, N), (ldc * 4, 4))
                Cm[:, :] = c
        elif name == "reef_attention":
            # softmax(alpha Q K^T (masked)) V per head; Q, K, V column blocks of one [seq][ld] tensor
            S, HD, heads, ld, ldo, oq, ok, ov, alpha_bits, flags = a[:10]
            alpha = _bits_to_float(alpha_bits)
            qkv = P[0][:S * ld].reshape(S, ld)
            mask = P[2].view(np.uint8)[:S] if flags & 1 else None
            out = P[1][:S * ldo].reshape(S, ldo)
            for h in range(heads):
                q, kk, v = (np.ascontiguousarray(qkv[:, o + h * HD:o + (h + 1) * HD]) for o in (oq, ok, ov))
                sc = batch_matmul(q[None], kk[None], True, alpha, acc64)[0]
                pr = softmax(sc, mask)
                out[:, h * HD:(h + 1) * HD] = batch_matmul(pr[None], v[None], False, 1.0, acc64)[0]
        elif name in ("add", "multiply"):
            lp = k["launch_params"]
            blocks, threads = lp[0] * lp[1] * lp[2], lp[3] * lp[4] * lp[5]
            P[2][:blocks * threads] = mocked(P[0], P[1], name == "multiply", blocks, threads)
        else:
            raise NotImplementedError(name)

    @staticmethod
    def _conv_opt(P, pos, flags):
        """bias, residual, (scale, shift), (out2, shift2) follow the fixed operands in flag order."""
        bias = res = scale = shift = out2 = shift2 = None
        if flags & 1:
            bias = P[pos]
            pos += 1
        if flags & 2:
            res = P[pos]
            pos += 1
        if flags & 4:
            scale, shift = P[pos], P[pos + 1]
            pos += 2
        if flags & 8:
            out2, shift2 = P[pos], P[pos + 1]
        return bias, res, scale, shift, out2, shift2
