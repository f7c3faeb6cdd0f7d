"""Pins the CPU oracle: brute-force definitions on tiny shapes, algebraic
invariants, and torch.nn.functional in fp64 on the CPU.  Each check is chosen
so that a dropped term, a wrong index or a transposed operand fails it."""
import itertools
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O

RNG = np.random.default_rng(1234)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def brute_conv(x, w, stride, pad, groups):
    Cin, H, W = x.shape
    Cout, cpg, kh, kw = w.shape
    Ho = (H + 2 * pad[0] - kh) // stride[0] + 1
    Wo = (W + 2 * pad[1] - kw) // stride[1] + 1
    out = np.zeros((Cout, Ho, Wo), np.float64)
    opg = Cout // groups
    for o, y, xx in itertools.product(range(Cout), range(Ho), range(Wo)):
        g = o // opg
        s = 0.0
        for c, ky, kx in itertools.product(range(cpg), range(kh), range(kw)):
            iy, ix = y * stride[0] + ky - pad[0], xx * stride[1] + kx - pad[1]
            if 0 <= iy < H and 0 <= ix < W:
                s += float(x[g * cpg + c, iy, ix]) * float(w[o, c, ky, kx])
        out[o, y, xx] = s
    return out


@pytest.mark.parametrize("Cin,H,W,Cout,k,s,p,g", [
    (3, 5, 7, 4, (3, 3), (1, 1), (1, 1), 1),
    (4, 6, 5, 6, (1, 1), (2, 2), (0, 0), 1),
    (2, 9, 8, 3, (7, 7), (2, 2), (3, 3), 1),
    (4, 5, 5, 4, (3, 3), (2, 2), (1, 1), 4),   # depthwise
    (6, 7, 6, 4, (1, 7), (1, 1), (0, 3), 2),   # asymmetric kernel, grouped
    (3, 6, 7, 2, (5, 3), (2, 1), (2, 0), 1),   # asymmetric stride and pad
])
def test_conv_brute_force(Cin, H, W, Cout, k, s, p, g):
    x, w = rnd(Cin, H, W), rnd(Cout, Cin // g, *k)
    ref = brute_conv(x, w, s, p, g)
    for acc64 in (False, True):
        got = O.conv2d(x, w, stride=s, pad=p, groups=g, acc64=acc64)
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("Cin,H,W,Cout,k,s,p,g", [
    (16, 14, 14, 32, (3, 3), (1, 1), (1, 1), 1),
    (32, 28, 28, 24, (1, 1), (2, 2), (0, 0), 1),
    (3, 32, 32, 8, (7, 7), (2, 2), (3, 3), 1),
    (24, 17, 17, 24, (3, 3), (2, 2), (1, 1), 24),
    (12, 17, 17, 20, (7, 1), (1, 1), (3, 0), 1),
])
def test_conv_vs_torch_fp64(Cin, H, W, Cout, k, s, p, g):
    x, w = rnd(Cin, H, W), rnd(Cout, Cin // g, *k)
    ref = F.conv2d(torch.from_numpy(x).double()[None], torch.from_numpy(w).double(), None, s, p, 1,
                   g)[0].numpy()
    got = O.conv2d(x, w, stride=s, pad=p, groups=g)
    np.testing.assert_allclose(got, ref, rtol=2e-5, atol=2e-5)
    got64 = O.conv2d(x, w, stride=s, pad=p, groups=g, acc64=True)
    np.testing.assert_allclose(got64, ref, rtol=1e-6, atol=1e-6)


def test_conv_epilogue_order():
    """relu(fma((acc + res) + bias, scale, shift)); each operand must matter."""
    x, w = rnd(4, 6, 6), rnd(5, 4, 3, 3)
    bias, res, scale, shift = rnd(5), rnd(5, 6, 6), rnd(5), rnd(5)
    acc = brute_conv(x, w, (1, 1), (1, 1), 1)
    full = np.maximum((acc + res + bias[:, None, None]) * scale[:, None, None] + shift[:, None, None], 0)
    got = O.conv2d(x, w, bias, res, scale, shift, pad=(1, 1), act=1)
    np.testing.assert_allclose(got, full, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(O.conv2d(x, w, bias, pad=(1, 1), act=1),
                               np.maximum(acc + bias[:, None, None], 0), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(O.conv2d(x, w, None, res, pad=(1, 1)), acc + res, rtol=1e-5, atol=1e-5)
    r6 = O.conv2d(x * 10, w, bias, pad=(1, 1), act=2)
    assert r6.min() >= 0 and r6.max() <= 6.0 and (r6 == 6.0).any()


def test_conv_linearity_and_1x1_is_gemm():
    x1, x2, w = rnd(8, 9, 9), rnd(8, 9, 9), rnd(6, 8, 3, 3)
    a = O.conv2d(x1 + 2 * x2, w, pad=(1, 1), acc64=True)
    b = O.conv2d(x1, w, pad=(1, 1), acc64=True) + 2 * O.conv2d(x2, w, pad=(1, 1), acc64=True)
    np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-4)
    w1 = rnd(6, 8, 1, 1)
    np.testing.assert_allclose(O.conv2d(x1, w1), (w1[:, :, 0, 0].astype(np.float64) @
                               x1.reshape(8, -1).astype(np.float64)).reshape(6, 9, 9), rtol=1e-5, atol=1e-5)


def test_dense_and_gelu():
    x, w, b = rnd(3, 17), rnd(5, 17), rnd(5)
    ref = x.astype(np.float64) @ w.astype(np.float64).T + b
    np.testing.assert_allclose(O.dense(x, w, b), ref, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(O.dense(x, w, b, act=1), np.maximum(ref, 0), rtol=1e-5, atol=1e-5)
    g = F.gelu(torch.from_numpy(ref), approximate="none").numpy()
    np.testing.assert_allclose(O.dense(x, w, b, act=3), g, rtol=1e-5, atol=1e-5)
    # closed-form points of the erf GELU
    pts = np.array([[0.0, 1.0, -1.0]], np.float32)
    want = [0.0, 0.5 * (1 + math.erf(1 / math.sqrt(2))), -0.5 * (1 + math.erf(-1 / math.sqrt(2)))]
    np.testing.assert_allclose(O.bias_gelu(pts)[0], want, rtol=1e-6, atol=1e-7)
    xb, bb = rnd(4, 6), rnd(6)
    np.testing.assert_allclose(O.bias_gelu(xb, bb),
                               F.gelu(torch.from_numpy(xb + bb).double()).numpy(), rtol=1e-5, atol=1e-6)


def test_batch_matmul_both_layouts():
    a, b = rnd(3, 5, 7), rnd(3, 4, 7)
    ref = np.einsum("bmk,bnk->bmn", a.astype(np.float64), b.astype(np.float64))
    np.testing.assert_allclose(O.batch_matmul(a, b, True, 0.5), 0.5 * ref, rtol=1e-5, atol=1e-5)
    b2 = rnd(3, 7, 4)
    ref2 = np.einsum("bmk,bkn->bmn", a.astype(np.float64), b2.astype(np.float64))
    np.testing.assert_allclose(O.batch_matmul(a, b2, False), ref2, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("mode,k,s,p,cpad", [(0, (3, 3), (2, 2), (1, 1), False),
                                           (1, (2, 2), (2, 2), (0, 0), False),
                                           (1, (3, 3), (1, 1), (1, 1), True),
                                           (1, (3, 3), (1, 1), (1, 1), False)])
def test_pool_vs_torch(mode, k, s, p, cpad):
    x = rnd(5, 9, 11)
    t = torch.from_numpy(x).double()[None]
    if mode == 0:
        ref = F.max_pool2d(t, k, s, p)[0].numpy()
    else:
        ref = F.avg_pool2d(t, k, s, p, count_include_pad=cpad)[0].numpy()
    np.testing.assert_allclose(O.pool2d(x, k, s, p, mode, count_include_pad=cpad), ref, rtol=1e-6,
                               atol=1e-6)


def test_maxpool_pads_with_lowest_and_bias_relu():
    x = -np.abs(rnd(2, 4, 4)) - 1.0       # all negative: zero padding would win if used
    out = O.pool2d(x, (3, 3), (2, 2), (1, 1), 0)
    assert (out < 0).all()
    bias = np.array([10.0, -100.0], np.float32)
    out2 = O.pool2d(x, (3, 3), (2, 2), (1, 1), 0, bias=bias, act=1)
    np.testing.assert_allclose(out2[0], out[0] + 10.0, rtol=1e-6)
    assert (out2[1] == 0).all()


def test_global_avgpool_softmax_layernorm():
    x = rnd(6, 49)
    np.testing.assert_allclose(O.global_avgpool(x), x.astype(np.float64).mean(1), rtol=1e-5, atol=1e-6)
    s = rnd(7, 1000) * 5
    sm = O.softmax(s)
    np.testing.assert_allclose(sm.sum(1), 1.0, rtol=1e-5)
    np.testing.assert_allclose(sm, F.softmax(torch.from_numpy(s).double(), 1).numpy(), rtol=1e-4, atol=1e-9)
    # shift invariance and no overflow for large logits
    np.testing.assert_allclose(O.softmax(s + 1000.0), sm, rtol=1e-3, atol=1e-7)
    h = rnd(5, 768)
    g, b, r = rnd(768), rnd(768), rnd(5, 768)
    ones, zeros = np.ones(768, np.float32), np.zeros(768, np.float32)
    plain = O.layernorm(h, ones, zeros, eps=1e-12)
    np.testing.assert_allclose(plain.mean(1), 0, atol=1e-5)
    np.testing.assert_allclose(plain.var(1), 1, rtol=1e-4)
    ref = F.layer_norm(torch.from_numpy(h + r).double(), (768,), torch.from_numpy(g).double(),
                       torch.from_numpy(b).double(), 1e-12).numpy()
    np.testing.assert_allclose(O.layernorm(h, g, b, r, 1e-12), ref, rtol=1e-4, atol=1e-5)


def test_eltwise_embedding_transpose_mocked():
    a, b = rnd(4, 10), rnd(4, 10)
    sc, sh = rnd(4), rnd(4)
    np.testing.assert_allclose(O.eltwise(a, b, sc, sh, act=1),
                               np.maximum((a + b) * sc[:, None] + sh[:, None], 0), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(O.eltwise(a, shift=sh), a + sh[:, None], rtol=1e-6)
    ids = np.array([3, 0, 7, 7], np.int64)
    tok, pos, seg = rnd(9, 6), rnd(4, 6), rnd(6)
    np.testing.assert_allclose(O.embedding(ids, tok, pos, seg), tok[ids] + pos + seg, rtol=1e-6)
    t = rnd(3, 4, 5)
    np.testing.assert_array_equal(O.transpose_102(t), t.transpose(1, 0, 2))
    bias = rnd(4, 5)
    np.testing.assert_allclose(O.transpose_102(t, bias), (t + bias[None]).transpose(1, 0, 2), rtol=1e-6)
    three = np.full(8192, 3.0, np.float32)
    tmp = O.mocked(three, three, False)
    np.testing.assert_array_equal(O.mocked(tmp, three, True), np.full(8192, 18.0, np.float32))


def test_masked_softmax_is_the_where_kernel_in_front_of_the_softmax():
    """The reference's attention mask (resource/bert/bert.cu:381-388): where(mask[col], -inf, x)
    on the scores, then the softmax.  Against torch; masked columns get probability 0 exactly,
    an all-zero mask changes nothing, and the unmasked columns renormalise among themselves."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((12, 37)).astype(np.float32) * 3
    mask = (rng.random(37) < 0.3).astype(np.uint8)
    mask[0] = 0
    got = O.softmax(x, mask)
    want = F.softmax(torch.from_numpy(x).double().masked_fill(torch.from_numpy(mask.astype(bool)), -np.inf), 1).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-9)
    assert (got[:, mask != 0] == 0).all() and np.allclose(got.sum(1), 1, atol=1e-5)
    np.testing.assert_array_equal(O.softmax(x, np.zeros(37, np.uint8)), O.softmax(x))
    keep = mask == 0
    np.testing.assert_allclose(got[:, keep], O.softmax(x[:, keep]), rtol=1e-6, atol=1e-9)


def test_reciprocal_division_of_the_kernels_is_exact_on_its_stated_range():
    """reef_common.hpp:div_small computes a / b for 0 <= a < 2^22, 0 < b < 2^22 as
    trunc(float(a) * rcp(float(b))) corrected by the sign and size of the remainder.  The
    hardware reciprocal is good to one unit in the last place: the same arithmetic in float32,
    with the reciprocal pushed one unit either way, must give the exact quotient everywhere it is
    probed (all small operands, random large ones, and the neighbours of every multiple)."""
    rng = np.random.default_rng(22)

    def div_small(a, b, nudge):
        rb = (np.float32(1.0) / b.astype(np.float32)).astype(np.float32)
        rb = np.nextafter(rb, np.float32(np.inf if nudge > 0 else -np.inf)) if nudge else rb
        q = (a.astype(np.float32) * rb).astype(np.float32).astype(np.int64)
        r = a - q * b
        return q + (r >= b) - (r < 0)

    small = np.arange(0, 2048, dtype=np.int64)
    a1, b1 = np.meshgrid(small, small[1:], indexing="ij")
    b2 = rng.integers(1, 1 << 22, 200000)
    a2 = rng.integers(0, 1 << 22, 200000)
    b3 = rng.integers(1, 5000, 200000)
    k3 = rng.integers(0, (1 << 22) // 5000, 200000)
    a3 = np.clip(b3 * k3 + rng.integers(-1, 2, 200000), 0, (1 << 22) - 1)     # around exact multiples
    for a, b in ((a1.ravel(), b1.ravel()), (a2, b2), (a3, b3)):
        for nudge in (-1, 0, 1):
            np.testing.assert_array_equal(div_small(a, b, nudge), a // b)
