"""GPU parity of every kernel family against the CPU oracle, through the C-ABI
(raw flavour, ExecutorBase).  Shapes cover the tile configurations, split-K,
ragged edges (M, N, K not multiples of the tile), strides, padding and the
fused epilogues."""
import numpy as np
import pytest

from reef_amd.modelgen import builder as MB
from reef_amd.modelgen import tiling
from tests.helpers import compare_storages, run_both

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(7)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def forced(tile, M, N, K, split, taps=1):
    return tiling.forced(tile, M, N, K, split, taps)


CONV_CASES = [
    # cin, H, W, cout, k, stride, pad
    (64, 14, 14, 64, 3, 1, 1),
    (32, 28, 28, 96, 1, 1, 0),
    (48, 28, 28, 80, 1, 2, 0),
    (3, 32, 32, 64, 7, 2, 3),        # K = 147, not a multiple of 4
    (24, 9, 11, 40, (1, 7), 1, (0, 3)),
    (24, 9, 11, 40, (7, 1), 1, (3, 0)),
    (16, 17, 17, 24, 5, 1, 2),
    (40, 15, 15, 136, 3, 2, 1),
    (256, 7, 7, 64, 3, 1, 1),        # N = 49
    (32, 8, 10, 48, (1, 3), 1, (0, 1)),
    (32, 10, 8, 48, (3, 1), 2, (1, 0)),
]


@pytest.mark.parametrize("tile", list(tiling.TILES))
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_tiles(tmp_path, tile, case):
    cin, H, W, cout, k, s, p = case
    g = MB.GraphBuilder("c")
    x = g.input("data", (cin, H, W))
    kh, kw = (k, k) if isinstance(k, int) else k
    ph, pw = (p, p) if isinstance(p, int) else p
    Ho, Wo = (H + 2 * ph - kh) // s + 1, (W + 2 * pw - kw) // s + 1
    if tile in tiling.DIRECT_TILES and not tiling.direct_ok(cin, kh, kw, tile):
        pytest.skip("the direct family is compiled for 1x1 (Cin % 8 == 0) and 3-, 7-, 9-tap filters, "
                    "its wide tiles for 1 and 9 taps")
    if tile in tiling.ROW_TILES:
        if not tiling.rows_ok(kh, kw, s, s, ph, pw):
            pytest.skip("the row form is compiled for 3x3 / stride 1 / padding 1")
        f = tiling.forced_rows(tile, cout, Ho, Wo, cin * 9, 1)
    else:
        f = forced(tile, cout, Ho * Wo, cin * kh * kw, 1, kh * kw)
    y = g.conv2d(x, cout, k, s, p, bias=True, act=MB.ACT_RELU, force=f)
    g.mark_output(y)
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W)})
    compare_storages(exe, orc, model, what="conv %s %s" % (tile, case))


@pytest.mark.parametrize("split", [2, 3, 8])
@pytest.mark.parametrize("tile", ["64x64", "128x64", "128x32", "32x32k4", "64x32k2", "32x64k2", "16x16k4"])
def test_conv_split_k_and_epilogues(tmp_path, tile, split):
    cin, H, W, cout = 96, 14, 14, 160
    g = MB.GraphBuilder("s")
    x = g.input("data", (cin, H, W))
    res = g.input("res", (cout, H, W))
    f = forced(tile, cout, H * W, cin * 9, split, 9)
    y1 = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU, force=f)
    y2 = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_NONE, residual=res, force=f)
    y3 = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU, residual=res, force=f)
    y4 = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_RELU, residual=res, affine=True, force=f)
    f1 = forced(tile, cout, H * W, cin * 9, 1, 9)
    y5 = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_RELU, residual=res, affine=True, force=f1)
    y6 = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU6, force=f1)
    g.mark_output(y6)
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W), "res": rnd(cout, H, W)})
    compare_storages(exe, orc, model, what="split-k %s x%d" % (tile, split))
    # split-K and single-pass results of the same layer agree to rounding
    a = exe.get_data(y4.idx, y4.size)
    b = exe.get_data(y5.idx, y5.size)
    # (different weights per conv, so only finiteness is common; shapes equal)
    assert a.shape == b.shape


@pytest.mark.parametrize("tile,split", [("64x64", 4), ("128x64", 6), ("128x32", 16), ("32x128", 3),
                                        ("64x128", 2), ("128x128", 2)])
def test_fused_split_k_equals_plain_split_k_bitwise(tmp_path, tile, split):
    """Split-K folded inside the kernel by the last-arriving workgroup sums the partial
    tiles in the same fixed order as the separate reduce launch: identical bits, also
    for the second (activated) output and on a rerun (counters reset themselves)."""
    cin, H, W, cout = 128, 14, 14, 192
    g = MB.GraphBuilder("f")
    x = g.input("data", (cin, H, W))
    res = g.input("res", (cout, H, W))
    f = forced(tile, cout, H * W, cin * 9, split)
    outs = {}
    for fused in (False, True):
        g._np = 0          # same parameter names -> same seeded weights for both variants
        a = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU, force=f, fused_reduce=fused)
        b, b2 = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_NONE, residual=res,
                         dual_act=MB.ACT_RELU, force=f, fused_reduce=fused)
        c = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_RELU, residual=res, affine=True,
                     force=f, fused_reduce=fused)
        outs[fused] = (a, b, b2, c)
    g.mark_output(outs[True][0])
    # both variants read the same parameter storages by name: keep one copy of each key
    seen = {}
    g.params = [kv for kv in g.params if not (kv[0] in seen or seen.setdefault(kv[0], 0))]
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W), "res": rnd(cout, H, W)})
    compare_storages(exe, orc, model, what="fused split-k %s x%d" % (tile, split))
    for rerun in range(2):
        for t_plain, t_fused in zip(outs[False], outs[True]):
            np.testing.assert_array_equal(exe.get_data(t_plain.idx, t_plain.size),
                                          exe.get_data(t_fused.idx, t_fused.size))
        exe.execute()


@pytest.mark.parametrize("split,fused", [(1, False), (2, False), (2, True), (5, True)])
@pytest.mark.parametrize("shape", [(72, 13, 13, 88), (40, 30, 37, 24), (32, 7, 7, 48), (16, 5, 50, 16)])
@pytest.mark.parametrize("tile", list(tiling.ROW_TILES))
def test_conv_row_form(tmp_path, tile, shape, split, fused):
    """Row form of the 3x3 / stride 1 / padding 1 convolution (G image rows x 14-column segments,
    horizontal taps from neighbouring lanes): images narrower and wider than a segment, widths
    that are no multiple of 14, heights that are no multiple of G, ragged M and Cin; every
    epilogue form, a second output and a channel slice; single pass, separate reduce, and the
    split folded inside the launch, which must give the bits of the separate reduce."""
    cin, H, W, cout = shape
    g = MB.GraphBuilder("r")
    x = g.input("data", (cin, H, W))
    res = g.input("res", (cout, H, W))
    f = tiling.forced_rows(tile, cout, H, W, cin * 9, split)
    if f["split_k"] != split:
        pytest.skip("too few channels for this split")
    fu = fused if split > 1 else None
    outs = {}
    for variant in ((False, True) if fused else (fused,)):
        g._np = 0
        v = variant if split > 1 else None
        a = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU, force=f, fused_reduce=v)
        b, b2 = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_NONE, residual=res,
                         dual_act=MB.ACT_RELU, force=f, fused_reduce=v)
        c = g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_RELU6, residual=res, affine=True,
                     force=f, fused_reduce=v)
        cat = g.temp((cout + 24, H, W))
        e = g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_NONE, force=f, fused_reduce=v, out=cat,
                     out_channel=16)
        outs[variant] = (a, b, b2, c, cat)
    g.mark_output(outs[fused][0])
    seen = {}
    g.params = [kv for kv in g.params if not (kv[0] in seen or seen.setdefault(kv[0], 0))]
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W), "res": rnd(cout, H, W)})
    compare_storages(exe, orc, model, what="row form %s %s x%d fused=%s" % (tile, shape, split, fused))
    if fused:
        for rerun in range(2):
            for t_plain, t_fused in zip(outs[False], outs[True]):
                np.testing.assert_array_equal(exe.get_data(t_plain.idx, t_plain.size),
                                              exe.get_data(t_fused.idx, t_fused.size))
            exe.execute()


@pytest.mark.parametrize("split,fused", [(1, False), (2, False), (2, True), (3, True)])
@pytest.mark.parametrize("tile", list(tiling.DIRECT_TILES))
def test_conv_direct_family_epilogues(tmp_path, tile, split, fused):
    """Direct-operand family (16 x 16/32/64 tiles, channels split over the wavefronts): every
    epilogue form, a second output, a channel slice of a concatenation buffer, ragged M / N / Cin,
    and a strided 1x1; without split-K, with a separate reduce launch, and with the split folded
    inside the launch.  The folded form must hold the same bits as the separate reduce (both
    add the partial tiles in ascending split order), also on a second run (counters reset)."""
    cin, H, W, cout = 72, 13, 13, 88          # Cin % 16 != 0, M % 16 != 0, N = 169
    g = MB.GraphBuilder("d")
    x = g.input("data", (cin, H, W))
    res = g.input("res", (cout, H, W))
    M, N = cout, H * W
    f9 = forced(tile, M, N, cin * 9, split, 9)
    f1 = forced(tile, M, N, cin, split, 1)
    Ho = (H - 1) // 2 + 1
    fs = forced(tile, M, Ho * Ho, cin, split, 1)

    def layers(fz):
        g._np = 0          # same parameter names -> same seeded weights for every variant
        outs = [g.conv2d(x, cout, 3, 1, 1, bias=True, act=MB.ACT_RELU, residual=res, force=f9, fused_reduce=fz),
                g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_RELU, residual=res, affine=True, force=f9,
                         fused_reduce=fz)]
        outs += list(g.conv2d(x, cout, 3, 1, 1, bias=False, act=MB.ACT_NONE, residual=res,
                              dual_act=MB.ACT_RELU, force=f9, fused_reduce=fz))
        outs.append(g.conv2d(x, cout, 1, 1, 0, bias=True, act=MB.ACT_RELU6, force=f1, fused_reduce=fz))
        outs += list(g.conv2d(x, cout, 1, 1, 0, bias=False, act=MB.ACT_NONE, residual=res,
                              dual_act=MB.ACT_RELU, force=f1, fused_reduce=fz))
        cat = g.temp((2 * cout, H, W))
        g.conv2d(x, cout, 3, 1, 1, force=f9, out=cat, out_channel=0, fused_reduce=fz)
        g.conv2d(x, cout, 1, 1, 0, force=f1, out=cat, out_channel=cout, fused_reduce=fz)
        outs.append(cat)
        outs.append(g.conv2d(x, cout, 1, 2, 0, force=fs, fused_reduce=fz))
        return outs

    first = layers(fused)
    plain = layers(False) if fused else None
    g.mark_output(first[-1])
    seen = {}
    g.params = [kv for kv in g.params if not (kv[0] in seen or seen.setdefault(kv[0], 0))]
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W), "res": rnd(cout, H, W)})
    compare_storages(exe, orc, model, what="direct family %s x%d%s" % (tile, split, " fused" if fused else ""))
    if fused:
        for rerun in range(2):
            for a, b in zip(first, plain):
                np.testing.assert_array_equal(exe.get_data(a.idx, a.size), exe.get_data(b.idx, b.size))
            exe.execute()


@pytest.mark.parametrize("split,fused", [(1, False), (2, False), (2, True)])
@pytest.mark.parametrize("tile", list(tiling.PRE_ACT_TILES))
def test_conv_pre_activation_folded_into_the_loads(tmp_path, tile, split, fused):
    """1x1 convolution that reads its input through a per-channel scale, shift and ReLU (the
    DenseNet pre-activation) inside its own loads: equals the oracle, which applies the
    pre-activation first, for ragged M / N / Cin, with a residual and second output, into a slice
    of a concatenation buffer, with plain and folded split-K."""
    cin, H, W, cout = 200, 13, 13, 88         # Cin % 128 != 0, M % 16 != 0, N = 169
    g = MB.GraphBuilder("p")
    x = g.input("data", (cin, H, W))
    res = g.input("res", (cout, H, W))
    f = forced(tile, cout, H * W, cin, split, 1)
    g.conv2d(x, cout, 1, 1, 0, bias=True, act=MB.ACT_RELU, force=f, fused_reduce=fused, pre_act=True)
    g.conv2d(x, cout, 1, 1, 0, bias=False, act=MB.ACT_NONE, residual=res, dual_act=MB.ACT_RELU, force=f,
             fused_reduce=fused, pre_act=True)
    cat = g.temp((2 * cout, H, W))
    g.conv2d(x, cout, 1, 1, 0, force=f, out=cat, out_channel=cout, fused_reduce=fused, pre_act=True)
    # a filter the folded form does not cover falls back to a separate elementwise launch
    y = g.conv2d(x, cout, 3, 1, 1, force=forced(tile, cout, H * W, cin * 9, 1, 9), pre_act=True)
    g.mark_output(y)
    names = [k["name"].split("#")[0] for k in g.kernels]
    assert names.count("reef_conv2d_p1_" + tile) == 3 and names.count("reef_eltwise") == 1
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(cin, H, W), "res": rnd(cout, H, W)})
    compare_storages(exe, orc, model, what="pre-activation %s x%d%s" % (tile, split, " fused" if fused else ""))


def test_conv_auto_heuristic_shapes(tmp_path):
    """The layer shapes of ResNet-152 at reduced channel counts, tiles picked by the generator."""
    g = MB.GraphBuilder("h")
    x = g.input("data", (64, 56, 56))
    a = g.conv2d(x, 64, 1, 1, 0)
    b = g.conv2d(a, 64, 3, 1, 1)
    c = g.conv2d(b, 256, 1, 1, 0, bias=False, act=MB.ACT_NONE)
    d = g.conv2d(c, 128, 1, 2, 0)
    e = g.conv2d(d, 128, 3, 1, 1)
    f = g.conv2d(e, 512, 1, 1, 0)
    h = g.conv2d(f, 256, 1, 2, 0)
    i = g.conv2d(h, 256, 3, 1, 1)
    j = g.conv2d(i, 1024, 1, 1, 0)
    k = g.conv2d(j, 512, 1, 2, 0)
    l = g.conv2d(k, 512, 3, 1, 1)
    m = g.conv2d(l, 2048, 1, 1, 0)
    g.mark_output(m)
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(64, 56, 56)})
    compare_storages(exe, orc, model, what="resnet shapes")


def test_bandwidth_ops(tmp_path):
    g = MB.GraphBuilder("b")
    x = g.input("data", (24, 19, 23))
    p1 = g.pool2d(x, 3, 2, 1, "max", bias=True, act=MB.ACT_RELU)
    p2 = g.pool2d(x, 2, 2, 0, "avg")
    p3 = g.pool2d(x, 3, 1, 1, "avg", count_include_pad=False)
    p4 = g.pool2d(x, 3, 1, 1, "avg", count_include_pad=True)
    e1 = g.eltwise(x, shift=True)
    e2 = g.eltwise(x, b=e1, scale=True, shift=True, act=MB.ACT_RELU)
    x4 = g.input("x4", (16, 8, 8))             # inner % 4 == 0 -> vector path
    e3 = g.eltwise(x4, b=x4, shift=True, act=MB.ACT_RELU6)
    d1 = g.dwconv2d(x, 3, 1, 1)
    d2 = g.dwconv2d(x, 3, 2, 1, act=MB.ACT_RELU)
    gp = g.global_avgpool(x)
    dn = g.dense(gp, 37, bias=True)
    dn2 = g.dense(x4, 50, bias=True, act=MB.ACT_RELU)     # in_f = 1024, vector path
    sm = g.softmax(dn, 1, 37)
    g.mark_output(sm)
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(24, 19, 23), "x4": rnd(16, 8, 8)})
    compare_storages(exe, orc, model, what="bandwidth ops")
    out = exe.get_output()
    assert abs(out.sum() - 1.0) < 1e-5


def test_transformer_ops(tmp_path):
    seq, hid, heads, vocab = 24, 96, 4, 211
    hd = hid // heads
    g = MB.GraphBuilder("t", weight_std=0.05)
    ids = g.input("input0", (seq,), "int64")
    emb = g.embedding(ids, vocab, seq, hid)
    ln0 = g.layernorm(emb, seq, hid)
    wq = g.param((hid, hid), 0.05)
    bq = g.param((hid,), 0.02)
    q = g.gemm(ln0, wq, seq, hid, hid, trans_b=True, bias=bq)                # [seq, hid]
    qh = g.transpose_102(q, seq, heads, hd)                                   # [heads, seq, hd]
    scores = g.gemm(qh, qh, seq, seq, hd, batch=heads, trans_b=True, alpha=0.25,
                    stride_a=seq * hd, stride_b=seq * hd, stride_c=seq * seq)  # Q.K^T
    amask = g.input("attention_mask", (seq,), "uint1")
    pr = g.softmax(scores, heads * seq, seq, mask=amask)      # key positions 19.. are padding
    ctx = g.gemm(pr, qh, seq, hd, seq, batch=heads, trans_b=False,
                 stride_a=seq * seq, stride_b=seq * hd, stride_c=seq * hd)     # P.V
    merged = g.transpose_102(ctx, heads, seq, hd)                              # [seq, heads, hd]
    ln1 = g.layernorm(merged, seq, hid, res=ln0)
    w1 = g.param((4 * hid, hid), 0.05)
    h1 = g.gemm(ln1, w1, seq, 4 * hid, hid, trans_b=True)
    act = g.bias_gelu(h1, seq, 4 * hid)
    w2 = g.param((hid, 4 * hid), 0.05)
    b2 = g.param((hid,), 0.02)
    h2 = g.gemm(act, w2, seq, hid, 4 * hid, trans_b=True, bias=b2, act=MB.ACT_GELU)
    cat = g.temp((2, seq, hid))
    g.copy_into(h2, cat, 0)
    g.copy_into(ln1, cat, seq * hid)
    g.mark_output(cat)
    token_ids = RNG.integers(0, vocab, seq).astype(np.int64)
    pad = np.zeros(seq, np.uint8)
    pad[19:] = 1
    exe, orc, model = run_both(g, tmp_path, {"input0": token_ids, "attention_mask": pad})
    compare_storages(exe, orc, model, what="transformer ops")
    probs = exe.get_data(pr.idx, heads * seq * seq).reshape(heads * seq, seq)
    assert (probs[:, 19:] == 0).all() and np.allclose(probs.sum(1), 1, atol=1e-5)


@pytest.mark.parametrize("tile", list(tiling.GEMM_DIRECT_TILES))
def test_gemm_nt_direct_tiles(tmp_path, tile):
    """C = act(alpha A B^T + bias) with both operands loaded straight into the matrix cores:
    ragged M and N, K not a multiple of the 128-wide step, bias + GELU, alpha, a batched product
    over strided views (the Q K^T of an attention head: lda = ldb = hidden > K)."""
    seq, hid, heads = 40, 200, 5          # M = 40 (2.5 row groups), K = 200 = 128 + 72
    hd = hid // heads                     # 40: K of the batched product, one partial step
    g = MB.GraphBuilder("gd", weight_std=0.05)
    x = g.input("x", (seq, hid))
    w = g.param((3 * hid + 8, hid), 0.05)                 # N = 608: ragged against 16 / 32
    bias = g.param((3 * hid + 8,), 0.02)
    y = g.gemm(x, w, seq, 3 * hid + 8, hid, trans_b=True, bias=bias, act=MB.ACT_GELU, force_tile=tile)
    z = g.gemm(x, w, seq, 3 * hid + 8, hid, trans_b=True, alpha=0.5, force_tile=tile)
    # heads as strided views of x: A[b] = x[:, b*hd:(b+1)*hd], same for B; C[b] = [seq, seq]
    s_ = g.gemm(x, x, seq, seq, hd, batch=heads, trans_b=True, alpha=0.25, lda=hid, ldb=hid,
                stride_a=hd, stride_b=hd, stride_c=seq * seq, force_tile=tile)
    g.mark_output(s_)
    assert all(k["name"].startswith("reef_gemm_ntd_" + tile) for k in g.kernels)
    exe, orc, model = run_both(g, tmp_path, {"x": rnd(seq, hid)})
    compare_storages(exe, orc, model, what="direct gemm " + tile)


def test_gemm_operands_at_offsets_inside_one_storage(tmp_path):
    """Q, K and V as the column blocks of ONE [seq][3 * hidden] projection (attrs offA/offB/offC):
    Q K^T on every direct tile and on a staged one, P V reading V at its offset and writing the
    context into the second half of a larger buffer.  Checked against the oracle and, for the
    offsets themselves, against numpy on the slices."""
    seq, hid, heads = 40, 96, 4
    hd = hid // heads                                     # 24
    g = MB.GraphBuilder("go", weight_std=0.05)
    x = g.input("x", (seq, hid))
    w = g.param((3 * hid, hid), 0.05)
    bias = g.param((3 * hid,), 0.02)
    qkv = g.gemm(x, w, seq, 3 * hid, hid, trans_b=True, bias=bias)
    kw = dict(batch=heads, trans_b=True, alpha=0.25, lda=3 * hid, ldb=3 * hid, stride_a=hd, stride_b=hd,
              stride_c=seq * seq, off_b=hid)
    scores = [g.gemm(qkv, qkv, seq, seq, hd, force_tile=t, **kw) for t in list(tiling.GEMM_DIRECT_TILES) + ["32x32k4"]]
    assert [k["name"].split("_")[2] for k in g.kernels[1:]] == ["ntd"] * len(tiling.GEMM_DIRECT_TILES) + ["nt"]
    probs = g.softmax(scores[0], heads * seq, seq)
    both = g.temp((2, seq, hid))
    g.gemm(probs, qkv, seq, hd, seq, batch=heads, trans_b=False, lda=seq, ldb=3 * hid, ldc=hid,
           stride_a=seq * seq, stride_b=hd, stride_c=hd, out=both, off_b=2 * hid, off_c=seq * hid)
    g.mark_output(both)
    exe, orc, model = run_both(g, tmp_path, {"x": rnd(seq, hid)})
    compare_storages(exe, orc, model, what="gemm operands at offsets")
    m = exe.get_data(qkv.idx, seq * 3 * hid).reshape(seq, 3, heads, hd).astype(np.float64)
    want = 0.25 * np.einsum("shd,thd->hst", m[:, 0], m[:, 1])
    for s_ in scores:
        got = exe.get_data(s_.idx, heads * seq * seq).reshape(heads, seq, seq)
        assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    p_ = exe.get_data(probs.idx, heads * seq * seq).reshape(heads, seq, seq).astype(np.float64)
    ctx = np.einsum("hst,thd->shd", p_, m[:, 2]).reshape(seq, hid)
    out = exe.get_data(both.idx, 2 * seq * hid).reshape(2, seq, hid)
    assert (out[0] == 0).all() and np.abs(out[1] - ctx).max() <= 1e-5 * np.abs(ctx).max()


def test_operands_as_channel_ranges_of_a_larger_buffer(tmp_path):
    """Kernels read and write parts of a storage through `arg_offsets`: one 1x1 convolution with a
    stacked filter writes [reduction | branch] into a block buffer, a 5x5 and a 3x3 row-form
    convolution read the reduction as a channel range and write their slices, a max-pool writes
    its slice directly, the next layers (convolution, average pool, global average pool) read the
    concatenation as a range that starts inside the storage.  Against the oracle, and the
    concatenation against numpy slices of the oracle-independent pieces."""
    C, H, W = 24, 19, 19
    g = MB.GraphBuilder("views", weight_std=None)
    x = g.input("data", (C, H, W))
    # [16 unused | reduction 16 | b1 32 | b5 16 | b3 16 | pool C]
    S = g.temp((16 + 16 + 32 + 16 + 16 + C, H, W))
    g.conv2d(x, 16 + 32, 1, out=S, out_channel=16)               # reduction and 1x1 branch at once
    red = S.channels(16, 16)
    g.conv2d(red, 16, 5, 1, 2, out=S, out_channel=64)            # staged tile, input at an offset
    g.conv2d(red, 16, 3, 1, 1, out=S, out_channel=80)            # row form, input at an offset
    g.pool2d(x, 3, 1, 1, "max", out=S.channels(96, C))
    cat = S.channels(32, 32 + 16 + 16 + C)                        # the block's output
    g.conv2d(cat, 40, 1)
    g.pool2d(cat, 3, 1, 1, "avg", count_include_pad=True)
    gp = g.global_avgpool(cat)
    z = g.conv2d(cat, 8, 3, 2, 0)
    g.mark_output(z)
    assert sum(1 for k in g.kernels if "arg_offsets" in k) == 7
    xin = rnd(C, H, W)
    exe, orc, model = run_both(g, tmp_path, {"data": xin})
    compare_storages(exe, orc, model, what="operand views")
    whole = exe.get_data(S.idx, S.size).reshape(-1, H, W)
    assert (whole[:16] == 0).all()                                # nobody writes in front of its slice
    pooled = np.pad(xin, ((0, 0), (1, 1), (1, 1)), constant_values=-np.inf)
    want = np.max([pooled[:, i:i + H, j:j + W] for i in range(3) for j in range(3)], axis=0)
    np.testing.assert_array_equal(whole[96:], want)              # the pool wrote its slice
    got_gp = exe.get_data(gp.idx, 88)
    np.testing.assert_allclose(got_gp, whole[32:].reshape(88, -1).mean(1), rtol=1e-5, atol=1e-6)
    assert np.isfinite(whole).all()


@pytest.mark.parametrize("seq,heads,hd,masked", [(128, 12, 64, False), (40, 4, 24, True), (77, 3, 64, True),
                                                 (16, 2, 16, False), (5, 1, 8, True)])
def test_attention_in_one_launch(tmp_path, seq, heads, hd, masked):
    """reef_attention against the oracle's three steps (scores, masked softmax, context) and against
    numpy on the projected tensor: the full BERT-base shape, ragged sequence lengths (not a multiple
    of the rows a workgroup takes), head sizes below 64, padding positions at the end."""
    hid = heads * hd
    g = MB.GraphBuilder("att", weight_std=0.05)
    x = g.input("x", (seq, hid))
    w = g.param((3 * hid, hid), 0.2)
    bias = g.param((3 * hid,), 0.1)
    qkv = g.gemm(x, w, seq, 3 * hid, hid, trans_b=True, bias=bias)
    mask = g.input("attention_mask", (seq,), "uint1") if masked else None
    ctx = g.attention(qkv, seq, heads, hd, 3 * hid, 0, hid, 2 * hid, 1.0 / np.sqrt(hd), mask=mask)
    g.mark_output(ctx)
    pad = np.zeros(seq, np.uint8)
    pad[seq - max(1, seq // 4):] = 1
    inputs = {"x": rnd(seq, hid)}
    if masked:
        inputs["attention_mask"] = pad
    exe, orc, model = run_both(g, tmp_path, inputs)
    compare_storages(exe, orc, model, what="attention")
    m = exe.get_data(qkv.idx, seq * 3 * hid).reshape(seq, 3, heads, hd).astype(np.float64)
    sc = np.einsum("shd,thd->hst", m[:, 0], m[:, 1]) / np.sqrt(hd)
    if masked:
        sc[:, :, pad != 0] = -np.inf
    pr = np.exp(sc - sc.max(-1, keepdims=True))
    pr /= pr.sum(-1, keepdims=True)
    want = np.einsum("hst,thd->shd", pr, m[:, 2]).reshape(seq, hid)
    got = exe.get_data(ctx.idx, seq * hid).reshape(seq, hid)
    # scores of magnitude 100 (weights of deviation 0.2 on 768 inputs) carry 1e-5 of absolute error in
    # fp32, which the exponential turns into that much relative error: the suite's 1e-4, not less
    assert np.isfinite(got).all() and np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_mocked_model_closed_form(tmp_path):
    """The reference's executor_base.mocked_kernel test: a = b = c = 3 -> 18 everywhere
    (src/reef/test/test.cpp:102-116)."""
    from reef_amd.modelgen import nets
    g = nets.mocked_kernel()
    three = np.full(8192, 3.0, np.float32)
    exe, orc, model = run_both(g, tmp_path, {"a": three, "b": three, "c": three})
    out = exe.get_output()
    assert out.shape == (8192,)
    np.testing.assert_array_equal(out, np.full(8192, 18.0, np.float32))
    np.testing.assert_array_equal(orc.get("output"), out)


XDW_CASES = [
    # cin, H, W, cout: 1x1 (+bias, ReLU6), then depthwise 3x3 / stride 1 / padding 1 (+bias, ReLU6)
    (24, 56, 56, 144),        # MobileNetV2, four segments per row
    (64, 14, 14, 384),
    (160, 7, 7, 960),         # two K steps, half a segment wide
    (16, 9, 30, 40),          # ragged everywhere: three segments (the last two columns wide), odd rows,
                              # output channels not a multiple of 16
    (8, 1, 1, 16),            # one pixel: every neighbour is padding
    (392, 5, 17, 32),         # four K steps
]


@pytest.mark.parametrize("tile", ["g2", "g4"])
@pytest.mark.parametrize("case", XDW_CASES)
def test_pointwise_then_depthwise_in_one_launch(tmp_path, tile, case):
    """reef_conv2d_xdw_<tile> against the oracle's two layers, in all three flavours: the raw and the
    padding flavour on one executor each, the preemptible flavour on the hybrid one; same bits in
    all of them (a task's arithmetic does not depend on the flavour)."""
    import ctypes
    import json
    from reef_amd import binding as B
    from tests.helpers import write_model
    cin, H, W, cout = case
    g = MB.GraphBuilder("x")
    x = g.input("data", (cin, H, W))
    y = g.conv2d_dw(x, cout, act=MB.ACT_RELU6, dw_act=MB.ACT_RELU6, tile=tile)
    z = g.conv2d_dw(y, 24, act=MB.ACT_NONE, dw_act=MB.ACT_RELU, tile=tile) if cout % 8 == 0 else y
    # the same input through a depthwise stage of stride 2 (two rows per tile only), then that again
    # on its result where the channel count allows
    y2 = g.conv2d_dw(x, cout, act=MB.ACT_RELU6, dw_act=MB.ACT_RELU6, stride=2)
    if cout % 8 == 0:
        g.conv2d_dw(y2, 40, act=MB.ACT_RELU, dw_act=MB.ACT_NONE, stride=2)
    g.mark_output(z)
    data = rnd(cin, H, W)
    exe, orc, model = run_both(g, tmp_path, {"data": data})
    worst = compare_storages(exe, orc, model, what="xdw %s %s" % (tile, case))
    want = exe.get_output()
    d = write_model(g, tmp_path)
    for kind, pre in ((B.TRANS, False), (B.HYBRID, True), (B.HYBRID, False)):
        e = B.Executor.from_dir(d, g.name, kind)
        e.set_input_checked("data", data)
        e.execute_preemptable() if pre else e.execute()
        np.testing.assert_array_equal(e.get_output(), want, err_msg="flavour %s %s" % (kind, pre))
        e.close()
    print("xdw %s %s: worst rel err %.2e" % (tile, case, worst[0]))


BLOCK_CASES = [
    # front, cin, H, W, middle channels, output channels
    ("stem", 3, 224, 224, 32, 16),      # MobileNetV2: stem + first block
    ("stem", 3, 61, 45, 32, 16),        # ragged: odd sizes, the last segment three columns wide
    ("stem", 1, 9, 9, 20, 7),           # one channel in, channel counts that fill no tile
    ("stem", 3, 2, 2, 32, 32),          # one output pixel: every neighbour is padding
    ("expand", 16, 112, 112, 96, 24),   # MobileNetV2: second block
    ("expand", 16, 33, 58, 96, 24),     # ragged
    ("expand", 4, 7, 30, 40, 9),        # channel counts that fill no tile
    ("expand", 8, 1, 2, 16, 32),        # one output pixel
]


@pytest.mark.parametrize("case", BLOCK_CASES)
def test_front_filter_depthwise_and_projection_in_one_launch(tmp_path, case):
    """reef_conv2d_sdp_<tile> / reef_conv2d_xdp2_<tile> against the oracle's three layers, each compiled
    tile, in all three flavours (same bits in all of them)."""
    from reef_amd import binding as B
    from tests.helpers import write_model
    front, cin, H, W, cmid, cout = case
    g = MB.GraphBuilder("blk")
    x = g.input("data", (cin, H, W))
    family = "sdp" if front == "stem" else "xdp2"
    outs = [g.conv2d_block(x, cmid, cout, front=front, tile=t) for t in MB.GraphBuilder.BLOCK_TILES[family]]
    other = g.conv2d_block(x, cmid, cout, front=front, act=MB.ACT_NONE, dw_act=MB.ACT_RELU)
    g.mark_output(other)
    assert [k["name"].split("_")[2] for k in g.kernels] == [family] * 3
    data = rnd(cin, H, W)
    exe, orc, model = run_both(g, tmp_path, {"data": data})
    worst = compare_storages(exe, orc, model, what="block %s" % (case,))
    want = exe.get_output()
    d = write_model(g, tmp_path)
    for kind, pre in ((B.TRANS, False), (B.HYBRID, True), (B.HYBRID, False)):
        e = B.Executor.from_dir(d, g.name, kind)
        e.set_input_checked("data", data)
        e.execute_preemptable() if pre else e.execute()
        np.testing.assert_array_equal(e.get_output(), want, err_msg="flavour %s %s" % (kind, pre))
        e.close()
    print("block %s: worst rel err %.2e" % (case, worst[0]))


def test_mobilenetv2_with_and_without_the_fused_front_half(tmp_path):
    """The network with expansion + depthwise in one launch holds, in every tensor both variants
    have (block outputs, logits), what the variant with two launches holds, to 1e-4: the fused
    kernel sums the 1x1 filter in another order than the tiles the separate layer uses."""
    from reef_amd.modelgen import nets
    x = nets.image_input("mobilenetv2", (3, 224, 224))
    outs = []
    for fuse in (False, True):
        g = nets.mobilenet_v2(fuse_expand_dw=fuse, fuse_gap=fuse, fuse_head=fuse)
        exe, orc, model = run_both(g, tmp_path / str(fuse), {"data": x})
        compare_storages(exe, orc, model, what="mobilenetv2 fuse=%s" % fuse)
        li = model["kernels"][-1]["args"][0]
        outs.append((len(g.kernels), exe.get_data(li, model["storage"][li]["size"])))
    # fused: expansion + depthwise, the last convolution averages, the layers at 112 x 112 are two launches
    assert outs[0][0] == 55 and outs[1][0] == 35
    from tests.helpers import max_rel_err, REL_TOL
    assert max_rel_err(outs[1][1], outs[0][1]) <= REL_TOL


@pytest.mark.parametrize("tile", list(MB.GraphBuilder.LN_GEMM_TILES))
def test_gemm_reading_its_rows_through_a_layernorm(tmp_path, tile):
    """reef_gemm_ntl_<tile>: C = act(LayerNorm(A) B^T + bias) (+ residual) and the normalised rows
    written beside it -- ragged M, N and K (K = 200: one full 128-wide step and a partial one; 50
    float4s per row do not divide among the threads of a row), rows far from zero mean; against
    the oracle's two-pass LayerNorm followed by its product, and the written rows against the
    LayerNorm kernel's own output."""
    seq, hid, n = 45, 200, 3 * 200 + 8
    g = MB.GraphBuilder("gl", weight_std=0.05)
    x = g.input("x", (seq, hid))
    r = g.input("r", (seq, n))
    w = g.param((n, hid), 0.05)
    bias = g.param((n,), 0.02)
    gamma, beta = g.layernorm_params(hid)
    n1 = g.temp((seq, hid))
    g.gemm(x, w, seq, n, hid, trans_b=True, bias=bias, act=MB.ACT_GELU, force_tile=tile, res=r,
           ln=dict(gamma=gamma, beta=beta, out=n1))
    g.gemm(x, w, seq, n, hid, trans_b=True, alpha=0.5, force_tile=tile, ln=dict(gamma=gamma, beta=beta, eps=1e-5))
    g.gemm(x, w, seq, n, hid, trans_b=True, force_tile=tile, res=r, ln=dict(gamma=gamma, beta=beta))
    sep = g.layernorm(x, seq, hid, gamma=gamma, beta=beta)
    g.mark_output(sep)
    assert [k["name"].split("#")[0] for k in g.kernels[:3]] == ["reef_gemm_ntl_" + tile] * 3
    exe, orc, model = run_both(g, tmp_path, {"x": 30.0 + 2.0 * rnd(seq, hid), "r": rnd(seq, n)})
    compare_storages(exe, orc, model, what="layernorm gemm " + tile)
    from tests.helpers import max_rel_err, REL_TOL
    got = exe.get_data(n1.idx, seq * hid)
    assert max_rel_err(got, exe.get_data(sep.idx, seq * hid)) <= REL_TOL


@pytest.mark.parametrize("tile,trans_b", [("16x32k4", True), ("32x32d4", True), ("32x32k4", True), ("64x64", True),
                                          ("64x64", False), ("32x128", False)])
def test_gemm_adds_a_residual_behind_the_activation(tmp_path, tile, trans_b):
    """C = act(A B + bias) + R, with R laid out as C is: a column block of a wider tensor, batched."""
    seq, hid, heads = 40, 200, 5
    hd = hid // heads
    g = MB.GraphBuilder("gr", weight_std=0.05)
    x = g.input("x", (seq, hid))
    r = g.input("r", (seq, 2 * hid))
    w = g.param((hid, hid), 0.05)
    bias = g.param((hid,), 0.02)
    out = g.temp((seq, 2 * hid))
    # the right half of `out` = gelu(x w + bias) + the right half of r
    g.gemm(x, w, seq, hid, hid, trans_b=trans_b, bias=bias, act=MB.ACT_GELU, ldc=2 * hid, off_c=hid, out=out,
           res=r, force_tile=tile)
    # per head: C[b] = x_b (w_b)^T or x_b w_b + r_b, heads as column blocks of the left half
    g.gemm(x, w, seq, hd, hd, batch=heads, trans_b=trans_b, lda=hid, ldb=hid, ldc=2 * hid, stride_a=hd,
           stride_b=hd, stride_c=hd, out=out, res=r, force_tile=tile)
    g.mark_output(out)
    exe, orc, model = run_both(g, tmp_path, {"x": rnd(seq, hid), "r": rnd(seq, 2 * hid)})
    compare_storages(exe, orc, model, what="gemm with residual " + tile)


def test_bert_with_and_without_the_layernorm_inside_the_projection(tmp_path):
    """Three BERT layers with the LayerNorms folded into the projections behind them hold, in the
    encoder output, what the network with a LayerNorm launch each holds, to 1e-4; both against
    the oracle in every storage."""
    from reef_amd.modelgen import nets
    from tests.helpers import max_rel_err, REL_TOL
    ids = nets.token_input("bert3", 128, 30522)
    outs = []
    for fuse in (False, True):
        g = nets.bert(layers=3, name="bert3", fuse_layernorm=fuse)
        exe, orc, model = run_both(g, tmp_path / str(fuse), {"input0": ids})
        compare_storages(exe, orc, model, what="bert3 fuse=%s" % fuse)
        oi = model["kernels"][-1]["args"][3]
        outs.append((len(g.kernels), exe.get_data(oi, 128 * 768)))
    assert outs[0][0] == 2 + 3 * 7 and outs[1][0] == 2 + 3 * 5
    assert max_rel_err(outs[1][1], outs[0][1]) <= REL_TOL


@pytest.mark.parametrize("split", [2, 3])
@pytest.mark.parametrize("tile", list(tiling.GEMM_DIRECT_TILES))
def test_gemm_direct_splits_k_across_workgroups(tmp_path, tile, split):
    """reef_gemm_ntd_<tile> with K split over 2 or 3 workgroups per tile and folded inside the
    launch (pair slots for a split of two where launches run to completion, arrival counters
    otherwise): ragged M and N, K = 520 (chunks of 384 + 136 or 256 + 256 + 8), bias + GELU +
    residual; against the oracle, the three flavours bit for bit, twice on one executor, pair
    slots and counters empty afterwards."""
    import json
    import os
    from reef_amd import binding as B
    from tests.helpers import write_model
    seq, hid, n = 40, 520, 200
    g = MB.GraphBuilder("gs", weight_std=0.05)
    x = g.input("x", (seq, hid))
    r = g.input("r", (seq, n))
    w = g.param((n, hid), 0.05)
    bias = g.param((n,), 0.02)
    y = g.gemm(x, w, seq, n, hid, trans_b=True, bias=bias, act=MB.ACT_GELU, res=r, force_tile=tile, split_k=split)
    one = g.gemm(x, w, seq, n, hid, trans_b=True, bias=bias, act=MB.ACT_GELU, res=r, force_tile=tile, split_k=1)
    g.mark_output(y)
    k0 = g.kernels[0]
    assert k0["attrs"][21] == split and k0["launch_params"][0] == split * g.kernels[1]["launch_params"][0]
    assert bool(k0["attrs"][5] & 16) == (split == 2)
    inputs = {"x": rnd(seq, hid), "r": rnd(seq, n)}
    exe, orc, model = run_both(g, tmp_path, inputs)
    compare_storages(exe, orc, model, what="split gemm %s x%d" % (tile, split))
    want = exe.get_output()
    from tests.helpers import max_rel_err, REL_TOL
    assert max_rel_err(want, exe.get_data(one.idx, seq * n)) <= REL_TOL
    d = write_model(g, tmp_path)
    ws = model["kernels"][0]["args"][-2]
    for kind, pre in ((B.TRANS, False), (B.HYBRID, True), (B.HYBRID, False), (B.HYBRID, True)):
        e = B.Executor.from_dir(d, g.name, kind)
        for name, arr in inputs.items():
            e.set_input_checked(name, arr)
        for _ in range(2):
            e.execute_preemptable() if pre else e.execute()
            np.testing.assert_array_equal(e.get_output(), want, err_msg="flavour %s %s" % (kind, pre))
        words = e.get_data(ws, model["storage"][ws]["size"] // 4, np.int32)
        if split == 2:
            assert words.size == 3 * seq * n and not words[2 * seq * n:].any()
        for i, s in enumerate(model["storage"]):
            if s["name"] == "reef_sync":
                assert not e.get_data(i, s["size"], np.int32).any()
        e.close()


SP7_CASES = [
    # cin, H, W, cout, input shift, pool shift, conv act, pool act
    (3, 224, 224, 64, True, True, MB.ACT_RELU, MB.ACT_RELU),      # the ResNet stem
    (3, 37, 45, 24, False, False, MB.ACT_RELU, MB.ACT_NONE),      # odd sizes, a partial channel tile
    (1, 64, 64, 16, True, False, MB.ACT_NONE, MB.ACT_RELU),       # one channel: K = 49
    (2, 30, 57, 40, False, True, MB.ACT_RELU6, MB.ACT_NONE),
    (3, 9, 9, 16, True, True, MB.ACT_RELU, MB.ACT_RELU),          # image smaller than one tile
]


@pytest.mark.parametrize("case", SP7_CASES)
def test_stem_convolution_and_pool_in_one_launch(tmp_path, case):
    """reef_conv2d_sp7_g2: input shift, 7x7 / 2 convolution + bias + activation and the 3x3 / 2
    max-pool + shift + activation behind it against the oracle's three steps, against the three
    launches on the device (1e-4: the fused kernel sums the taps in another order), and bit for
    bit in the three flavours."""
    from reef_amd import binding as B
    from tests.helpers import write_model, max_rel_err, REL_TOL
    cin, H, W, cout, in_shift, pool_shift, act, pool_act = case
    g = MB.GraphBuilder("sp7")
    x = g.input("data", (cin, H, W))
    y = g.conv2d_pool(x, cout, act=act, in_shift=in_shift, pool_shift=pool_shift, pool_act=pool_act)
    g.mark_output(y)
    assert g.kernels[0]["name"].startswith("reef_conv2d_sp7_g2") and len(g.kernels) == 1
    # the same parameters through launches of their own
    g3 = MB.GraphBuilder("sp7")
    x3 = g3.input("data", (cin, H, W))
    t = g3.eltwise(x3, shift=True) if in_shift else x3
    t = g3.conv2d(t, cout, 7, 2, 3, bias=True, act=act)
    g3.mark_output(g3.pool2d(t, 3, 2, 1, "max", bias=pool_shift, act=pool_act))
    assert [k for k, _ in g3.params if not k.endswith("k")] == [k for k, _ in g.params]
    data = 2.0 * rnd(cin, H, W) - 0.5
    exe, orc, model = run_both(g, tmp_path / "one", {"data": data})
    worst = compare_storages(exe, orc, model, what="sp7 %s" % (case,))
    want = exe.get_output()
    exe3, orc3, model3 = run_both(g3, tmp_path / "three", {"data": data})
    assert max_rel_err(want, exe3.get_output()) <= REL_TOL
    d = write_model(g, tmp_path / "one")
    for kind, pre in ((B.TRANS, False), (B.HYBRID, True), (B.HYBRID, False)):
        e = B.Executor.from_dir(d, g.name, kind)
        e.set_input_checked("data", data)
        e.execute_preemptable() if pre else e.execute()
        np.testing.assert_array_equal(e.get_output(), want, err_msg="flavour %s %s" % (kind, pre))
        e.close()
    print("sp7 %s: worst rel err %.2e" % (case, worst[0]))


def test_average_pool_reading_through_a_pre_activation(tmp_path):
    """reef_pool2d with REEF_POOL_F_PRE: relu(in * scale[c] + shift[c]) then a 2x2 average (what a
    DenseNet transition pools), and a 3x3 / stride 2 / padding 1 max-pool of the same with a bias
    and ReLU behind it, and the global average of the same (REEF_GAP_F_PRE); odd sizes, against the oracle."""
    g = MB.GraphBuilder("prepool")
    x = g.input("data", (37, 19, 23))
    ps, pt = g.pre_act_params(37)
    a = g.pool2d(x, 2, 2, 0, "avg", pre=(ps, pt))
    b = g.pool2d(x, 3, 2, 1, "max", bias=True, act=MB.ACT_RELU, pre=(ps, pt))
    g.global_avgpool(x, pre=(ps, pt))
    g.mark_output(a)
    assert a.shape == (37, 9, 11) and b.shape == (37, 10, 12)
    exe, orc, model = run_both(g, tmp_path, {"data": rnd(37, 19, 23)})
    compare_storages(exe, orc, model, what="pool with pre-activation")


@pytest.mark.parametrize("case", [(320, 7, 7, 1280, 1, 0, False, False), (64, 5, 6, 40, 1, 0, True, True),
                                  (48, 4, 4, 24, 3, 1, True, False), (32, 3, 5, 16, 1, 0, False, False)])
def test_convolution_that_averages_its_own_output(tmp_path, case):
    """REEF_F_GAP_OUTPUT: a direct kernel whose pixel groups cover the image writes the global
    average of what it would have written (bias, residual, scale / shift, activation first);
    against the oracle and against convolution + average pool as two launches; the three flavours
    bit for bit."""
    from reef_amd import binding as B
    from tests.helpers import write_model, max_rel_err, REL_TOL
    cin, H, W, cout, k, pad, residual, affine = case

    def build(gap):
        g = MB.GraphBuilder("gapconv")
        x = g.input("data", (cin, H, W))
        r = g.input("res", (cout, H, W)) if residual else None
        y = g.conv2d(x, cout, k, 1, pad, bias=not affine, act=MB.ACT_RELU6, residual=r, affine=affine, gap=gap)
        g.mark_output(y if gap else g.global_avgpool(y))
        return g
    g, g2 = build(True), build(False)
    assert len(g.kernels) == 1 and len(g2.kernels) == 2 and g.kernels[0]["attrs"][12] & 2048
    inputs = {"data": rnd(cin, H, W)}
    if residual:
        inputs["res"] = rnd(cout, H, W)
    exe, orc, model = run_both(g, tmp_path / "one", inputs)
    compare_storages(exe, orc, model, what="gap conv %s" % (case,))
    want = exe.get_output()[:cout].copy()
    exe2, _, _ = run_both(g2, tmp_path / "two", inputs)
    assert max_rel_err(want, exe2.get_output()[:cout]) <= REL_TOL
    d = write_model(g, tmp_path / "one")
    for kind, pre in ((B.TRANS, False), (B.HYBRID, True), (B.HYBRID, False)):
        e = B.Executor.from_dir(d, g.name, kind)
        for name, arr in inputs.items():
            e.set_input_checked(name, arr)
        e.execute_preemptable() if pre else e.execute()
        np.testing.assert_array_equal(e.get_output()[:cout], want, err_msg="flavour %s %s" % (kind, pre))
        e.close()
