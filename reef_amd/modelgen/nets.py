"""Network definitions for the benchmark configurations.

ResNet follows the graph the reference's generator compiles --
``relay.testing.resnet`` (script/tvm_generate_model.py:34-36): the pre-activation
(v2) residual network with the stride on the first convolution of a unit, batch
norms folded into the neighbouring convolution as a bias, and the wiring read
off resource/resnet152/resnet152.json kernels[0..18]:

  data + shift -> conv 7x7/2 (+bias, relu) -> maxpool 3x3/2 (+bias, relu)
  unit with projection : conv1 1x1/s (+b, relu) -> conv2 3x3 (+b, relu)
                         shortcut 1x1/s (bare, from the activated input)
                         conv3 1x1 + residual(shortcut)             -> raw x
                         x + shift, relu                            -> next unit's input
  identity unit        : conv1 -> conv2 -> conv3 + residual(x)      -> raw x'
  last unit of a stage : conv3 + residual + bias, relu (the raw sum is not needed)
  last unit of the net : conv3 + residual, * scale + shift, relu
  global average pool -> dense (+bias) -> softmax
"""
import math
import numpy as np

from . import rng
from .builder import ACT_NONE, ACT_RELU, ACT_RELU6, ACT_GELU, GraphBuilder

IMAGENET_MEAN = (0.485, 0.456, 0.406)
IMAGENET_STD = (0.229, 0.224, 0.225)


def image_input(name, shape, seed=rng.BASE_SEED):
    """U(0,1) image, then per-channel ImageNet normalisation."""
    c, h, w = shape
    x = rng.uniform_f32(name + "/data", c * h * w, seed).reshape(c, h, w)
    mean = np.array(IMAGENET_MEAN, np.float32)[:c, None, None]
    std = np.array(IMAGENET_STD, np.float32)[:c, None, None]
    return ((x - mean) / std).astype(np.float32)


def resnet(num_layers=152, image=(3, 224, 224), classes=1000, name=None, seed=rng.BASE_SEED,
           fused_reduce=False, fuse_act=True, stack_first=True, fuse_stem=True, fuse_gap=False):
    """fused_reduce: fold split-K inside the conv kernels.  fuse_act: let the unit's last
    conv also write the next unit's activated input (one kernel instead of conv + add/relu).
    The first unit of a bottleneck stage has two 1x1 convolutions on the same input with the same
    stride: conv1 (+bias, ReLU) and the projection shortcut (bare).  They are one convolution
    with the stacked filter and two outputs: the bare result, whose shortcut rows are the
    residual of the unit's last convolution, and relu(result + shift), whose conv1 rows feed the
    3x3 convolution (channel ranges of the two outputs, operand views).  stack_first=False keeps
    them two launches, as the reference's graph has them.
    fuse_stem: the shift on the input, the 7x7 convolution and the max-pool behind it are one launch
    (reef_conv2d_sp7_g2) instead of three; same parameters in the same order."""
    if num_layers >= 50:
        bottleneck = True
        filters = [64, 256, 512, 1024, 2048]
        units = {50: [3, 4, 6, 3], 101: [3, 4, 23, 3], 152: [3, 8, 36, 3]}[num_layers]
    else:
        bottleneck = False
        filters = [64, 64, 128, 256, 512]
        units = {18: [2, 2, 2, 2], 34: [3, 4, 6, 3]}[num_layers]
    g = GraphBuilder(name or "resnet%d" % num_layers, seed)
    g.fused_reduce = fused_reduce
    data = g.input("data", image)
    if fuse_stem and image[0] <= 3:
        act = g.conv2d_pool(data, filters[0], act=ACT_RELU, in_shift=True, pool_shift=True, pool_act=ACT_RELU)
    else:
        x = g.eltwise(data, shift=True)                                  # bn_data (shift only)
        x = g.conv2d(x, filters[0], 7, 2, 3, bias=True, act=ACT_RELU)    # conv0 + bn0 + relu
        act = g.pool2d(x, 3, 2, 1, "max", bias=True, act=ACT_RELU)       # pool + first bn1 + relu
    raw = pooled = None
    n_stages = len(units)
    for si in range(n_stages):
        cout = filters[si + 1]
        for ui in range(units[si]):
            first = ui == 0
            last_of_stage = ui == units[si] - 1
            last_of_net = last_of_stage and si == n_stages - 1
            stride = (1 if si == 0 else 2) if first else 1
            mid = cout // 4 if bottleneck else cout
            if bottleneck and first and stack_first:
                both, both_act = g.conv2d(act, mid + cout, 1, stride, 0, bias=False, act=ACT_NONE, dual_act=ACT_RELU)
                y = g.conv2d(both_act.channels(0, mid), mid, 3, 1, 1, bias=True, act=ACT_RELU)
                shortcut = both.channels(mid, cout)
                last_k, last_p = 1, 0
            elif bottleneck:
                y = g.conv2d(act, mid, 1, stride, 0, bias=True, act=ACT_RELU)
                y = g.conv2d(y, mid, 3, 1, 1, bias=True, act=ACT_RELU)
                shortcut = g.conv2d(act, cout, 1, stride, 0, bias=False, act=ACT_NONE) if first else raw
                last_k, last_p = 1, 0
            else:
                y = g.conv2d(act, mid, 3, stride, 1, bias=True, act=ACT_RELU)
                shortcut = g.conv2d(act, cout, 1, stride, 0, bias=False, act=ACT_NONE) if first else raw
                last_k, last_p = 3, 1
            if last_of_net:
                # fuse_gap: the network's last convolution averages its own output (one pixel tile covers 7 x 7)
                gap = fuse_gap and GraphBuilder.gap_tile(y.shape[0], last_k, last_k, y.shape[1] * y.shape[2]) is not None
                act = g.conv2d(y, cout, last_k, 1, last_p, bias=False, act=ACT_RELU,
                               residual=shortcut, affine=True, gap=gap)
                pooled = act if gap else None
            elif last_of_stage:
                act = g.conv2d(y, cout, last_k, 1, last_p, bias=True, act=ACT_RELU,
                               residual=shortcut)
            elif fuse_act:
                raw, act = g.conv2d(y, cout, last_k, 1, last_p, bias=False, act=ACT_NONE,
                                    residual=shortcut, dual_act=ACT_RELU)
            else:
                raw = g.conv2d(y, cout, last_k, 1, last_p, bias=False, act=ACT_NONE,
                               residual=shortcut)
                act = g.eltwise(raw, shift=True, act=ACT_RELU)
    if pooled is None:
        pooled = g.global_avgpool(act)
    logits = g.dense(pooled, classes, bias=True)
    out = g.softmax(logits, 1, classes)
    g.mark_output(out)
    return g


def mocked_kernel(name="mocked_kernel"):
    """The reference's mocked model (resource/mocked_kernel/mocked_kernel.json):
    temp = b + a[t]; output = temp[t] * c."""
    g = GraphBuilder(name)
    g.unique_names = False   # keep the reference's kernel names and profile keys
    a = g.input("a", (8192,))
    b = g.input("b", (8192,))
    temp = g.temp((8192,), "temp")
    c = g.input("c", (8192,))
    out = g.temp((8192,), "output")
    g.mocked("add", b, a, temp)
    g.mocked("multiply", temp, c, out)
    return g


def mobilenet_v2(image=(3, 224, 224), classes=1000, name="mobilenetv2", seed=rng.BASE_SEED, fuse_expand_dw=True,
                 fuse_gap=True, fuse_head=True):
    """MobileNetV2, width 1.0: 3x3/2 stem, 17 inverted-residual blocks (1x1 expand + ReLU6,
    depthwise 3x3 + ReLU6, linear 1x1 projection, residual add when stride 1 and equal
    channels), 1x1 to 1280, global average pool, classifier.  Batch norms are folded
    into the convolutions as biases; the residual add is the projection's epilogue.
    fuse_expand_dw: the 1x1 expansion of a block and the depthwise convolution behind it are one
    launch and the expanded tensor is never written
    (GraphBuilder.conv2d_dw); False keeps the two launches.
    fuse_head: the layers on the 112 x 112 image are two launches instead of six: stem + first
    block (no expansion: depthwise filter and projection to 16 channels), and the second block
    (16 -> 96 -> 24 channels, stride 2) -- GraphBuilder.conv2d_block, every channel of a pixel tile
    in one workgroup; same parameters in the same order."""
    g = GraphBuilder(name, seed)
    x = g.input("data", image)
    cfg = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
           (6, 320, 1, 1)]
    cin = 32
    stem_done = False
    if fuse_head and image[0] <= 3 and cfg[0][0] == 1 and cfg[0][3] == 1 and GraphBuilder.block_fits("stem", image[0], 32, cfg[0][1], image[2]):
        x = g.conv2d_block(x, 32, cfg[0][1], front="stem")
        cin, stem_done = cfg[0][1], True
    else:
        x = g.conv2d(x, 32, 3, 2, 1, bias=True, act=ACT_RELU6)
    for bi, (t, c, n, s) in enumerate(cfg):
        for i in range(n):
            if bi == 0 and stem_done:
                continue
            stride = s if i == 0 else 1
            y = x
            if fuse_head and t != 1 and stride == 2 and GraphBuilder.block_fits("expand", cin, cin * t, c, x.shape[2]):
                x = g.conv2d_block(x, cin * t, c, front="expand")
                cin = c
                continue
            # (not the stride-2 block at 112 x 112: its 1x1 result is 96 x 112 x 112, and forming it
            # tile by tile with the rows and columns neighbours share costs more than the launch and
            # the round trip saved: 14.9 against 13.1 us)
            if t != 1 and fuse_expand_dw and cin % 8 == 0 and not (stride == 2 and y.shape[1] * y.shape[2] > 3136):
                y = g.conv2d_dw(y, cin * t, act=ACT_RELU6, dw_act=ACT_RELU6, stride=stride)
            else:
                if t != 1:
                    y = g.conv2d(y, cin * t, 1, 1, 0, bias=True, act=ACT_RELU6)
                y = g.dwconv2d(y, 3, stride, 1, bias=True, act=ACT_RELU6)
            res = x if (stride == 1 and cin == c) else None
            x = g.conv2d(y, c, 1, 1, 0, bias=True, act=ACT_NONE, residual=res)
            cin = c
    # fuse_gap: the last convolution averages its own output where one pixel tile covers the image
    if fuse_gap and GraphBuilder.gap_tile(cin, 1, 1, x.shape[1] * x.shape[2]) is not None:
        pooled = g.conv2d(x, 1280, 1, 1, 0, bias=True, act=ACT_RELU6, gap=True)
    else:
        x = g.conv2d(x, 1280, 1, 1, 0, bias=True, act=ACT_RELU6)
        pooled = g.global_avgpool(x)
    logits = g.dense(pooled, classes, bias=True)
    out = g.softmax(logits, 1, classes)
    g.mark_output(out)
    return g


def densenet(blocks=(6, 12, 48, 32), growth=32, image=(3, 224, 224), classes=1000, name="densenet201",
             seed=rng.BASE_SEED, fuse_stem=True, pool_first=True, under_load=False):
    """DenseNet-BC (201: blocks 6/12/48/32, growth 32): every layer reads the running
    concatenation through its own BN + ReLU (it cannot be folded into the producing
    convolution because each consumer has its own statistics; it is folded into the input
    loads of the consuming 1x1 convolution where a kernel for that exists), then
    1x1 -> 128 (+bias, ReLU) and 3x3 -> 32, which writes straight into its channel slice
    of the concatenation buffer.
    fuse_stem: the 7x7 convolution and the max-pool behind it are one launch (reef_conv2d_sp7_g2).
    pool_first: a transition is BN + ReLU, a 1x1 filter (no bias) and a 2x2 average pool.  Filter
    and average are both linear and the filter is pointwise, so they commute: the pool reads the
    concatenation through the BN + ReLU and the filter runs on a quarter of the pixels, writing
    straight into the next block's buffer -- a quarter of the transition's multiplications, same
    parameters in the same order; the network's last BN + ReLU is applied by the global average
    pool as it reads.  False keeps the textbook order and a launch for that BN + ReLU.
    under_load: tile choices for a model that runs as a best-effort model beside others
    (tuned.TUNED_UNDER_LOAD) instead of those for a model that has the device to itself."""
    g = GraphBuilder(name, seed, under_load=under_load)
    x = g.input("data", image)
    fuse_stem = fuse_stem and image[0] <= 3
    y = None if fuse_stem else g.conv2d(x, 2 * growth, 7, 2, 3, bias=True, act=ACT_RELU)
    stem_hw = ((image[1] - 1) // 2 + 1, (image[2] - 1) // 2 + 1)       # the 7x7 / 2 convolution's output
    c = 2 * growth
    for bi, n_layers in enumerate(blocks):
        # the pool in front of a block writes the first channels of the block's buffer itself
        pool = (3, 2, 1, "max") if bi == 0 else (2, 2, 0, "avg")
        if isinstance(y, tuple):
            H, W = y[0].shape[1:]          # already pooled
        else:
            yh, yw = stem_hw if y is None else y.shape[1:]
            H = (yh + 2 * pool[2] - pool[0]) // pool[1] + 1
            W = (yw + 2 * pool[2] - pool[0]) // pool[1] + 1
        total = c + n_layers * growth
        buf = g.temp((total, H, W))
        if y is None:
            g.conv2d_pool(x, c, act=ACT_RELU, out=buf.channels(0, c))
        elif isinstance(y, tuple):
            # transition with the pool in front: y = (pooled pre-activated input, weights of the 1x1 filter)
            g.conv2d(y[0], c, 1, 1, 0, bias=False, act=ACT_NONE, out=buf, out_channel=0, given={"w": y[1]})
        else:
            g.pool2d(y, *pool, out=buf.channels(0, c))
        for li in range(n_layers):
            cur = c + li * growth
            y = g.conv2d(buf.channels(0, cur), 4 * growth, 1, 1, 0, bias=True, act=ACT_RELU, pre_act=True)
            g.conv2d(y, growth, 3, 1, 1, bias=False, act=ACT_NONE, out=buf, out_channel=cur)
        c = total
        x = buf
        if bi != len(blocks) - 1:
            if pool_first:
                # parameters in the order the textbook form makes them: weights, pre-scale, pre-shift
                w = g.param((c // 2, c, 1, 1), math.sqrt(2.0 / c))
                ps, pt = g.pre_act_params(c)
                y = (g.pool2d(x, 2, 2, 0, "avg", pre=(ps, pt)), w)
            else:
                y = g.conv2d(x, c // 2, 1, 1, 0, bias=False, act=ACT_NONE, pre_act=True)
            c = c // 2
    if pool_first:
        pooled = g.global_avgpool(x, pre=g.pre_act_params(c))     # the last BN + ReLU on the way into the pool
    else:
        a = g.eltwise(x, scale=True, shift=True, act=ACT_RELU)
        pooled = g.global_avgpool(a)
    logits = g.dense(pooled, classes, bias=True)
    out = g.softmax(logits, 1, classes)
    g.mark_output(out)
    return g


def inception_v3(image=(3, 299, 299), classes=1000, name="inceptionv3", seed=rng.BASE_SEED):
    """Inception-v3 (the 299x299 network): every convolution is conv + folded BN + ReLU.
    The 1x1 convolutions of a block that read the block's input (the 1x1 branch and the reductions
    in front of the 5x5 / 3x3 / 7-tap branches) are ONE convolution with the stacked filter: same
    input, same epilogue, and each of them alone fills less than the device.  Its result
    [reductions | 1x1 branch] is written in front of and into the block's output buffer, so the
    1x1 branch lands where the concatenation wants it and the reductions are read back as channel
    ranges (operand views); the other branches write straight into their channel slices.
    The pool branch (3x3 average pool, then a 1x1 convolution + bias + ReLU) joins the stacked
    filter too: averaging and a 1x1 filter commute, so the filter is applied first, as more rows
    of the stacked convolution, and the pool then averages the few result channels instead of
    all input channels and adds the bias and the ReLU.  Those rows must leave the convolution
    bare, so the stacked convolution uses its two-output epilogue: out = the bare result (the
    pool reads its rows of it), out2 = relu(out + shift) in the block buffer (everything else)."""
    g = GraphBuilder(name, seed)

    def conv(x, cout, k, s=1, p=0, out=None, ch=0):
        return g.conv2d(x, cout, k, s, p, bias=True, act=ACT_RELU, out=out, out_channel=ch)

    def stacked(x, pool_ch, rest, S):
        """[pool branch | rest] 1x1 filters on x at once.  relu(result + shift) goes to the first
        channels of S (the pool branch's rows of it are never read); returns the bare result."""
        bare, _ = g.conv2d(x, pool_ch + rest, 1, 1, 0, bias=False, act=ACT_NONE, dual_act=ACT_RELU, out2=S)
        return bare

    def pool_branch(bare, pool_ch, out):
        g.pool2d(bare.channels(0, pool_ch), 3, 1, 1, "avg", count_include_pad=True, bias=True, act=ACT_RELU, out=out)

    x = g.input("data", image)
    x = conv(x, 32, 3, 2)            # 149
    x = conv(x, 32, 3)               # 147
    x = conv(x, 64, 3, 1, 1)         # 147
    x = g.pool2d(x, 3, 2, 0, "max")  # 73
    x = conv(x, 80, 1)
    x = conv(x, 192, 3)              # 71
    x = g.pool2d(x, 3, 2, 0, "max")  # 35

    def inception_a(x, pool_ch):
        _, H, W = x.shape
        r = pool_ch + 48 + 64                            # what lies in front of the output
        S = g.temp((r + 64 + 64 + 96 + pool_ch, H, W))
        bare = stacked(x, pool_ch, 48 + 64 + 64, S)      # [pool branch | 5x5 reduction | 3x3 reduction | 1x1 branch]
        conv(S.channels(pool_ch, 48), 64, 5, 1, 2, out=S, ch=r + 64)
        conv(conv(S.channels(pool_ch + 48, 64), 96, 3, 1, 1), 96, 3, 1, 1, out=S, ch=r + 128)
        pool_branch(bare, pool_ch, S.channels(r + 224, pool_ch))
        return S.channels(r, 224 + pool_ch)

    x = inception_a(x, 32)
    x = inception_a(x, 64)
    x = inception_a(x, 64)

    def inception_b(x):
        cin, H, W = x.shape
        Ho = (H - 3) // 2 + 1
        out = g.temp((384 + 96 + cin, Ho, Ho))
        conv(x, 384, 3, 2, out=out, ch=0)
        conv(conv(conv(x, 64, 1), 96, 3, 1, 1), 96, 3, 2, out=out, ch=384)
        g.pool2d(x, 3, 2, 0, "max", out=out.channels(384 + 96, cin))
        return out

    x = inception_b(x)               # 768 x 17 x 17

    def inception_c(x, c7):
        _, H, W = x.shape
        r = 192 + 2 * c7
        S = g.temp((r + 768, H, W))
        bare = stacked(x, 192, c7 + c7 + 192, S)         # [pool branch | 7-tap reduction | double 7-tap reduction | 1x1 branch]
        conv(conv(S.channels(192, c7), c7, (1, 7), 1, (0, 3)), 192, (7, 1), 1, (3, 0), out=S, ch=r + 192)
        y = conv(conv(conv(S.channels(192 + c7, c7), c7, (7, 1), 1, (3, 0)), c7, (1, 7), 1, (0, 3)), c7, (7, 1), 1, (3, 0))
        conv(y, 192, (1, 7), 1, (0, 3), out=S, ch=r + 384)
        pool_branch(bare, 192, S.channels(r + 576, 192))
        return S.channels(r, 768)

    for c7 in (128, 160, 160, 192):
        x = inception_c(x, c7)

    def inception_d(x):
        cin, H, W = x.shape
        Ho = (H - 3) // 2 + 1
        out = g.temp((320 + 192 + cin, Ho, Ho))
        red = conv(x, 192 + 192, 1)                      # both reductions
        conv(red.channels(0, 192), 320, 3, 2, out=out, ch=0)
        y = conv(conv(red.channels(192, 192), 192, (1, 7), 1, (0, 3)), 192, (7, 1), 1, (3, 0))
        conv(y, 192, 3, 2, out=out, ch=320)
        g.pool2d(x, 3, 2, 0, "max", out=out.channels(320 + 192, cin))
        return out

    x = inception_d(x)               # 1280 x 8 x 8

    def inception_e(x):
        _, H, W = x.shape
        r = 192 + 384 + 448
        S = g.temp((r + 2048, H, W))
        bare = stacked(x, 192, 384 + 448 + 320, S)       # [pool branch | 3-tap reduction | 3x3 reduction | 1x1 branch]
        y = S.channels(192, 384)
        conv(y, 384, (1, 3), 1, (0, 1), out=S, ch=r + 320)
        conv(y, 384, (3, 1), 1, (1, 0), out=S, ch=r + 704)
        y = conv(S.channels(192 + 384, 448), 384, 3, 1, 1)
        conv(y, 384, (1, 3), 1, (0, 1), out=S, ch=r + 1088)
        conv(y, 384, (3, 1), 1, (1, 0), out=S, ch=r + 1472)
        pool_branch(bare, 192, S.channels(r + 1856, 192))
        return S.channels(r, 2048)

    x = inception_e(x)
    x = inception_e(x)               # 2048 x 8 x 8
    pooled = g.global_avgpool(x)
    logits = g.dense(pooled, classes, bias=True)
    out = g.softmax(logits, 1, classes)
    g.mark_output(out)
    return g


def bert(layers=12, hidden=768, heads=12, ffn=3072, seq=128, vocab=30522, name="bert_base",
         seed=rng.BASE_SEED, attention_mask=False, fused_attention=True, fuse_layernorm=True,
         under_load=False):
    """BERT encoder (base: 12 layers, hidden 768, 12 heads, FFN 3072, sequence 128), fp32,
    weights ~ N(0, 0.02).  Token ids are an int64 input, as in the reference's BERT model
    (resource/bert/bert.json storage[0]).  The per-head views of Q, K, V and of the context
    are expressed as GEMM strides, so no transpose kernels are needed, and the three projections
    of a layer are ONE product with the stacked weight [3 * hidden][hidden]: Q, K and V are the
    column blocks of its [seq][3 * hidden] result, which the attention products address by
    offset and leading dimension (a third of the launches of three separate products, each of
    which fills only 192 of the 256 CUs' workgroup slots once).
    attention_mask: a second input `attention_mask` (uint1, one byte per token, non-zero = padding)
    that every softmax applies to the key positions.  The reference's BERT derives that mask
    inside the graph -- as all zeros (fused_full_equal_reshape, bert.cu:313) -- and applies it
    with a kernel of its own per layer (bert.cu:381-388); here it is an operand of the softmax,
    and a storage nobody has set is all zeros, as every storage is after loading.
    fuse_layernorm: a LayerNorm whose result feeds a projection (the one before Q/K/V and the one
    before the FFN) is not a launch of its own: the projection normalises the rows on the way into
    its tiles and writes them out for the next residual (reef_gemm_ntl_*); only the last
    LayerNorm of the network remains a kernel, and the residual sums are made by the epilogues
    of the products in front -- 24 launches fewer, same parameters in the same order.
    under_load: tile choices for a model that runs as a best-effort model beside others
    (tuned.GEMM_UNDER_LOAD) instead of those for a model that has the device to itself."""
    g = GraphBuilder(name, seed, weight_std=0.02, under_load=under_load)
    hd = hidden // heads
    ids = g.input("input0", (seq,), "int64")
    mask = g.input("attention_mask", (seq,), "uint1") if attention_mask else None
    x = g.embedding(ids, vocab, seq, hidden, pos=True, seg=True)

    # fuse_layernorm: the residual sum is made by the product in front of the LayerNorm (its
    # epilogue adds the residual), the LayerNorm by the product behind it
    def norm_then_project(pre, res, wt, bias, n, act=0):
        """LayerNorm(pre (+ res)) and its projection: (normalised rows, product)."""
        gamma, beta = g.layernorm_params(hidden)
        w_, b_ = wt(), bias()
        if fuse_layernorm:
            assert res is None
            normed = g.temp((seq, hidden))
            out = g.gemm(pre, w_, seq, n, hidden, trans_b=True, bias=b_, act=act,
                         ln=dict(gamma=gamma, beta=beta, out=normed))
            return normed, out
        normed = g.layernorm(pre, seq, hidden, res=res, gamma=gamma, beta=beta)
        return normed, g.gemm(normed, w_, seq, n, hidden, trans_b=True, bias=b_, act=act)

    def project_back(a, wt, k, res):
        """a x wt^T + bias and the residual: the sum itself (fused) or (product, residual) for the LayerNorm kernel."""
        w_ = g.param((hidden, k), 0.02)
        b_ = g.param((hidden,), 0.02)
        if fuse_layernorm:
            return g.gemm(a, w_, seq, hidden, k, trans_b=True, bias=b_, res=res), None
        return g.gemm(a, w_, seq, hidden, k, trans_b=True, bias=b_), res

    pre, res = x, None
    inv_sqrt = 1.0 / (hd ** 0.5)
    for _ in range(layers):
        x, qkv = norm_then_project(pre, res, lambda: g.param((3 * hidden, hidden), 0.02),
                                   lambda: g.param((3 * hidden,), 0.02), 3 * hidden)
        if fused_attention and g.attention_ok(seq, hd, 3 * hidden, hidden, (0, hidden, 2 * hidden)):
            # scores, masked softmax and context of all heads in one launch: the scores of a
            # workgroup's query rows stay in its registers and LDS
            ctx = g.attention(qkv, seq, heads, hd, 3 * hidden, 0, hidden, 2 * hidden, inv_sqrt, mask=mask)
        else:
            scores = g.gemm(qkv, qkv, seq, seq, hd, batch=heads, trans_b=True, alpha=inv_sqrt,
                            lda=3 * hidden, ldb=3 * hidden, ldc=seq, stride_a=hd, stride_b=hd, stride_c=seq * seq,
                            off_b=hidden)
            probs = g.softmax(scores, heads * seq, seq, mask=mask)
            ctx = g.temp((seq, hidden))
            g.gemm(probs, qkv, seq, hd, seq, batch=heads, trans_b=False, lda=seq, ldb=3 * hidden, ldc=hidden,
                   stride_a=seq * seq, stride_b=hd, stride_c=hd, out=ctx, off_b=2 * hidden)
        pre, res = project_back(ctx, None, hidden, x)
        x, h = norm_then_project(pre, res, lambda: g.param((ffn, hidden), 0.02), lambda: g.param((ffn,), 0.02),
                                 ffn, ACT_GELU)
        pre, res = project_back(h, None, ffn, x)
    g.mark_output(g.layernorm(pre, seq, hidden, res=res))
    return g


def token_input(name, seq, vocab, seed=rng.BASE_SEED):
    return rng.randint(name + "/ids", seq, vocab, seed)


# The networks of the benchmark configurations in the roles they have there: DenseNet-201 and
# BERT-base are best-effort models in every configuration that names them, so they are generated
# for that role (under_load).
BUILDERS = {
    "resnet18": lambda: resnet(18), "resnet50": lambda: resnet(50), "resnet152": lambda: resnet(152),
    "mobilenetv2": mobilenet_v2, "densenet201": lambda: densenet(under_load=True), "inceptionv3": inception_v3,
    "bert_base": lambda: bert(under_load=True), "mocked_kernel": mocked_kernel,
}
