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
           fused_reduce=False, fuse_act=True):
    """fused_reduce: fold split-K inside the conv kernels.  fuse_act: let the unit's last
    conv also write the next unit's activated input (one kernel instead of conv + add/relu)."""
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
    x = g.eltwise(data, shift=True)                                  # bn_data (shift only)
    x = g.conv2d(x, filters[0], 7, 2, 3, bias=True, act=ACT_RELU)    # conv0 + bn0 + relu
    act = g.pool2d(x, 3, 2, 1, "max", bias=True, act=ACT_RELU)       # pool + first bn1 + relu
    raw = None
    n_stages = len(units)
    for si in range(n_stages):
        cout = filters[si + 1]
        for ui in range(units[si]):
            first = ui == 0
            last_of_stage = ui == units[si] - 1
            last_of_net = last_of_stage and si == n_stages - 1
            stride = (1 if si == 0 else 2) if first else 1
            mid = cout // 4 if bottleneck else cout
            if bottleneck:
                y = g.conv2d(act, mid, 1, stride, 0, bias=True, act=ACT_RELU)
                y = g.conv2d(y, mid, 3, 1, 1, bias=True, act=ACT_RELU)
                last_k, last_p = 1, 0
            else:
                y = g.conv2d(act, mid, 3, stride, 1, bias=True, act=ACT_RELU)
                last_k, last_p = 3, 1
            shortcut = g.conv2d(act, cout, 1, stride, 0, bias=False, act=ACT_NONE) if first else raw
            if last_of_net:
                act = g.conv2d(y, cout, last_k, 1, last_p, bias=False, act=ACT_RELU,
                               residual=shortcut, affine=True)
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
