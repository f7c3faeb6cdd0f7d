"""reef_ops_conv2d: one fused convolution on plain device pointers (the call a kernel of the
reference's fused_nn_conv2d_* family serves, resource/resnet152/resnet152.cu:35,376) against the
CPU oracle, through the C-ABI.  Tolerance: 1e-4 of the output's largest magnitude (fp32)."""
import numpy as np
import pytest

from oracle import oracle as O
from reef_amd import binding as B
from tests.helpers import max_rel_err, REL_TOL

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(11)

# cin, H, W, cout, k, stride, pad, act, bias, residual
CASES = [
    (256, 14, 14, 256, 3, 1, 1, 1, True, False),     # row form, split folded inside the launch
    (64, 56, 56, 64, 3, 1, 1, 1, True, True),        # row form, single pass
    (1024, 14, 14, 256, 1, 1, 0, 1, True, False),    # 1x1 direct, split
    (256, 14, 14, 1024, 1, 1, 0, 0, False, True),    # 1x1 + residual
    (256, 56, 56, 128, 1, 2, 0, 1, True, False),     # strided 1x1
    (3, 64, 64, 64, 7, 2, 3, 1, True, False),        # 7x7 stem: K = 147, unaligned loader
    (24, 9, 11, 40, (1, 7), 1, (0, 3), 2, True, False),
    (16, 17, 17, 24, 5, 1, 2, 0, True, True),        # 25 taps: staged tile
    (40, 15, 15, 136, 3, 2, 1, 1, True, False),      # 3x3 stride 2: tap form
    (20, 5, 5, 8, 1, 1, 0, 0, False, False),         # 1x1 with Cin % 8 != 0: staged tile
]


def run_case(case, noalloc=False):
    cin, H, W, cout, k, s, p, act, has_bias, has_res = case
    kh, kw = (k, k) if isinstance(k, int) else k
    ph, pw = (p, p) if isinstance(p, int) else p
    Ho, Wo = (H + 2 * ph - kh) // s + 1, (W + 2 * pw - kw) // s + 1
    x = RNG.standard_normal((cin, H, W)).astype(np.float32)
    w = (RNG.standard_normal((cout, cin, kh, kw)) * np.sqrt(2.0 / (cin * kh * kw))).astype(np.float32)
    bias = RNG.standard_normal(cout).astype(np.float32) if has_bias else None
    res = RNG.standard_normal((cout, Ho, Wo)).astype(np.float32) if has_res else None
    ref = O.conv2d(x, w, bias, res, None, None, (s, s), (ph, pw), 1, act, 6.0, False)
    d = B.Conv2dDesc(cin, H, W, cout, kh, kw, s, s, ph, pw, act)
    bx, bw = B.DeviceBuffer.from_array(x), B.DeviceBuffer.from_array(w)
    bb = B.DeviceBuffer.from_array(bias) if has_bias else None
    br = B.DeviceBuffer.from_array(res) if has_res else None
    out = B.DeviceBuffer(cout * Ho * Wo * 4)
    out.fill(0xFF)
    st = B.ops_conv2d(d, bx, bw, bb, br, out, noalloc=noalloc)
    return st, out.to_array().reshape(cout, Ho, Wo), ref


@pytest.mark.parametrize("case", CASES)
def test_conv2d_op_matches_oracle(case):
    B.ops_init()
    st, got, ref = run_case(case)
    assert st == 0, B.last_error()
    assert np.isfinite(got).all()
    assert max_rel_err(got, ref) <= REL_TOL


def test_conv2d_op_rejects_bad_arguments():
    B.ops_init()
    buf = B.DeviceBuffer(1024)
    assert B.ops_conv2d(B.Conv2dDesc(0, 4, 4, 4, 1, 1, 1, 1, 0, 0, 0), buf, buf, None, None, buf) == 1
    assert "bad shape" in B.last_error()
    assert B.ops_conv2d(B.Conv2dDesc(4, 2, 2, 4, 5, 5, 1, 1, 0, 0, 0), buf, buf, None, None, buf) == 1
    assert B.ops_conv2d(B.Conv2dDesc(4, 4, 4, 4, 1, 1, 1, 1, 0, 0, 9), buf, buf, None, None, buf) == 1
