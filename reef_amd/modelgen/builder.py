"""Graph builder that writes REEF model directories for the gfx950 kernels.

Writes the reference's model resource format (graph JSON + ``.param`` +
``.profile.json``; reader src/reef/executor/model.cpp:13-156, writers
script/generate_final_schedule.py:109-144 and script/tvm_generate_model.py:66-76)
with one added key per kernel, ``attrs`` (the shape attributes the shape-generic
kernels need, include/reef_kernels.h), plus ``op`` for human readers.  JSON
values are restricted to ints, strings, lists and dicts, which is all the
reference's parser accepts (src/reef/util/json.cpp).

Every tensor gets its own storage (no buffer reuse), as the reference forces for
its own models (script/generate_final_schedule.py:37-40), so a best-effort task
can be restarted from any kernel after a preemption.
"""
import json
import math
import os
import shutil
import struct

import numpy as np

from . import rng, tiling
from ..paths import code_object

ACT_NONE, ACT_RELU, ACT_RELU6, ACT_GELU = 0, 1, 2, 3
F_BIAS, F_RESIDUAL, F_AFFINE, F_DUAL, F_FUSED_REDUCE, F_PRE_ACT, F_PAIR_FOLD, F_DW_OUTPUT = 1, 2, 4, 8, 16, 32, 64, 128
F_PROJ_OUTPUT = 4096
F_POOL_OUTPUT, F_IN_SHIFT, F_POOL_SHIFT, F_GAP_OUTPUT = 256, 512, 1024, 2048
WG = 256


def float_bits(x):
    return struct.unpack("<i", struct.pack("<f", float(x)))[0]


class Tensor:
    """A storage index plus its logical shape; `off`: the element of the storage at which the
    tensor starts (a view of a part of a larger buffer, the kernels' `arg_offsets`)."""

    def __init__(self, idx, shape, off=0):
        self.idx = idx
        self.shape = tuple(int(s) for s in shape)
        self.off = int(off)

    @property
    def size(self):
        return int(np.prod(self.shape))

    def channels(self, first, count):
        """Channels [first, first + count) of a [C][H][W] tensor: contiguous, so a tensor itself."""
        C, H, W = self.shape
        assert 0 <= first and first + count <= C
        return Tensor(self.idx, (count, H, W), self.off + first * H * W)


class GraphBuilder:
    def __init__(self, name, seed=rng.BASE_SEED, weight_std=None, under_load=False):
        self.name = name
        self.seed = seed
        # the model is meant to run as a best-effort model beside others: tile choices measured
        # with several clients on the device come before those measured alone (tuned.py)
        self.under_load = under_load
        self.weight_std = weight_std   # fixed std (BERT: 0.02); None = He-normal
        self.storage = []
        self.kernels = []
        self.graph_args = []
        self.params = []               # (key, float32 array)
        self._param_pos = {}           # storage index of a parameter -> its place in params
        self.flops = 0                 # algorithmic FLOPs of contractions
        self.kernel_flops = []         # per kernel call
        self.kernel_bytes = []         # algorithmic bytes per kernel call
        self.kernel_est_us = []
        self._np = 0
        self._sync_idx = None
        # "symbol#instance" names give every kernel call its own profile entry
        # (the profile is keyed by kernel name, model.cpp:57-80).
        self.unique_names = True
        # split-K folded inside the conv kernel (False: separate reef_splitk_reduce launch)
        self.fused_reduce = False
        # multi-tap filters on the direct / row tiles also get a copy of their weights in the
        # layout those kernels load fastest (pack_conv_weights); parameter key = weight key + "k"
        self.pack_weights = True
        self.pair_fold = os.environ.get("REEF_PAIR_FOLD", "1") != "0"

    # ------------------------------------------------------------ storages
    def _storage(self, name, size, stype="float32"):
        self.storage.append({"name": name, "size": int(size), "stype": stype})
        return len(self.storage) - 1

    def input(self, name, shape, stype="float32"):
        idx = self._storage(name, int(np.prod(shape)), stype)
        self.graph_args.append(idx)
        return Tensor(idx, shape)

    def temp(self, shape, name="null"):
        return Tensor(self._storage(name, int(np.prod(shape))), shape)

    def workspace(self, n_floats):
        return Tensor(self._storage("temp_arg", int(n_floats) * 4, "byte"), (n_floats,))

    def param(self, shape, std=None, kind="normal", value=None):
        key = "p%d" % self._np
        self._np += 1
        n = int(np.prod(shape))
        if value is not None:
            arr = np.full(n, value, np.float32)
        elif kind == "normal":
            arr = rng.normal_f32(self.name + "/" + key, n, std, self.seed)
        else:
            raise ValueError(kind)
        idx = self._storage(key, n)
        self.graph_args.append(idx)
        self.params.append((key, arr))
        self._param_pos[idx] = len(self.params) - 1
        return Tensor(idx, shape)

    def param_array(self, t):
        """The values of a parameter made by param() (as they stand now)."""
        return self.params[self._param_pos[t.idx]][1]

    def derived_param(self, key, arr):
        """A tensor computed from parameters when the model is generated (its key ends in "k", as the
        packed weight copies' do: readers that want the network's own parameters skip those)."""
        assert key.endswith("k")
        arr = np.ascontiguousarray(arr, np.float32).reshape(-1)
        idx = self._storage(key, arr.size)
        self.graph_args.append(idx)
        self.params.append((key, arr))
        return Tensor(idx, (arr.size,))

    def _sync_counters(self, n):
        """Reserves n counters in the model's sync storage; returns (storage idx, first counter)."""
        if self._sync_idx is None:
            self._sync_idx = self._storage("reef_sync", 0, "int32")
        off = self.storage[self._sync_idx]["size"]
        self.storage[self._sync_idx]["size"] = off + int(n)
        return self._sync_idx, off

    def mark_output(self, t):
        self.storage[t.idx]["name"] = "output"

    # ------------------------------------------------------------ kernels
    def _emit(self, name, tasks, args, attrs, op, flops=0, nbytes=0, est_us=1.0, block=(WG, 1, 1)):
        # an operand is a storage index or a Tensor; a Tensor that starts inside its storage
        # makes the kernel carry "arg_offsets" (bytes; fp32 operands)
        offs = [4 * a.off if isinstance(a, Tensor) else 0 for a in args]
        assert all(o % 16 == 0 for o in offs), "operand views must start on 16 bytes"
        self.kernels.append({
            "name": "%s#%d" % (name, len(self.kernels)) if self.unique_names else name,
            "launch_params": [int(tasks), 1, 1, block[0], block[1], block[2]],
            "args": [a.idx if isinstance(a, Tensor) else int(a) for a in args],
            "attrs": [int(a) for a in attrs],
            "op": op,
        })
        if any(offs):
            self.kernels[-1]["arg_offsets"] = offs
        self.kernel_flops.append(int(flops))
        self.kernel_bytes.append(int(nbytes))
        self.kernel_est_us.append(float(est_us))

    def conv2d(self, x, cout, k, stride=1, pad=0, bias=True, act=ACT_RELU, residual=None,
               affine=False, force=None, dual_act=None, fused_reduce=None, out=None, out_channel=0,
               pre_act=False, given=None, out2=None, gap=False):
        """Fused conv + (residual) + (bias) + (scale, shift) + activation on MFMA.
        gap: return the global average of the layer's output, a (cout,) tensor, instead of the
        output (direct tiles whose pixel groups cover the image: Ho * Wo <= 64; no split).
        pre_act: the layer reads its input through a per-channel scale, shift and ReLU of its own
        (DenseNet pre-activation); folded into the convolution's input loads where a kernel for it
        exists (1x1 filters on the direct tiles), a separate elementwise launch otherwise.
        dual_act: also emit out2 = dual_act(out + shift2[c]) and return (out, out2).
        fused_reduce: fold split-K inside the kernel (default: self.fused_reduce).
        out / out_channel: write into channels [out_channel, out_channel + cout) of an existing
        tensor (a concatenation buffer) instead of a new one.
        given: operands that exist already (an imported graph): {"w", "bias", "scale", "shift"} ->
        Tensor; what is not given is created as a seeded parameter.
        out2: with dual_act, an existing tensor whose first `cout` channels take the second output
        (the two outputs share one destination offset, so both start at their tensors' first
        element here)."""
        given = given or {}
        if fused_reduce is None:
            fused_reduce = self.fused_reduce
        kh, kw = (k, k) if isinstance(k, int) else k
        sh, sw = (stride, stride) if isinstance(stride, int) else stride
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        cin, H, W = x.shape
        Ho = (H + 2 * ph - kh) // sh + 1
        Wo = (W + 2 * pw - kw) // sw + 1
        M, N, K = cout, Ho * Wo, cin * kh * kw
        std = self.weight_std if self.weight_std is not None else math.sqrt(2.0 / K)
        w = given.get("w") or self.param((cout, cin, kh, kw), std)
        w_arr = None if "w" in given else self.params[-1][1]
        flags = 0
        opt = []
        if bias:
            flags |= F_BIAS
            opt.append((given.get("bias") or self.param((cout,), 0.01)).idx)
        if residual is not None:
            flags |= F_RESIDUAL
            assert residual.shape == (cout, Ho, Wo), (residual.shape, (cout, Ho, Wo))
            opt.append(residual)
        if affine:
            flags |= F_AFFINE
            if "scale" in given:
                opt.append(given["scale"].idx)
            else:
                opt.append(self.param((cout,), 0.1, value=None).idx)   # scale ~ N(0, 0.1) + 1 below
                self.params[-1] = (self.params[-1][0], self.params[-1][1] + 1.0)
            opt.append((given.get("shift") or self.param((cout,), 0.01)).idx)
        dst_off = 0
        if out is None:
            out = self.temp((cout, Ho, Wo))
        else:
            assert out.shape[1:] == (Ho, Wo) and out_channel + cout <= out.shape[0]
            dst_off = out.off + out_channel * Ho * Wo
        if dual_act is not None:
            assert not affine
            flags |= F_DUAL
            if out2 is None:
                out2 = self.temp((cout, Ho, Wo))
            else:
                assert dst_off == 0 and out2.off == 0 and out2.shape[1:] == (Ho, Wo) and cout <= out2.shape[0]
            opt.append(out2.idx)
            opt.append(self.param((cout,), 0.01).idx)
        act2 = dual_act or ACT_NONE
        if gap:
            assert out.idx is not None and dual_act is None and not pre_act and dst_off == 0
            tile = self.gap_tile(cin, kh, kw, N)
            assert tile is not None, "no direct tile covers this image"
            force = tiling.forced(tile, M, N, K, 1, kh * kw)
            flags |= F_GAP_OUTPUT
            self.storage[out.idx]["size"] = cout            # the storage holds the averages only
            out = Tensor(out.idx, (cout,))
        t = force or tiling.choose(M, N, K, fused=fused_reduce, pointwise=(kh, kw) == (1, 1),
                                   taps=kh * kw, direct=tiling.direct_ok(cin, kh, kw),
                                   rows=tiling.rows_ok(kh, kw, sh, sw, ph, pw), image=(Ho, Wo),
                                   under_load=self.under_load)
        if t.get("fused"):
            fused_reduce = True       # the measured table asks for the split folded into the launch
        pre = []
        if pre_act:
            if (t["tile"] in tiling.PRE_ACT_TILES and (kh, kw, ph, pw) == (1, 1, 0, 0)
                    and tiling.direct_ok(cin, kh, kw, t["tile"])):
                ps = self.param((cin,), 0.1)
                self.params[-1] = (self.params[-1][0], self.params[-1][1] + 1.0)   # scale ~ 1 + N(0, 0.1)
                pre = [ps.idx, self.param((cin,), 0.01).idx]
            else:
                x = self.eltwise(x, scale=True, shift=True, act=ACT_RELU)
        flops = 2 * M * N * K
        self.flops += flops
        nbytes = 4 * (x.size + M * K + M * N + (M if bias else 0) + (M * N if residual is not None else 0)
                      + (2 * M if affine else 0))
        base = [cin, H, W, cout, Ho, Wo, kh, kw, sh, sw, ph, pw]
        # loader family: direct (only with its own tile), pointwise (1x1/s1/p0, N % 4 == 0),
        # unaligned (K % 4 != 0), general
        if t["tile"] in tiling.ROW_TILES:
            assert tiling.rows_ok(kh, kw, sh, sw, ph, pw) and t["k_chunk"] % 144 == 0
            mode, fam = 5, "r9_"
        elif t["tile"] in tiling.DIRECT_TILES:
            assert tiling.direct_ok(cin, kh, kw, t["tile"]), (cin, kh, kw, t["tile"])
            assert t["k_chunk"] % (kh * kw * (8 if kh * kw == 1 else 1)) == 0
            mode, fam = (4, "p1_") if pre else (3, "d%d_" % (kh * kw))
        elif (kh, kw, sh, sw, ph, pw) == (1, 1, 1, 1, 0, 0) and N % 4 == 0 and K % 4 == 0:
            mode, fam = 1, "pw_"
        elif K % 4 != 0:
            mode, fam = 2, "u_"
        else:
            mode, fam = 0, ""
        kname = "reef_conv2d_" + fam + t["tile"]
        packed = []
        if self.pack_weights and w_arr is not None and (fam, t["tile"]) in PACKED_KERNELS:
            key = self.storage[w.idx]["name"] + "k"
            arr = pack_conv_weights(w_arr.reshape(cout, cin, kh * kw))
            pidx = self._storage(key, arr.size)
            self.graph_args.append(pidx)
            self.params.append((key, arr))
            packed = [pidx]
            kname = "reef_conv2d_" + fam[:-1] + "k_" + t["tile"]
            nbytes_pack = 4 * (arr.size - M * K)        # the copy is read instead of the original
        else:
            nbytes_pack = 0
        if out2 is not None:
            nbytes += 4 * (M * N + M)
        if pre:
            flags |= F_PRE_ACT
            nbytes += 4 * 2 * cin
        if t["split_k"] == 1:
            args = [x, w.idx, out.idx] + opt + pre
            attrs = base + [flags, act, t["tile_id"], 1, t["k_chunk"], t["m_tiles"], t["n_tiles"], act2,
                            0, mode, dst_off, len(args) if packed else 0]
            self._emit(kname, t["tasks"], args + packed, attrs, "conv2d", flops, nbytes + nbytes_pack, t["est_us"])
        elif fused_reduce:
            # workspace: split_k partial tensors; counters: one int per output tile in
            # the model's single sync storage
            # a split of two in the direct family: a third region, the pair slots (REEF_F_PAIR_FOLD)
            pair = t["split_k"] == 2 and mode in (3, 4, 5) and self.pair_fold
            ws = self.workspace((t["split_k"] + (1 if pair else 0)) * M * N)
            sync_idx, sync_off = self._sync_counters(t["m_tiles"] * t["n_tiles"])
            args = [x, w.idx, out.idx] + opt + pre + [ws.idx, sync_idx]
            flags |= F_PAIR_FOLD if pair else 0
            attrs = base + [flags | F_FUSED_REDUCE, act, t["tile_id"], t["split_k"], t["k_chunk"],
                            t["m_tiles"], t["n_tiles"], act2, sync_off, mode, dst_off, len(args) if packed else 0]
            self._emit(kname, t["tasks"], args + packed, attrs, "conv2d", flops, nbytes + nbytes_pack, t["est_us"])
        else:
            ws = self.workspace(t["split_k"] * M * N)
            args = [x, w.idx, ws.idx] + pre
            attrs = base + [F_PRE_ACT if pre else 0, ACT_NONE, t["tile_id"], t["split_k"], t["k_chunk"],
                            t["m_tiles"], t["n_tiles"], ACT_NONE, 0, mode, 0, len(args) if packed else 0]
            self._emit(kname, t["tasks"], args + packed, attrs, "conv2d", flops,
                       4 * (x.size + M * K + t["split_k"] * M * N) + nbytes_pack, t["est_us"])
            self._emit("reef_splitk_reduce", math.ceil(M * N / 1024), [ws.idx, out.idx] + opt,
                       [M, N, t["split_k"], flags & ~F_PRE_ACT, act, act2, dst_off], "splitk_reduce", 0,
                       4 * ((t["split_k"] + 1) * M * N), 2.0)
        return out if out2 is None else (out, out2)

    @staticmethod
    def gap_tile(cin, kh, kw, n_pixels):
        """The narrowest direct tile whose pixel groups cover an image of n_pixels, or None."""
        for tile in ("16x16k4", "16x32k4", "16x64k4"):
            if tiling.TILES[tile][2] >= n_pixels and tiling.direct_ok(cin, kh, kw, tile):
                return tile
        return None

    def conv2d_pool(self, x, cout, act=ACT_RELU, in_shift=False, pool_shift=False, pool_act=ACT_NONE, out=None):
        """7x7 / stride 2 / padding 3 convolution (+ bias, act) of an image of at most 3 channels and the
        3x3 / stride 2 / padding 1 max-pool (+ shift, pool_act) behind it in one launch
        (reef_conv2d_sp7_g2).  in_shift: a per-channel shift on the input, inside the image.
        Parameters are made in the order: input shift, weights, bias, pool shift."""
        cin, H, W = x.shape
        assert cin <= 3, "the fused stem takes at most 3 input channels"
        sh_in = self.param((cin,), 0.01) if in_shift else None
        w = self.param((cout, cin, 7, 7), self.weight_std if self.weight_std is not None else math.sqrt(2.0 / (cin * 49)))
        b = self.param((cout,), 0.01)
        sh_pool = self.param((cout,), 0.01) if pool_shift else None
        Hc, Wc = (H + 6 - 7) // 2 + 1, (W + 6 - 7) // 2 + 1
        Ho, Wo = (Hc + 2 - 3) // 2 + 1, (Wc + 2 - 3) // 2 + 1
        out = Tensor(out.idx, (cout, Ho, Wo), out.off) if out is not None else self.temp((cout, Ho, Wo))
        mt, nt = math.ceil(cout / 16), math.ceil(Ho / 2) * math.ceil(Wo / 14)
        flags = F_BIAS | F_POOL_OUTPUT | (F_IN_SHIFT if in_shift else 0) | (F_POOL_SHIFT if pool_shift else 0)
        args = [x, w.idx, out, b.idx] + ([sh_in.idx] if in_shift else []) + ([sh_pool.idx] if pool_shift else [])
        flops = 2 * cout * cin * 49 * Hc * Wc
        self.flops += flops
        self._emit("reef_conv2d_sp7_g2", mt * nt, args,
                   [cin, H, W, cout, Ho, Wo, 7, 7, 2, 2, 3, 3, flags, act, tiling.TILES["g2"][0], 1,
                    math.ceil(cin * 49 / 4) * 4, mt, nt, pool_act, 0, 7, 0, 0],
                   "conv2d", flops, 4 * (x.size + w.size + cout + out.size), 8.0)
        return out

    XDW_TILES = {"g2": 2, "g4": 4}     # reef_conv2d_xdw_<tile>: image rows per tile

    def conv2d_dw(self, x, cout, act=ACT_RELU6, dw_act=ACT_RELU6, tile=None, stride=1):
        """1x1 convolution (+ bias, act) followed by a depthwise 3x3 convolution (padding 1, stride 1
        or 2, + bias, dw_act) as ONE launch (reef_conv2d_xdw_<tile>, reef_conv2d_xdw2_g2): the front
        half of a MobileNetV2 block without the expanded tensor in memory.  Parameters are created in
        the order the two separate layers would create them."""
        cin, H, W = x.shape
        assert cin % 8 == 0 and stride in (1, 2)
        w = self.param((cout, cin, 1, 1), self.weight_std if self.weight_std is not None else math.sqrt(2.0 / cin))
        b = self.param((cout,), 0.01)
        wd = self.param((cout, 1, 3, 3), self.weight_std if self.weight_std is not None else math.sqrt(2.0 / 9))
        bd = self.param((cout,), 0.01)
        Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
        out = self.temp((cout, Ho, Wo))
        if stride == 2:
            tile = "g2"
        elif tile is None:
            # two image rows per tile; four on large images, where four still leave every CU several
            # workgroups and the rows computed twice by neighbouring tiles weigh more (measured on
            # the shapes of MobileNetV2: 56 x 56 10.7 against 11.9 us, 28 x 28 and below two rows)
            tile = "g4" if H * W >= 3136 else "g2"
        G = self.XDW_TILES[tile]
        mt, nt = math.ceil(cout / 16), math.ceil(Ho / G) * math.ceil(Wo / tiling.ROW_SEG)
        flops = 2 * cout * (H * W * cin + Ho * Wo * 9)
        self.flops += flops
        attrs = [cin, H, W, cout, Ho, Wo, 1, 1, stride, stride, 0, 0, F_BIAS | F_DW_OUTPUT, act, tiling.TILES[tile][0],
                 1, math.ceil(cin / 128) * 128, mt, nt, dw_act, 0, 6, 0, 0]
        self._emit("reef_conv2d_xdw%s_%s" % ("2" if stride == 2 else "", tile), mt * nt,
                   [x, w.idx, out.idx, b.idx, wd.idx, bd.idx], attrs, "conv2d",
                   flops, 4 * (x.size + cout * cin + 11 * cout + out.size), 6.0)
        return out

    BLOCK_TILES = {"sdp": ("g2", "g4"), "xdp2": ("g1", "g2")}      # reef_conv2d_<family>_<tile> that exist

    @staticmethod
    def block_fits(front, cin, cmid, cout, width):
        """Whether a front filter + depthwise 3x3 + projection go into one launch of the block family:
        few enough channels for one workgroup to hold all of them (the kernels move the middle
        channels, and the expansion form its input channels and columns, in fours resp. pairs)."""
        if cmid % 4 != 0 or cout > 32:
            return False
        if front == "stem":
            return cin <= 3 and cmid <= 32
        return cin <= 16 and cin % 4 == 0 and cmid <= 96 and width % 2 == 0

    def conv2d_block(self, x, cmid, cout, front="expand", act=ACT_RELU6, dw_act=ACT_RELU6, tile=None):
        """A whole MobileNetV2 block as ONE launch: the front filter (+ bias, act) -- front="stem": the
        network's 3x3 / stride 2 / padding 1 first layer, then a stride-1 depthwise stage
        (reef_conv2d_sdp_<tile>); front="expand": a 1x1 expansion, then a stride-2 depthwise stage
        (reef_conv2d_xdp2_<tile>) --, the depthwise 3x3 filter (padding 1, + bias, dw_act) and the linear
        1x1 projection (+ bias) to cout channels.  For the blocks at the head of the network: a workgroup
        holds every channel of its pixels, and neither the front filter's result nor the depthwise
        stage's is written.  Parameters are created in the order the three layers would create them."""
        cin, H, W = x.shape
        stem = front == "stem"
        assert self.block_fits(front, cin, cmid, cout, W)
        kf = 3 if stem else 1
        std = lambda fan: self.weight_std if self.weight_std is not None else math.sqrt(2.0 / fan)
        w = self.param((cmid, cin, kf, kf), std(cin * kf * kf))
        b = self.param((cmid,), 0.01)
        wd = self.param((cmid, 1, 3, 3), std(9))
        bd = self.param((cmid,), 0.01)
        wp = self.param((cout, cmid, 1, 1), std(cmid))
        bp = self.param((cout,), 0.01)
        Ho, Wo = (H - 1) // 2 + 1, (W - 1) // 2 + 1
        out = self.temp((cout, Ho, Wo))
        family = "sdp" if stem else "xdp2"
        if tile is None:
            tile = "g4" if stem else "g1"
        assert tile in self.BLOCK_TILES[family]
        G = tiling.ROW_TILES[tile]
        nt = math.ceil(Ho / G) * math.ceil(Wo / tiling.ROW_SEG)
        mid_px = Ho * Wo if stem else H * W
        flops = 2 * (cmid * cin * kf * kf * mid_px + cmid * 9 * Ho * Wo + cout * cmid * Ho * Wo)
        self.flops += flops
        attrs = [cin, H, W, cmid, Ho, Wo, kf, kf, 2, 2, kf // 2, kf // 2, F_BIAS | F_DW_OUTPUT | F_PROJ_OUTPUT, act,
                 tiling.TILES[tile][0], 1, math.ceil(cin * kf * kf / 4) * 4, 1, nt, dw_act, cout, 8, 0, 0]
        self._emit("reef_conv2d_%s_%s" % (family, tile), nt,
                   [x, w.idx, out.idx, b.idx, wd.idx, bd.idx, wp.idx, bp.idx], attrs, "conv2d",
                   flops, 4 * (x.size + w.size + 11 * cmid + wp.size + cout + out.size), 7.0)
        return out

    def dwconv2d(self, x, k, stride=1, pad=0, bias=True, act=ACT_RELU6, out=None, given=None):
        """given: {"w", "bias"} -> existing storages instead of new parameters; out: existing
        storage for the result (an imported graph brings its own)."""
        given = given or {}
        C, H, W = x.shape
        Ho = (H + 2 * pad - k) // stride + 1
        Wo = (W + 2 * pad - k) // stride + 1
        std = self.weight_std if self.weight_std is not None else math.sqrt(2.0 / (k * k))
        w = given.get("w") or self.param((C, 1, k, k), std)
        args = [x.idx, w.idx, None]
        flags = 0
        if bias:
            flags |= 1
            b = given.get("bias") or self.param((C,), 0.01)
        out = Tensor(out.idx, (C, Ho, Wo)) if out is not None else self.temp((C, Ho, Wo))
        args[2] = out.idx
        if bias:
            args.append(b.idx)
        self.flops += 2 * C * Ho * Wo * k * k
        self._emit("reef_dwconv2d", math.ceil(out.size / WG), args,
                   [C, H, W, Ho, Wo, k, k, stride, stride, pad, pad, flags, act], "dwconv2d",
                   2 * C * Ho * Wo * k * k, 4 * (x.size + out.size + C * k * k + C), 2.0)
        return out

    def pool2d(self, x, k, stride, pad, mode="max", bias=False, act=ACT_NONE, count_include_pad=False,
               ceil_mode=False, out=None, bias_t=None, pre=None):
        """pre: (scale, shift) parameters -- the input is read through relu(x * scale[c] + shift[c])."""
        C, H, W = x.shape
        kh, kw = (k, k) if isinstance(k, int) else k
        rnd = math.ceil if ceil_mode else math.floor
        Ho = int(rnd((H + 2 * pad - kh) / stride)) + 1
        Wo = int(rnd((W + 2 * pad - kw) / stride)) + 1
        out = Tensor(out.idx, (C, Ho, Wo), out.off) if out is not None else self.temp((C, Ho, Wo))
        args = [x, out]
        flags = 0
        if bias:
            flags = 1
            args.append((bias_t or self.param((C,), 0.01)).idx)
        if pre is not None:
            flags |= 2
            args += [pre[0].idx, pre[1].idx]
        self._emit("reef_pool2d", math.ceil(out.size / WG), args,
                   [C, H, W, Ho, Wo, kh, kw, stride, stride, pad, pad, 0 if mode == "max" else 1,
                    1 if count_include_pad else 0, flags, act], "pool2d", 0,
                   4 * (x.size + out.size), 2.0)
        return out

    def global_avgpool(self, x, out=None, pre=None):
        """pre: (scale, shift) parameters -- the input is read through relu(x * scale[c] + shift[c])."""
        C = x.shape[0]
        out = Tensor(out.idx, (C,)) if out is not None else self.temp((C,))
        self._emit("reef_global_avgpool", math.ceil(C / 4),
                   [x, out.idx] + ([pre[0].idx, pre[1].idx] if pre is not None else []),
                   [C, x.size // C, 1 if pre is not None else 0],
                   "global_avgpool", 0, 4 * (x.size + C), 2.0)
        return out

    def eltwise(self, a, b=None, scale=False, shift=False, act=ACT_NONE, out=None, shift_t=None):
        C = a.shape[0]
        inner = a.size // C
        out = Tensor(out.idx, a.shape) if out is not None else self.temp(a.shape)
        args = [a.idx, out.idx]
        flags = 0
        n_in = 1
        if b is not None:
            assert b.size == a.size
            flags |= 1
            args.append(b.idx)
            n_in = 2
        if scale:
            flags |= 2
            p = self.param((C,), 0.1)
            self.params[-1] = (self.params[-1][0], self.params[-1][1] + 1.0)
            args.append(p.idx)
        if shift:
            flags |= 4
            args.append((shift_t or self.param((C,), 0.01 if not isinstance(shift, float) else shift)).idx)
        self._emit("reef_eltwise", math.ceil(a.size / 1024), args, [C, inner, flags, act], "eltwise",
                   0, 4 * (n_in + 1) * a.size, 2.0)
        return out

    def dense(self, x, out_f, bias=True, act=ACT_NONE, rows=1, out=None, w=None, bias_t=None):
        in_f = x.size // rows
        std = self.weight_std if self.weight_std is not None else math.sqrt(2.0 / in_f)
        w = w or self.param((out_f, in_f), std)
        out = Tensor(out.idx, (rows, out_f)) if out is not None else self.temp((rows, out_f))
        args = [x.idx, w.idx, out.idx]
        flags = 0
        if bias:
            flags = 1
            args.append((bias_t or self.param((out_f,), 0.01)).idx)
        self.flops += 2 * rows * in_f * out_f
        self._emit("reef_dense", math.ceil(out_f / 4), args, [rows, in_f, out_f, flags, act],
                   "dense", 2 * rows * in_f * out_f, 4 * (x.size + in_f * out_f + rows * out_f), 2.0)
        return out

    def softmax(self, x, rows, cols, out=None, mask=None):
        """mask: a uint1 storage of `cols` bytes; a non-zero byte turns its column into -inf."""
        out = Tensor(out.idx, (rows, cols)) if out is not None else self.temp((rows, cols))
        args = [x.idx, out.idx] + ([mask.idx] if mask is not None else [])
        self._emit("reef_softmax", math.ceil(rows / 4), args, [rows, cols, 1 if mask is not None else 0],
                   "softmax", 0, 8 * rows * cols, 2.0)
        return out

    def pre_act_params(self, c):
        """scale ~ 1 + N(0, 0.1), shift ~ N(0, 0.01): what conv2d(pre_act=True) makes for itself."""
        ps = self.param((c,), 0.1)
        self.params[-1] = (self.params[-1][0], self.params[-1][1] + 1.0)
        return ps, self.param((c,), 0.01)

    def layernorm_params(self, cols):
        """gamma ~ 1 + N(0, 0.1), beta ~ N(0, 0.01): the parameters layernorm() makes for itself."""
        gamma = self.param((cols,), 0.1)
        self.params[-1] = (self.params[-1][0], self.params[-1][1] + 1.0)
        return gamma, self.param((cols,), 0.01)

    def layernorm(self, x, rows, cols, res=None, eps=1e-12, out=None, gamma=None, beta=None):
        if gamma is None:
            gamma, b = self.layernorm_params(cols)
            beta = b if beta is None else beta
        if beta is None:
            beta = self.param((cols,), 0.01)
        out = Tensor(out.idx, (rows, cols)) if out is not None else self.temp((rows, cols))
        args = [x.idx, gamma.idx, beta.idx, out.idx]
        flags = 0
        if res is not None:
            flags = 1
            args.append(res.idx)
        self._emit("reef_layernorm", math.ceil(rows / 4), args, [rows, cols, flags, float_bits(eps)],
                   "layernorm", 0, 4 * rows * cols * (3 if res is not None else 2), 2.0)
        return out

    def bias_gelu(self, x, rows, cols, bias=True, out=None):
        out = Tensor(out.idx, (rows, cols)) if out is not None else self.temp((rows, cols))
        args = [x.idx, out.idx]
        if bias:
            args.append(self.param((cols,), 0.01).idx)
        self._emit("reef_bias_gelu", math.ceil(rows * cols / 1024), args, [rows, cols, 1 if bias else 0],
                   "bias_gelu", 0, 8 * rows * cols, 2.0)
        return out

    def embedding(self, ids, vocab, seq, hidden, pos=True, seg=True, tok=None, out=None):
        tok = tok or self.param((vocab, hidden), self.weight_std or 0.02)
        out = Tensor(out.idx, (seq, hidden)) if out is not None else self.temp((seq, hidden))
        args = [ids.idx, tok.idx, out.idx]
        flags = 0
        if pos:
            flags |= 1
            args.append(self.param((seq, hidden), self.weight_std or 0.02).idx)
        if seg:
            flags |= 2
            args.append(self.param((hidden,), self.weight_std or 0.02).idx)
        self._emit("reef_embedding", math.ceil(seq * hidden / 1024), args, [seq, hidden, flags, vocab],
                   "embedding", 0, 4 * seq * hidden * 3, 2.0)
        return out

    ATTENTION_MAX_SEQ, ATTENTION_MAX_HEAD_DIM, ATTENTION_ROWS = 128, 64, 8    # REEF_AT_* of include/reef_kernels.h

    @classmethod
    def attention_ok(cls, seq, head_dim, ld, ldo, offs):
        """Whether reef_attention takes this shape (all keys of a head fit a workgroup's LDS)."""
        return (seq <= cls.ATTENTION_MAX_SEQ and head_dim <= cls.ATTENTION_MAX_HEAD_DIM
                and all(v % 4 == 0 for v in (head_dim, ld, ldo) + tuple(offs)))

    def attention(self, qkv, seq, heads, head_dim, ld, off_q, off_k, off_v, alpha, mask=None, out=None, ldo=None):
        """softmax(alpha Q K^T (masked)) V for every head in one launch; Q, K, V are column blocks
        of qkv [seq][ld] (head h at columns off + h * head_dim), the context goes to
        out [seq][ldo] at columns h * head_dim."""
        ldo = heads * head_dim if ldo is None else ldo
        assert self.attention_ok(seq, head_dim, ld, ldo, (off_q, off_k, off_v))
        out = Tensor(out.idx, (seq, ldo)) if out is not None else self.temp((seq, ldo))
        args = [qkv.idx, out.idx] + ([mask.idx] if mask is not None else [])
        flops = 4 * heads * seq * seq * head_dim
        self.flops += flops
        self._emit("reef_attention", heads * math.ceil(seq / self.ATTENTION_ROWS), args,
                   [seq, head_dim, heads, ld, ldo, off_q, off_k, off_v, float_bits(alpha), 1 if mask is not None else 0],
                   "attention", flops, 4 * (3 * seq * heads * head_dim + seq * ldo), 4.0)
        return out

    def copy_into(self, src, dst, dst_off):
        self._emit("reef_copy", math.ceil(src.size / 1024), [src.idx, dst.idx], [src.size, dst_off],
                   "copy", 0, 8 * src.size, 2.0)

    def transpose_102(self, x, d0, d1, d2, bias=None, out=None):
        out = Tensor(out.idx, (d1, d0, d2)) if out is not None else self.temp((d1, d0, d2))
        args = [x.idx, out.idx]
        flags = 0
        if bias is not None:
            flags = 1
            args.append(bias.idx)
        self._emit("reef_transpose", math.ceil(d0 * d1 * d2 / 1024), args, [d0, d1, d2, flags],
                   "transpose", 0, 8 * d0 * d1 * d2, 2.0)
        return out

    def gemm(self, a, b, M, N, K, batch=1, trans_b=True, bias=None, act=ACT_NONE, alpha=1.0,
             lda=None, ldb=None, ldc=None, stride_a=0, stride_b=0, stride_c=0, out=None, force_tile=None,
             off_a=0, off_b=0, off_c=0, ln=None, res=None, split_k=None):
        """C[b] = act(alpha * A[b] x B[b] (+bias)) (+res[b]); operands are storages with explicit strides.
        res: a residual laid out as C is.
        split_k: K split across workgroups and folded inside the launch (direct tiles, batch 1);
        None = what tiling.choose_gemm finds (1 or 2).
        force_tile: a staged tile name or, for trans_b, one of tiling.GEMM_DIRECT_TILES.
        off_a / off_b / off_c: element at which the first matrix starts inside its storage.
        ln: dict(gamma=, beta=, eps=1e-12, out=None) -- the product behind a LayerNorm of the rows
        of A; `out`, if given, receives the normalised rows (kernels reef_gemm_ntl_<tile>: staged
        tiles, one K-contiguous B).  b, gamma and beta must be parameters: the kernel works from
        b scaled by gamma and two vectors derived from them (include/reef_kernels.h)."""
        lda = K if lda is None else lda
        ldb = (K if trans_b else N) if ldb is None else ldb
        ldc = N if ldc is None else ldc
        if out is None:
            out = self.temp((batch, M, N))
        assert off_a % 4 == 0 and off_b % 4 == 0 and off_c % 4 == 0, "gemm operands must be 16-byte aligned"
        direct_ok = (trans_b and K % 8 == 0 and lda % 4 == 0 and ldb % 4 == 0 and stride_a % 4 == 0
                     and stride_b % 4 == 0)
        if ln is not None:
            assert trans_b and batch == 1 and off_a == 0, "the LayerNorm form: one K-contiguous B, A without offset"
            direct_ok = False
            if force_tile is None:
                force_tile = self.LN_GEMM_TILE
            assert force_tile in self.LN_GEMM_TILES, "no LayerNorm form of this tile"
        if force_tile is not None:
            t = tiling.forced(force_tile, M, N, K, 1)
        else:
            t = tiling.choose_gemm(M, N, K, batch, direct_ok, under_load=self.under_load)
        direct = t["tile"] in tiling.GEMM_DIRECT_TILES
        assert direct_ok or not direct, "this GEMM has no direct form"
        args = [a.idx, b.idx, out.idx]
        if ln is not None:
            # Wg = W gamma (column k scaled by gamma[k]); c1 = its row sums; c2 = W beta
            assert ldb == K and off_b == 0, "the LayerNorm form takes the weight matrix whole"
            W = self.param_array(b).reshape(N, K).astype(np.float64)
            gm = self.param_array(ln["gamma"]).astype(np.float64)
            bt = self.param_array(ln["beta"]).astype(np.float64)
            wkey = self.storage[b.idx]["name"]
            Wg = (W * gm[None, :]).astype(np.float32)
            args[1] = self.derived_param(wkey + "gk", Wg).idx      # the storage named wkey keeps W itself
            ln = dict(ln, c1=self.derived_param(wkey + "sk", Wg.astype(np.float64).sum(axis=1)),
                      c2=self.derived_param(wkey + "tk", W @ bt))
        flags = 0
        if bias is not None:
            flags = 1
            args.append(bias.idx)
        if res is not None:
            flags |= 8
            args.append(res.idx)
        attrs_split = []
        tasks = batch * t["m_tiles"] * t["n_tiles"]
        if split_k is None:
            split_k = t.get("gemm_split", 1)
        if split_k > 1:
            assert direct and batch == 1, "only the direct tiles split K, and only without a batch"
            k_chunk = math.ceil(math.ceil(K / split_k) / 128) * 128
            split_k = math.ceil(K / k_chunk)
        if split_k > 1:
            pair = split_k == 2 and self.pair_fold
            ws = self.workspace((split_k + (1 if pair else 0)) * M * N)
            sync_idx, sync_off = self._sync_counters(t["m_tiles"] * t["n_tiles"])
            args += [ws.idx, sync_idx]
            flags |= 16 if pair else 0
            attrs_split = [split_k, k_chunk, sync_off]
            tasks *= split_k
        attrs_ln = []
        if ln is not None:
            flags |= 2
            args += [ln["c1"].idx, ln["c2"].idx, ln["gamma"].idx, ln["beta"].idx]
            if ln.get("out") is not None:
                flags |= 4
                args.append(ln["out"].idx)
            attrs_ln = [float_bits(ln.get("eps", 1e-12))]
        flops = 2 * batch * M * N * K
        self.flops += flops
        assert K % 4 == 0 and lda % 4 == 0 and stride_a % 4 == 0, "gemm operands must be 16-byte aligned"
        if trans_b:
            assert ldb % 4 == 0 and stride_b % 4 == 0, "gemm operands must be 16-byte aligned"
        self._emit("reef_gemm_%s_%s" % ("ntl" if ln is not None else "ntd" if direct else "nt" if trans_b else "nn", t["tile"]),
                   tasks, args,
                   [batch, M, N, K, 1 if trans_b else 0, flags, act, float_bits(alpha), t["tile_id"],
                    t["m_tiles"], t["n_tiles"], lda, ldb, ldc, stride_a, stride_b, stride_c,
                    off_a, off_b, off_c] + ((attrs_ln or [0]) + attrs_split if attrs_split else attrs_ln),
                   "gemm", flops, 4 * batch * (M * K + N * K + M * N), t["est_us"])
        return out

    LN_GEMM_TILES = ("32x32k4", "64x32k2")     # tiles that exist as reef_gemm_ntl_<tile>
    LN_GEMM_TILE = "32x32k4"

    def mocked(self, name, a, b, out):
        self._emit(name, 64, [a.idx, b.idx, out.idx], [], "mocked", 0, 3 * 8192 * 4, 14.0,
                   block=(4, 8, 4))

    # ------------------------------------------------------------ output
    def model_dict(self):
        shared = {}
        for k in self.kernels:
            n = k["name"]
            sym = n.split("#")[0]
            if sym == "reef_conv2d_sp7_g2":
                shared[n] = (3 * 15 * 64 + 16 * (5 * 32 + 1) + 32 + 16 * 3 * 49) * 4 + 16     # TileSp7: input patch, pooled-from block, weight rows
            elif sym.startswith("reef_conv2d_sdp_") or sym.startswith("reef_conv2d_xdp2_"):
                # TileBlk: patch, the three layers' parameters, the front filter's result, the depthwise stage's
                stem, G = sym.startswith("reef_conv2d_sdp_"), tiling.ROW_TILES[sym.split("_")[-1]]
                R, S, CM, KC = (G + 2, 1, 32, 1) if stem else (2 * G + 1, 2, 96, 4)
                NG = R * S
                patch = 3 * (2 * R + 1) * 36 if stem else NG * 16 * (4 * KC + 4)
                wfs = 36 if stem else 4 * KC + 4
                floats = (patch + CM * wfs + CM + CM * 9 + CM + 32 + CM * (NG * 16 + (20 if NG % 2 == 0 else 4))
                          + G * 16 * (CM + 4))
                shared[n] = floats * 4 + 16
            elif sym.startswith("reef_conv2d_xdw"):
                G, S = self.XDW_TILES[sym.split("_")[-1]], 2 if sym.startswith("reef_conv2d_xdw2_") else 1
                NG = (G + 2) if S == 1 else (2 * G + 1) * 2      # TileXdw: pixel groups of the 1x1 result
                PS = (96 if S == 2 else 64 if G == 4 else 160) + 4     # a chunk of input channels per pixel / weight row
                shared[n] = (NG * 16 * PS + 16 * PS + 16 * (NG * 16 + 20)) * 4 + 16
            elif sym.startswith("reef_conv2d_") or sym.startswith("reef_gemm_"):
                shared[n] = tiling.lds_bytes(sym.split("_")[-1])
                if sym.startswith("reef_gemm_ntl_"):
                    shared[n] += 2 * tiling.TILES[sym.split("_")[-1]][1] * 4    # mean, 1/std of the tile's rows
            else:
                shared[n] = 4   # the reference's floor (generate_final_schedule.py:117-143)
        return {"storage": self.storage, "kernels": self.kernels, "args": self.graph_args,
                "shared_memory": shared}

    def profile_dict(self, measured_us=None, occupancy_levels=8):
        """Estimated (or measured) per-kernel latency table, keyed by kernel name as the
        reference's profile is (model.cpp:57-80).  Kernels sharing a name share one
        entry; the table keeps the slowest instance, which keeps DKP conservative."""
        lat = {}
        total = 0
        for i, k in enumerate(self.kernels):
            us = measured_us[i] if measured_us is not None else self.kernel_est_us[i]
            us = max(1, int(math.ceil(us)))
            total += us
            e = lat.setdefault(k["name"], {"total_latency": 0, "latency": [0] * occupancy_levels})
            e["total_latency"] = max(e["total_latency"], us)
            e["latency"] = [max(v, us) for v in e["latency"]]
        return {"model_latency": total, "kernel_latency": lat}

    def write(self, out_dir, link_code_objects=True, measured_us=None):
        os.makedirs(out_dir, exist_ok=True)
        base = os.path.join(out_dir, self.name)
        with open(base + ".json", "w") as f:
            json.dump(self.model_dict(), f)
        with open(base + ".profile.json", "w") as f:
            json.dump(self.profile_dict(measured_us), f, separators=(",", ":"))
        if self.params:   # the file is optional (src/reef/server/server.cpp:64-68)
            write_params(base + ".param", self.params)
        if link_code_objects:
            for fl in ("raw", "be", "trans"):
                dst = "%s.%s.co" % (base, fl)
                if os.path.lexists(dst):
                    os.remove(dst)
                shutil.copyfile(code_object(fl), dst)
        meta = {"flops": self.flops, "kernel_flops": self.kernel_flops,
                "kernel_bytes": self.kernel_bytes}
        with open(base + ".meta.json", "w") as f:
            json.dump(meta, f)
        return base


# (loader family prefix, tile) of the kernels that exist in a packed-weights form
PACKED_KERNELS = {("r9_", "g1"), ("r9_", "g2"), ("r9_", "g4"), ("d9_", "16x16k4"), ("d9_", "16x32k4"),
                  ("d9_", "32x32d4"), ("d3_", "16x16k4"), ("d3_", "16x32k4"), ("d7_", "16x16k4"),
                  ("d7_", "16x32k4"), ("d25_", "16x16k4"), ("d25_", "16x32k4")}


def pack_conv_weights(w):
    """[Cout][Cin][taps] weights -> the layout of attr REEF_CONV_WPACK:
    [ceil(Cout/16)][ceil(Cin/4)][ceil(taps/4)][4 channels][16 rows][4 taps], zero-padded."""
    M, C, R = w.shape
    mt, c4, g4 = -(-M // 16), -(-C // 4), -(-R // 4)
    pad = np.zeros((mt * 16, c4 * 4, g4 * 4), np.float32)
    pad[:M, :C, :R] = w
    # pad[mt*16 + i, c4*4 + kq, g*4 + j] -> out[mt, c4, g, kq, i, j]
    out = pad.reshape(mt, 16, c4, 4, g4, 4).transpose(0, 2, 4, 3, 1, 5)
    return np.ascontiguousarray(out).reshape(-1)


def write_params(path, params):
    """``.param`` writer (script/tvm_generate_model.py:66-76)."""
    with open(path, "wb") as f:
        f.write(b"TVM_MODEL_PARAMS\0")
        f.write(struct.pack("<Q", len(params)))
        for key, arr in params:
            arr = np.ascontiguousarray(arr, dtype="<f4").reshape(-1)
            f.write(key.encode("ascii") + b"\0")
            f.write(struct.pack("<Q", arr.size))
            f.write(arr.tobytes())
