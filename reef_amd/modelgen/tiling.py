"""Tile and split-K choice for the implicit-GEMM convolution / GEMM kernels.

The reference takes grid and block sizes from TVM's tuned schedules
(script/generate_final_schedule.py:98: launch_params come from the raw
schedule).  Here the generator picks, per layer, one of the compiled tile
configurations and a split-K factor from a small analytic cost model of a
256-CU part: batch-1 layers are tiny (49..3136 output pixels), so most need
split-K to put a workgroup on every CU.
"""
import math

from .tuned import TUNED, TUNED_UNDER_LOAD, GEMM_UNDER_LOAD

# name -> (id, BM, BN, relative MFMA efficiency of the inner loop, workgroups per CU)
TILES = {
    "128x128": (0, 128, 128, 1.00, 2),
    "128x64": (1, 128, 64, 0.85, 2),
    "64x64": (2, 64, 64, 0.60, 4),
    "128x32": (3, 128, 32, 0.60, 3),
    "32x128": (4, 32, 128, 0.60, 3),
    "64x128": (5, 64, 128, 0.85, 2),
    # k<n>: the workgroup's four wavefronts split K n ways on one small tile
    "32x32k4": (6, 32, 32, 0.50, 2),
    "64x32k2": (7, 64, 32, 0.55, 3),
    "32x64k2": (8, 32, 64, 0.55, 3),
    # direct family (reef_conv2d_d<taps>_16x16k4): picked through the measured table, an explicit
    # request, or for a shape outside the table by the cost model direct_cost below
    "16x16k4": (9, 16, 16, 0.40, 2),
    "16x32k4": (10, 16, 32, 0.40, 2),
    "16x64k4": (11, 16, 64, 0.40, 2),
    "32x32d4": (12, 32, 32, 0.40, 2),   # direct; the name differs from the staged 32x32k4
    # row form of the direct 3x3 / stride 1 / padding 1 convolution (reef_conv2d_r9_<name>): BM output
    # channels x G image rows x one 14-column segment; BN here is the nominal 16 G lanes it computes
    "g1": (13, 16, 16, 0.40, 2),
    "g2": (14, 16, 32, 0.40, 2),
    "g4": (15, 16, 64, 0.40, 2),
    "g7": (16, 16, 112, 0.40, 2),
    "g2m2": (17, 32, 32, 0.40, 2),
    "g4m2": (18, 32, 64, 0.40, 2),
}
# row form: image rows per tile
ROW_TILES = {"g1": 1, "g2": 2, "g4": 4, "g7": 7, "g2m2": 2, "g4m2": 4}
ROW_SEG = 14
DIRECT_TILE = "16x16k4"
DIRECT_TILES = ("16x16k4", "16x32k4", "16x64k4", "32x32d4")
# filter sizes kh*kw each direct tile is compiled for
PRE_ACT_TILES = ("16x16k4", "16x32k4", "32x32d4")   # tiles with a pre-activation 1x1 kernel (reef_conv2d_p1_*)
DIRECT_TAPS = {"16x16k4": (1, 3, 7, 9, 25), "16x32k4": (1, 3, 7, 9, 25), "16x64k4": (1, 9), "32x32d4": (1, 9)}
# wavefronts that share one output block and split K inside the workgroup
KW = {"32x32k4": 4, "64x32k2": 2, "32x64k2": 2}
GEMM_TILES = ("128x128", "64x64", "32x128", "32x32k4", "64x32k2")


GEMM_DIRECT_TILES = ("16x16k4", "16x32k4", "32x32d4")   # reef_gemm_ntd_<tile>


def choose_gemm(M, N, K, batch=1, direct_ok=False, under_load=False):
    """Tile of a GEMM, and for a direct tile whether K is split in two across workgroups.
    Without a measured table: the staged choice of the analytic model, against the direct tiles
    (both operands K-contiguous) scored by the rule the batch-1 convolutions were found to
    follow -- a workgroup's time grows with the cache lines it has to pull in, (BM + BN) K / 32
    of them, and workgroups beyond one per CU queue up.  A split of two (folded inside the
    launch through the pair slots) halves a workgroup's lines and doubles the workgroups, at a
    price measured on BERT-base's 128 x 768 x 3072 product (32x32d4: 25.8 us whole, 16.8 us
    split in two, against 19.4 us for 16x32k4 whole; splits of three and more meet on counters
    and were slower throughout).
    under_load: the product belongs to a model that shares the device with other streams; a
    choice measured for that case (tuned.GEMM_UNDER_LOAD) comes first."""
    if under_load and direct_ok and batch == 1 and (M, N, K) in GEMM_UNDER_LOAD:
        tile, split = GEMM_UNDER_LOAD[(M, N, K)]
        t = forced(tile, M, N, K, 1)
        t["gemm_split"] = split
        return t
    staged = choose(M, N, K, allow_split=False, tiles=GEMM_TILES)
    if not direct_ok:
        return staged

    def cost(bm, bn, split=1):
        wgs = batch * math.ceil(M / bm) * math.ceil(N / bn) * split
        return math.ceil(wgs / NUM_CUS) * (bm + bn) * (K / split) / 32.0 + (GEMM_PAIR_FOLD_LINES if split == 2 else 0)
    cands = [(t, 1) for t in GEMM_DIRECT_TILES]
    if batch == 1 and K >= 1024:
        cands += [(t, 2) for t in GEMM_DIRECT_TILES]
    best, split = min(cands, key=lambda c: (cost(TILES[c[0]][1], TILES[c[0]][2], c[1]), c[1],
                                            -TILES[c[0]][1] * TILES[c[0]][2]))
    _, bm, bn, _, _ = TILES[staged["tile"]]
    if cost(bm, bn) * GEMM_STAGED_BONUS <= cost(TILES[best][1], TILES[best][2], split):
        return staged
    t = forced(best, M, N, K, 1)
    t["gemm_split"] = split
    return t


GEMM_PAIR_FOLD_LINES = 900.0    # what a split of two costs, in the cost rule's cache lines
GEMM_STAGED_BONUS = 1.0


def step_k(tile, taps=1):
    """Granularity of a split's share of K (taps = kh*kw, direct family only: 16 channels of a
    filter with taps > 1, one K step; 128 channels of a 1x1 filter, two of its 64-channel steps --
    rounding to 64 instead was measured on DenseNet-201 and changes nothing)."""
    if tile in DIRECT_TILES:
        return 128 if taps == 1 else 16 * taps
    return BK * KW.get(tile, 1)


def direct_ok(cin, kh, kw, tile=DIRECT_TILE):
    """Whether the direct family has a kernel for this filter (and tile)."""
    taps = kh * kw
    if taps not in DIRECT_TAPS[tile]:
        return False
    return taps > 1 or cin % 8 == 0


def rows_ok(kh, kw, sh, sw, ph, pw):
    """Whether the row form has a kernel for this filter."""
    return (kh, kw, sh, sw, ph, pw) == (3, 3, 1, 1, 1, 1)


def forced_rows(tile, M, H, W, K, split=1):
    """Launch geometry of a row-form tile: spatial tiles are G image rows x one 14-column segment."""
    tid, bm, _, _, _ = TILES[tile]
    G = ROW_TILES[tile]
    bk = 16 * 9
    k_chunk = math.ceil(math.ceil(K / split) / bk) * bk
    s = math.ceil(K / k_chunk)
    mt = math.ceil(M / bm)
    nt = math.ceil(H / G) * math.ceil(W / ROW_SEG)
    return dict(tile=tile, tile_id=tid, BM=bm, BN=16 * G, split_k=s, k_chunk=k_chunk, m_tiles=mt,
                n_tiles=nt, tasks=s * mt * nt, est_us=1.0)


def forced(tile, M, N, K, split=1, taps=1):
    """The launch geometry of a given tile and split-K factor (no cost model)."""
    assert tile not in ROW_TILES, "row-form tiles take the image shape: forced_rows"
    tid, bm, bn, _, _ = TILES[tile]
    bk = step_k(tile, taps)
    k_chunk = math.ceil(math.ceil(K / split) / bk) * bk
    s = math.ceil(K / k_chunk)
    mt, nt = math.ceil(M / bm), math.ceil(N / bn)
    return dict(tile=tile, tile_id=tid, BM=bm, BN=bn, split_k=s, k_chunk=k_chunk, m_tiles=mt,
                n_tiles=nt, tasks=s * mt * nt, est_us=1.0)

NUM_CUS = 256
BK = 32
# Cost model constants (microseconds); calibrated against measured kernels.
T_STEP_128x128 = 1.9     # one BK=32 step of a 128x128 tile on one CU at efficiency 1.0
T_FIXED = 2.0            # prologue + epilogue of a workgroup
T_REDUCE_LAUNCH = 3.0    # extra launch of the split-K reduce
T_FUSED_REDUCE = 1.0     # fence + last-arrival fold inside the conv kernel
HBM_BYTES_PER_US = 4.0e6
# The constants above describe a workgroup in a long, warm run; in a model (cold operands, one
# launch per layer) the staged tiles measure about three times that, on small and on
# device-filling layers alike (sweeps behind tuned.py; bench.py's steady_state_conv).  With the
# factor the estimate is in the same microseconds as direct_cost, and choosing between the two
# families by estimate loses 7 % against the measured best over the 181 shapes of the sweeps.
STAGED_SCALE = 3.0


def _steps_time(bm, bn, eff, steps):
    return steps * T_STEP_128x128 * (bm * bn) / (128.0 * 128.0) / eff


def choose(M, N, K, allow_split=True, tiles=None, max_split=32, fused=True, pointwise=False,
           taps=1, direct=False, rows=False, image=None, under_load=False):
    """Returns dict(tile, tile_id, BM, BN, split_k, k_chunk, m_tiles, n_tiles, tasks).
    Measured choices (tuned.py) win over the analytic model for the shapes they cover; an entry
    that names the direct tile counts only if the caller says the filter qualifies.
    under_load: the layer belongs to a model that shares the device with other streams; the
    entries measured for that case (TUNED_UNDER_LOAD) come before those measured alone."""
    if allow_split and tiles is None and not fused:
        key = (M, N, K, 1 if pointwise else 0)
        hit = TUNED.get(key)
        if under_load and key in TUNED_UNDER_LOAD:
            hit = TUNED_UNDER_LOAD[key] + (hit[2] if hit is not None else 0.0,)
        if hit is not None and hit[0] in ROW_TILES:
            if rows and image is not None:
                t = forced_rows(hit[0], M, image[0], image[1], K, abs(hit[1]))
                t["est_us"] = hit[2]
                t["fused"] = hit[1] < 0
                return t
            hit = None
        if hit is not None and (hit[0] not in DIRECT_TILES or direct):
            # a negative split factor in the table: the split is folded inside the launch
            t = forced(hit[0], M, N, K, abs(hit[1]), taps)
            t["est_us"] = hit[2]
            t["fused"] = hit[1] < 0
            return t
    best = None
    if allow_split and tiles is None and direct:
        best = _choose_direct(M, N, K, taps, fused, rows, image)
    for name in (tiles or [t for t in TILES if t not in DIRECT_TILES and t not in ROW_TILES]):
        tid, bm, bn, eff, occ = TILES[name]
        m_tiles, n_tiles = math.ceil(M / bm), math.ceil(N / bn)
        nt = m_tiles * n_tiles
        splits = [1]
        if allow_split:
            splits += [s for s in (2, 3, 4, 6, 8, 12, 16, 24, 32) if s <= max_split]
        bk = step_k(name)
        for s in splits:
            k_chunk = math.ceil(math.ceil(K / s) / bk) * bk
            s_eff = math.ceil(K / k_chunk)
            if s_eff != s and s != 1:
                continue
            wgs = nt * s_eff
            rounds = math.ceil(wgs / (NUM_CUS * occ))
            # co-resident workgroups share the CU's matrix pipe
            share = min(occ, math.ceil(wgs / NUM_CUS))
            t = rounds * (_steps_time(bm, bn, eff, k_chunk // bk) * share + T_FIXED)
            if s_eff > 1:
                t += (T_FUSED_REDUCE if fused else T_REDUCE_LAUNCH) + (s_eff + 1) * M * N * 4 / HBM_BYTES_PER_US
            t *= STAGED_SCALE
            cand = (t, name, s_eff, k_chunk, m_tiles, n_tiles)
            if best is None or cand[0] < best[0] - 1e-9:
                best = cand
    if len(best) == 2:          # a direct or row-form geometry, complete already
        return best[1]
    t, name, s, k_chunk, m_tiles, n_tiles = best
    tid, bm, bn, _, _ = TILES[name]
    return dict(tile=name, tile_id=tid, BM=bm, BN=bn, split_k=s, k_chunk=k_chunk,
                m_tiles=m_tiles, n_tiles=n_tiles, tasks=s * m_tiles * n_tiles, est_us=t)


# Cost of a direct-family launch in microseconds, for shapes the measured table does not cover.
# Linear in what the batch-1 sweeps showed to matter: the cache lines a workgroup pulls in,
# (BM + BN) K_chunk / 32, times the rounds of workgroups the device needs; the workgroups per
# CU; and what a split of K adds (folded inside the launch, or as a launch of its own).  The
# constants are a least-squares fit over the 4095 direct candidates of the sweeps behind
# tuned.py (181 shapes of four networks, rms error 12 %); choosing by this model instead of by
# measurement costs 7 % on average over those shapes (worst case 1.5x), where the staged tiles
# alone cost 62 % (worst 2.8x).
DIRECT_COST = dict(fixed=3.57, per_line_round=0.00377, fused_split=2.20, separate_split=2.92,
                   per_wg_per_cu=0.689, per_split=0.172)


def direct_cost(tile, geom, fused):
    _, bm, bn, _, _ = TILES[tile]
    c = DIRECT_COST
    s = geom["split_k"]
    lines = (bm + bn) * geom["k_chunk"] / 32.0
    t = c["fixed"] + c["per_line_round"] * lines * math.ceil(geom["tasks"] / NUM_CUS) \
        + c["per_wg_per_cu"] * geom["tasks"] / NUM_CUS
    if s > 1:
        t += (c["fused_split"] if fused else c["separate_split"]) + c["per_split"] * s
    return t


def _choose_direct(M, N, K, taps, fused, rows, image):
    """Best direct (or row-form) tile and split by direct_cost; (cost, geometry)."""
    best = None
    for tile in DIRECT_TILES:
        if taps not in DIRECT_TAPS[tile]:
            continue
        for s in (1, 2, 3, 4, 6, 8, 12, 16):
            g = forced(tile, M, N, K, s, taps)
            if g["split_k"] != s:
                continue
            t = direct_cost(tile, g, fused)
            if best is None or t < best[0] - 1e-9:
                g["est_us"] = t
                g["fused"] = fused and s > 1
                best = (t, g)
    if rows and image is not None and best is not None:
        # the row form of the same nominal tile loads each input value once instead of once per
        # tap: measured 5 to 10 % ahead of the tap form on the 3x3 layers of the table
        for tile in ("g2", "g4"):
            for s in (1, 2, 3, 4, 6, 8):
                g = forced_rows(tile, M, image[0], image[1], K, s)
                if g["split_k"] != s:
                    continue
                t = 0.93 * direct_cost(tile, g, fused)
                if t < best[0] - 1e-9:
                    g["est_us"] = t
                    g["fused"] = fused and s > 1
                    best = (t, g)
    return best


def lds_bytes(tile):
    if tile in DIRECT_TILES or tile in ROW_TILES:
        # four wavefronts x (BM/16)(BN/16) partial 16x16 tiles (skewed rows) + leave / last-arrival flags
        return 4 * (TILES[tile][1] // 16) * (TILES[tile][2] // 16) * 320 * 4 + 16
    _, bm, bn, _, _ = TILES[tile]
    bk = step_k(tile)
    a = bm * (bk + 4)
    b = max(bk * bn, bn * (bk + 4))
    return 2 * (a + b) * 4 + 16
