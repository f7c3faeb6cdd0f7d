#include "executor/op_extents.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "reef_kernels.h"

namespace reef {
namespace executor {

int op_from_symbol(const std::string& n) {
    struct { const char* prefix; int op; } table[] = {
        {"reef_conv2d_", REEF_OP_CONV2D}, {"reef_gemm_", REEF_OP_GEMM},
        {REEF_K_SPLITK_REDUCE, REEF_OP_SPLITK_REDUCE}, {REEF_K_DWCONV2D, REEF_OP_DWCONV2D},
        {REEF_K_POOL2D, REEF_OP_POOL2D}, {REEF_K_GLOBAL_AVGPOOL, REEF_OP_GLOBAL_AVGPOOL},
        {REEF_K_ELTWISE, REEF_OP_ELTWISE}, {REEF_K_DENSE, REEF_OP_DENSE},
        {REEF_K_SOFTMAX, REEF_OP_SOFTMAX}, {REEF_K_LAYERNORM, REEF_OP_LAYERNORM},
        {REEF_K_BIAS_GELU, REEF_OP_BIAS_GELU}, {REEF_K_EMBEDDING, REEF_OP_EMBEDDING},
        {REEF_K_COPY, REEF_OP_COPY}, {REEF_K_TRANSPOSE, REEF_OP_TRANSPOSE},
        {REEF_K_MOCK_ADD, REEF_OP_MOCK_ADD}, {REEF_K_MOCK_MULTIPLY, REEF_OP_MOCK_MULTIPLY},
        {REEF_K_ATTENTION, REEF_OP_ATTENTION},
    };
    for (auto& e : table) {
        const size_t len = std::strlen(e.prefix);
        const bool is_prefix = e.prefix[len - 1] == '_';
        if (is_prefix ? n.compare(0, len, e.prefix) == 0 : n == e.prefix) return e.op;
    }
    return REEF_OP_NONE;
}

namespace {

typedef long long i64;

i64 cdiv(i64 a, i64 b) { return (a + b - 1) / b; }

// The kernels divide task, tile and pixel numbers through a float reciprocal with a remainder
// correction (div_small), which is exact for operands below 2^22; and a tensor must stay below
// 1 GiB, the byte offset that stands for "outside" in their buffer loads.
constexpr i64 kDivSmallLimit = 1ll << 22;
constexpr i64 kTensorLimit = 1ll << 30;

// The operands of one launch in pointer-slot order, each with the bytes it needs.
struct Needs {
    struct Slot { const char* role; i64 bytes; };
    std::vector<Slot> slots;
    i64 tasks = -1;  // workgroups the launch must have; -1 = whatever the graph file says
    std::string bad; // non-empty: the attributes contradict themselves
    void f32(const char* role, i64 elements) { slots.push_back({role, 4 * elements}); }
    void raw(const char* role, i64 bytes) { slots.push_back({role, bytes}); }
};

struct Attrs {
    const std::vector<int32_t>& v;
    i64 operator[](int i) const { return (size_t)i < v.size() ? v[(size_t)i] : 0; }
};

bool all_positive(const Attrs& a, std::initializer_list<int> idx) {
    for (int i : idx)
        if (a[i] <= 0) return false;
    return true;
}

void conv2d(const std::string& symbol, const Attrs& a, Needs& n) {
    if (a.v.size() <= (size_t)REEF_CONV_N_TILES) { n.bad = "too few attributes for a convolution"; return; }
    if (!all_positive(a, {REEF_CONV_CIN, REEF_CONV_H, REEF_CONV_W, REEF_CONV_COUT, REEF_CONV_HO, REEF_CONV_WO,
                          REEF_CONV_KH, REEF_CONV_KW, REEF_CONV_SH, REEF_CONV_SW, REEF_CONV_SPLIT_K,
                          REEF_CONV_M_TILES, REEF_CONV_N_TILES}) ||
        a[REEF_CONV_PH] < 0 || a[REEF_CONV_PW] < 0 || a[REEF_CONV_DST_OFF] < 0 || a[REEF_CONV_SYNC_OFF] < 0) {
        n.bad = "a dimension of the convolution is not positive";
        return;
    }
    const i64 cin = a[REEF_CONV_CIN], H = a[REEF_CONV_H], W = a[REEF_CONV_W], M = a[REEF_CONV_COUT];
    const i64 Ho = a[REEF_CONV_HO], Wo = a[REEF_CONV_WO], kh = a[REEF_CONV_KH], kw = a[REEF_CONV_KW];
    // the sizes a convolution gives; behind a fused 3x3 / stride 2 / padding 1 max-pool (sp7) the pooled ones
    i64 want_ho = (H + 2 * a[REEF_CONV_PH] - kh) / a[REEF_CONV_SH] + 1;
    i64 want_wo = (W + 2 * a[REEF_CONV_PW] - kw) / a[REEF_CONV_SW] + 1;
    if (a[REEF_CONV_FLAGS] & REEF_F_POOL_OUTPUT) {
        want_ho = (want_ho + 2 - 3) / 2 + 1;
        want_wo = (want_wo + 2 - 3) / 2 + 1;
    }
    if (Ho != want_ho || Wo != want_wo || H + 2 * a[REEF_CONV_PH] < kh || W + 2 * a[REEF_CONV_PW] < kw) {
        n.bad = "the output size does not follow from input, filter, stride and padding";
        return;
    }
    const i64 N = Ho * Wo, split = a[REEF_CONV_SPLIT_K], flags = a[REEF_CONV_FLAGS], off = a[REEF_CONV_DST_OFF];
    if (N >= kDivSmallLimit || H * W >= kDivSmallLimit ||
        split * a[REEF_CONV_M_TILES] * a[REEF_CONV_N_TILES] >= kDivSmallLimit) {
        n.bad = "an image or the task count is 4 Mi or more (the kernels' index arithmetic is exact below that)";
        return;
    }
    if (4 * cin * H * W >= kTensorLimit || 4 * M * cin * kh * kw >= kTensorLimit || 4 * (off + M * N) >= kTensorLimit) {
        n.bad = "a tensor of the convolution is 1 GiB or more";
        return;
    }
    const bool fused = flags & REEF_F_FUSED_REDUCE;
    // the loader family is part of the symbol: what it was compiled for must be what the layer is
    const i64 K = cin * kh * kw, taps = kh * kw;
    const bool unit = kh == 1 && kw == 1 && a[REEF_CONV_PH] == 0 && a[REEF_CONV_PW] == 0;
    const std::string fam = symbol.substr(std::strlen("reef_conv2d_"));
    const std::string head = fam.substr(0, fam.find('_'));  // "d9", "d9k", "r9k", "pw", a tile for the general family
    if (head.empty()) { n.bad = "not a convolution symbol"; return; }
    i64 mode = REEF_CONV_MODE_GENERAL;
    bool fits = K % 4 == 0, packed = false;
    if (fam.compare(0, 3, "pw_") == 0) {
        mode = REEF_CONV_MODE_POINTWISE;
        fits = unit && a[REEF_CONV_SH] == 1 && a[REEF_CONV_SW] == 1 && N % 4 == 0 && K % 4 == 0;
    } else if (fam.compare(0, 2, "u_") == 0) {
        mode = REEF_CONV_MODE_UNALIGNED;
        fits = true;
    } else if (fam.compare(0, 3, "xdw") == 0) {
        // a 1x1 filter and the depthwise 3x3 filter behind it (padding 1, stride 1: xdw_g<G>, stride 2:
        // xdw2_g2) in one launch; SH = SW carry the depthwise stride
        mode = REEF_CONV_MODE_XDW;
        const i64 G = a[REEF_CONV_TILE] == REEF_TILE_R9G2 ? 2 : a[REEF_CONV_TILE] == REEF_TILE_R9G4 ? 4 : 0;
        const i64 ds = a[REEF_CONV_SH];
        const std::string want = ds == 1 ? std::string("xdw_g") + (char)('0' + G) : std::string("xdw2_g2");
        fits = kh == 1 && kw == 1 && a[REEF_CONV_PH] == 0 && a[REEF_CONV_PW] == 0 && a[REEF_CONV_SW] == ds &&
               (ds == 1 || (ds == 2 && G == 2)) && cin % 8 == 0 && G > 0 && fam == want && split == 1 &&
               flags == (REEF_F_BIAS | REEF_F_DW_OUTPUT) && off == 0 && a[REEF_CONV_M_TILES] == cdiv(M, 16) &&
               a[REEF_CONV_N_TILES] == cdiv(Ho, G) * cdiv(Wo, 14) && a[REEF_CONV_ACT] <= REEF_ACT_RELU6 &&
               a[REEF_CONV_ACT2] <= REEF_ACT_RELU6;
    } else if (fam.compare(0, 4, "sdp_") == 0 || fam.compare(0, 5, "xdp2_") == 0) {
        // a whole block in one launch, every channel in one workgroup: front filter (sdp: the 3x3 / stride 2 /
        // padding 1 stem on at most 3 channels, depthwise stride 1; xdp2: a 1x1 expansion of at most 16
        // channels, SH = SW = 2 the depthwise stride), depthwise 3x3, projection to REEF_CONV_PROJ channels.
        // The kernels move the middle channels in fours, xdp2 also its input channels, and its input
        // columns in pairs.
        mode = REEF_CONV_MODE_BLOCK;
        const bool stem = fam[0] == 's';
        const i64 G = a[REEF_CONV_TILE] == REEF_TILE_R9G1 ? 1 : a[REEF_CONV_TILE] == REEF_TILE_R9G2 ? 2
                    : a[REEF_CONV_TILE] == REEF_TILE_R9G4 ? 4 : 0;
        const std::string want = std::string(stem ? "sdp_g" : "xdp2_g") + (char)('0' + G);
        const bool front = stem ? kh == 3 && kw == 3 && a[REEF_CONV_PH] == 1 && a[REEF_CONV_PW] == 1 && cin <= 3 &&
                                      M <= 32 && (G == 2 || G == 4)
                                : kh == 1 && kw == 1 && a[REEF_CONV_PH] == 0 && a[REEF_CONV_PW] == 0 && cin <= 16 &&
                                      cin % 4 == 0 && W % 2 == 0 && M <= 96 && (G == 1 || G == 2);
        fits = front && M % 4 == 0 && a[REEF_CONV_SH] == 2 && a[REEF_CONV_SW] == 2 && fam == want && split == 1 && off == 0 &&
               flags == (REEF_F_BIAS | REEF_F_DW_OUTPUT | REEF_F_PROJ_OUTPUT) && a[REEF_CONV_PROJ] >= 1 &&
               a[REEF_CONV_PROJ] <= 32 && a[REEF_CONV_M_TILES] == 1 &&
               a[REEF_CONV_N_TILES] == cdiv(Ho, G) * cdiv(Wo, 14) && a[REEF_CONV_ACT] <= REEF_ACT_RELU6 &&
               a[REEF_CONV_ACT2] <= REEF_ACT_RELU6;
    } else if (fam == "sp7_g2") {
        // 7x7 / stride 2 / padding 3 convolution of at most 3 channels and the 3x3 / stride 2 / padding 1
        // max-pool behind it in one launch; HO, WO are the pooled sizes
        mode = REEF_CONV_MODE_SP7;
        fits = kh == 7 && kw == 7 && a[REEF_CONV_SH] == 2 && a[REEF_CONV_SW] == 2 && a[REEF_CONV_PH] == 3 &&
               a[REEF_CONV_PW] == 3 && cin <= 3 && split == 1 && off == 0 && (flags & REEF_F_BIAS) &&
               (flags & REEF_F_POOL_OUTPUT) &&
               (flags & ~(i64)(REEF_F_BIAS | REEF_F_POOL_OUTPUT | REEF_F_IN_SHIFT | REEF_F_POOL_SHIFT)) == 0 &&
               a[REEF_CONV_TILE] == REEF_TILE_R9G2 && a[REEF_CONV_M_TILES] == cdiv(M, 16) &&
               a[REEF_CONV_N_TILES] == cdiv(Ho, 2) * cdiv(Wo, 14) && a[REEF_CONV_ACT] <= REEF_ACT_RELU6 &&
               a[REEF_CONV_ACT2] <= REEF_ACT_RELU6;
    } else if (fam.compare(0, 3, "p1_") == 0) {
        mode = REEF_CONV_MODE_DIRECT_PRE;
        fits = unit && cin % 8 == 0 && (flags & REEF_F_PRE_ACT);
    } else if (fam.compare(0, 2, "r9") == 0) {
        mode = REEF_CONV_MODE_ROWS;
        packed = head.back() == 'k';
        fits = kh == 3 && kw == 3 && a[REEF_CONV_SH] == 1 && a[REEF_CONV_SW] == 1 && a[REEF_CONV_PH] == 1 &&
               a[REEF_CONV_PW] == 1;
    } else if (fam[0] == 'd') {
        mode = REEF_CONV_MODE_DIRECT;
        const i64 compiled = std::atoi(fam.c_str() + 1);
        packed = head.back() == 'k';
        fits = compiled == taps && (taps > 1 || cin % 8 == 0);
    }
    if (!fits || mode != a[REEF_CONV_MODE] || ((flags & REEF_F_PRE_ACT) != 0) != (mode == REEF_CONV_MODE_DIRECT_PRE) ||
        ((flags & REEF_F_DW_OUTPUT) != 0) != (mode == REEF_CONV_MODE_XDW || mode == REEF_CONV_MODE_BLOCK) ||
        ((flags & REEF_F_PROJ_OUTPUT) != 0) != (mode == REEF_CONV_MODE_BLOCK) ||
        ((flags & REEF_F_POOL_OUTPUT) != 0) != (mode == REEF_CONV_MODE_SP7) ||
        ((flags & (REEF_F_IN_SHIFT | REEF_F_POOL_SHIFT)) != 0 && mode != REEF_CONV_MODE_SP7)) {
        n.bad = "the layer is not one that this symbol's loader family was compiled for";
        return;
    }
    if (packed != (a[REEF_CONV_WPACK] != 0)) { n.bad = "packed weights and symbol do not go together"; return; }
    if (a[REEF_CONV_K_CHUNK] <= 0 || split * a[REEF_CONV_K_CHUNK] < K) {
        n.bad = "the splits do not cover the reduction";
        return;
    }
    n.f32("input", cin * H * W);
    n.f32("weights", M * cin * kh * kw);
    if (flags & REEF_F_GAP_OUTPUT) {
        if (mode != REEF_CONV_MODE_DIRECT || split != 1 || a[REEF_CONV_N_TILES] != 1 || off != 0 || (flags & REEF_F_DUAL)) {
            n.bad = "the averaged output needs a direct kernel, no split, one pixel tile and a single output";
            return;
        }
        n.f32("averaged output", M);
    } else if (split > 1 && !fused) n.f32("partial sums", split * M * N);
    else if (mode == REEF_CONV_MODE_BLOCK) n.f32("output", a[REEF_CONV_PROJ] * N);
    else n.f32("output", off + M * N);
    if (flags & REEF_F_BIAS) n.f32("bias", M);
    if (flags & REEF_F_RESIDUAL) n.f32("residual", M * N);
    if (flags & REEF_F_AFFINE) { n.f32("scale", M); n.f32("shift", M); }
    if (flags & REEF_F_DUAL) { n.f32("second output", off + M * N); n.f32("second shift", M); }
    if (flags & REEF_F_PRE_ACT) { n.f32("input scale", cin); n.f32("input shift", cin); }
    if (flags & REEF_F_DW_OUTPUT) { n.f32("depthwise weights", M * 9); n.f32("depthwise bias", M); }
    if (flags & REEF_F_PROJ_OUTPUT) { n.f32("projection weights", a[REEF_CONV_PROJ] * M); n.f32("projection bias", a[REEF_CONV_PROJ]); }
    if (flags & REEF_F_IN_SHIFT) n.f32("input shift", cin);
    if (flags & REEF_F_POOL_SHIFT) n.f32("pool shift", M);
    if (fused) {
        n.f32("partial sums", (split + ((flags & REEF_F_PAIR_FOLD) ? 1 : 0)) * M * N);
        n.raw("tile counters", 4 * (a[REEF_CONV_SYNC_OFF] + a[REEF_CONV_M_TILES] * a[REEF_CONV_N_TILES]));
    }
    if (a[REEF_CONV_WPACK] != 0) {
        if (a[REEF_CONV_WPACK] != (i64)n.slots.size()) { n.bad = "the packed weights are not the last operand"; return; }
        n.f32("packed weights", cdiv(M, 16) * cdiv(cin, 4) * cdiv(kh * kw, 4) * 4 * 16 * 4);
    }
    n.tasks = split * a[REEF_CONV_M_TILES] * a[REEF_CONV_N_TILES];
}

void splitk_reduce(const Attrs& a, Needs& n) {
    if (!all_positive(a, {REEF_RED_M, REEF_RED_N, REEF_RED_SPLIT_K}) || a[REEF_RED_DST_OFF] < 0) {
        n.bad = "a dimension of the reduction is not positive";
        return;
    }
    const i64 M = a[REEF_RED_M], MN = M * a[REEF_RED_N], flags = a[REEF_RED_FLAGS], off = a[REEF_RED_DST_OFF];
    n.f32("partial sums", a[REEF_RED_SPLIT_K] * MN);
    n.f32("output", off + MN);
    if (flags & REEF_F_BIAS) n.f32("bias", M);
    if (flags & REEF_F_RESIDUAL) n.f32("residual", MN);
    if (flags & REEF_F_AFFINE) { n.f32("scale", M); n.f32("shift", M); }
    if (flags & REEF_F_DUAL) { n.f32("second output", off + MN); n.f32("second shift", M); }
    n.tasks = cdiv(MN, 1024);
}

void gemm(const std::string& symbol, const Attrs& a, Needs& n) {
    if (a.v.size() <= (size_t)REEF_GEMM_STRIDE_C) { n.bad = "too few attributes for a matrix product"; return; }
    if (!all_positive(a, {REEF_GEMM_BATCH, REEF_GEMM_M, REEF_GEMM_N, REEF_GEMM_K, REEF_GEMM_M_TILES,
                          REEF_GEMM_N_TILES, REEF_GEMM_LDA, REEF_GEMM_LDB, REEF_GEMM_LDC})) {
        n.bad = "a dimension of the matrix product is not positive";
        return;
    }
    for (int i : {REEF_GEMM_STRIDE_A, REEF_GEMM_STRIDE_B, REEF_GEMM_STRIDE_C, REEF_GEMM_OFF_A, REEF_GEMM_OFF_B,
                  REEF_GEMM_OFF_C})
        if (a[i] < 0) { n.bad = "a stride or an offset of the matrix product is negative"; return; }
    const i64 b1 = a[REEF_GEMM_BATCH] - 1, M = a[REEF_GEMM_M], N = a[REEF_GEMM_N], K = a[REEF_GEMM_K];
    const bool trans_b = a[REEF_GEMM_TRANS_B] != 0;
    if ((K | a[REEF_GEMM_LDA] | a[REEF_GEMM_STRIDE_A] | a[REEF_GEMM_OFF_A] | a[REEF_GEMM_OFF_B] | a[REEF_GEMM_OFF_C]) & 3 ||
        (trans_b && ((a[REEF_GEMM_LDB] | a[REEF_GEMM_STRIDE_B]) & 3))) {
        n.bad = "K, a leading dimension, a stride or an offset is not a multiple of 4 (128-bit loads)";
        return;
    }
    n.f32("A", a[REEF_GEMM_OFF_A] + b1 * a[REEF_GEMM_STRIDE_A] + (M - 1) * a[REEF_GEMM_LDA] + K);
    if (trans_b) n.f32("B", a[REEF_GEMM_OFF_B] + b1 * a[REEF_GEMM_STRIDE_B] + (N - 1) * a[REEF_GEMM_LDB] + K);
    else n.f32("B", a[REEF_GEMM_OFF_B] + b1 * a[REEF_GEMM_STRIDE_B] + (K - 1) * a[REEF_GEMM_LDB] + N);
    n.f32("C", a[REEF_GEMM_OFF_C] + b1 * a[REEF_GEMM_STRIDE_C] + (M - 1) * a[REEF_GEMM_LDC] + N);
    const i64 fl = a[REEF_GEMM_FLAGS];
    const i64 c_elems = a[REEF_GEMM_OFF_C] + b1 * a[REEF_GEMM_STRIDE_C] + (M - 1) * a[REEF_GEMM_LDC] + N;
    if (fl & REEF_GEMM_F_BIAS) n.f32("bias", N);
    if (fl & REEF_GEMM_F_RES) n.f32("residual", c_elems);
    // A read through a LayerNorm of its rows: only the kernels named ntl do that, and they do nothing else
    const bool ln_kernel = symbol.compare(0, 14, "reef_gemm_ntl_") == 0;
    if (ln_kernel != ((fl & REEF_GEMM_F_LN) != 0)) { n.bad = "the LayerNorm flag and the kernel's name contradict each other"; return; }
    if (!ln_kernel && (fl & REEF_GEMM_F_LN_OUT)) { n.bad = "LayerNorm operands on a plain matrix product"; return; }
    if (ln_kernel) {
        if (!trans_b || b1 != 0 || a[REEF_GEMM_OFF_A] != 0) { n.bad = "the LayerNorm form takes one K-contiguous B and A without offset"; return; }
        if (a.v.size() <= (size_t)REEF_GEMM_LN_EPS_BITS) { n.bad = "the LayerNorm form needs its epsilon"; return; }
        // the kernel numbers the float4s of a row block (at most 128 rows) and divides those numbers
        if (K > (1 << 16)) { n.bad = "the LayerNorm form takes rows of at most 65536 columns"; return; }
        n.f32("column sums of the scaled weights", N);
        n.f32("weights times beta", N);
        n.f32("gamma", K);
        n.f32("beta", K);
        if (fl & REEF_GEMM_F_LN_OUT) n.f32("normalised A", (M - 1) * a[REEF_GEMM_LDA] + K);
    }
    n.tasks = a[REEF_GEMM_BATCH] * a[REEF_GEMM_M_TILES] * a[REEF_GEMM_N_TILES];
    // K split across workgroups, folded inside the launch: the direct kernels only
    const i64 split = a[REEF_GEMM_SPLIT_K];
    if (split < 0 || split == 1) { n.bad = "a split of K is 0 (none) or at least 2"; return; }
    if ((fl & REEF_GEMM_F_PAIR_FOLD) && split != 2) { n.bad = "the pair fold is for a split of two"; return; }
    if (split > 1) {
        const i64 chunk = a[REEF_GEMM_K_CHUNK];
        if (symbol.compare(0, 14, "reef_gemm_ntd_") != 0 || b1 != 0) { n.bad = "only the direct kernels split K, and only without a batch"; return; }
        if (chunk <= 0 || chunk % 128 != 0 || chunk * split < K || chunk * (split - 1) >= K) {
            n.bad = "the K chunks are not multiples of 128 that cover K without an empty one";
            return;
        }
        if (a[REEF_GEMM_SYNC_OFF] < 0) { n.bad = "negative counter offset"; return; }
        n.f32("split-K workspace", (split + ((fl & REEF_GEMM_F_PAIR_FOLD) ? 1 : 0)) * M * N);
        n.raw("arrival counters", 4 * (a[REEF_GEMM_SYNC_OFF] + a[REEF_GEMM_M_TILES] * a[REEF_GEMM_N_TILES]));
        n.tasks *= split;
    }
    if (n.tasks >= kDivSmallLimit) n.bad = "4 Mi workgroups or more (the kernels' index arithmetic is exact below that)";
}

void attention(const Attrs& a, Needs& n) {
    if (!all_positive(a, {REEF_AT_SEQ, REEF_AT_HEAD_DIM, REEF_AT_HEADS, REEF_AT_LD, REEF_AT_LDO}) ||
        a[REEF_AT_OFF_Q] < 0 || a[REEF_AT_OFF_K] < 0 || a[REEF_AT_OFF_V] < 0) {
        n.bad = "a dimension of the attention is not positive";
        return;
    }
    if (a[REEF_AT_SEQ] > REEF_AT_MAX_SEQ || a[REEF_AT_HEAD_DIM] > REEF_AT_MAX_HEAD_DIM) {
        n.bad = "the sequence or the head is larger than the kernel's staging area";
        return;
    }
    if ((a[REEF_AT_HEAD_DIM] | a[REEF_AT_LD] | a[REEF_AT_LDO] | a[REEF_AT_OFF_Q] | a[REEF_AT_OFF_K] | a[REEF_AT_OFF_V]) & 3) {
        n.bad = "head size, a leading dimension or an offset is not a multiple of 4 (128-bit loads)";
        return;
    }
    const i64 seq = a[REEF_AT_SEQ], width = a[REEF_AT_HEADS] * a[REEF_AT_HEAD_DIM];
    i64 last = a[REEF_AT_OFF_Q];
    if (a[REEF_AT_OFF_K] > last) last = a[REEF_AT_OFF_K];
    if (a[REEF_AT_OFF_V] > last) last = a[REEF_AT_OFF_V];
    n.f32("queries, keys and values", last + (seq - 1) * a[REEF_AT_LD] + width);
    n.f32("context", (seq - 1) * a[REEF_AT_LDO] + width);
    if (a[REEF_AT_FLAGS] & 1) n.raw("mask", seq);
    n.tasks = a[REEF_AT_HEADS] * cdiv(seq, REEF_AT_ROWS);
}

// Fills `n` for the ops that are a few lines each; false for an op that is not judged.
bool small_op(int op, const Attrs& a, i64 grid, Needs& n) {
    switch (op) {
    case REEF_OP_DWCONV2D: {
        if (!all_positive(a, {REEF_DW_C, REEF_DW_H, REEF_DW_W, REEF_DW_HO, REEF_DW_WO, REEF_DW_KH, REEF_DW_KW,
                              REEF_DW_SH, REEF_DW_SW}) || a[REEF_DW_PH] < 0 || a[REEF_DW_PW] < 0 ||
            a[REEF_DW_HO] != (a[REEF_DW_H] + 2 * a[REEF_DW_PH] - a[REEF_DW_KH]) / a[REEF_DW_SH] + 1 ||
            a[REEF_DW_WO] != (a[REEF_DW_W] + 2 * a[REEF_DW_PW] - a[REEF_DW_KW]) / a[REEF_DW_SW] + 1) {
            n.bad = "the sizes of the depthwise convolution do not fit each other";
            return true;
        }
        const i64 C = a[REEF_DW_C], out = C * a[REEF_DW_HO] * a[REEF_DW_WO];
        if (a[REEF_DW_HO] * a[REEF_DW_WO] >= kDivSmallLimit || 4 * C * a[REEF_DW_H] * a[REEF_DW_W] >= kTensorLimit) {
            n.bad = "an image of 4 Mi pixels or a tensor of 1 GiB or more";
            return true;
        }
        n.f32("input", C * a[REEF_DW_H] * a[REEF_DW_W]);
        n.f32("weights", C * a[REEF_DW_KH] * a[REEF_DW_KW]);
        n.f32("output", out);
        if (a[REEF_DW_FLAGS] & 1) n.f32("bias", C);
        n.tasks = cdiv(out, 256);
        return true;
    }
    case REEF_OP_POOL2D: {
        if (!all_positive(a, {REEF_POOL_C, REEF_POOL_H, REEF_POOL_W, REEF_POOL_HO, REEF_POOL_WO, REEF_POOL_KH,
                              REEF_POOL_KW, REEF_POOL_SH, REEF_POOL_SW}) || a[REEF_POOL_PH] < 0 || a[REEF_POOL_PW] < 0) {
            n.bad = "a dimension of the pooling is not positive";
            return true;
        }
        const i64 C = a[REEF_POOL_C], out = C * a[REEF_POOL_HO] * a[REEF_POOL_WO];
        if (a[REEF_POOL_HO] * a[REEF_POOL_WO] >= kDivSmallLimit || 4 * C * a[REEF_POOL_H] * a[REEF_POOL_W] >= kTensorLimit) {
            n.bad = "an image of 4 Mi pixels or a tensor of 1 GiB or more";
            return true;
        }
        n.f32("input", C * a[REEF_POOL_H] * a[REEF_POOL_W]);
        n.f32("output", out);
        if (a[REEF_POOL_FLAGS] & 1) n.f32("bias", C);
        if (a[REEF_POOL_FLAGS] & REEF_POOL_F_PRE) { n.f32("input scale", C); n.f32("input shift", C); }
        n.tasks = cdiv(out, 256);
        return true;
    }
    case REEF_OP_GLOBAL_AVGPOOL:
        if (!all_positive(a, {REEF_GAP_C, REEF_GAP_HW})) { n.bad = "a dimension of the pooling is not positive"; return true; }
        n.f32("input", a[REEF_GAP_C] * a[REEF_GAP_HW]);
        n.f32("output", a[REEF_GAP_C]);
        if (a[REEF_GAP_FLAGS] & REEF_GAP_F_PRE) { n.f32("input scale", a[REEF_GAP_C]); n.f32("input shift", a[REEF_GAP_C]); }
        n.tasks = cdiv(a[REEF_GAP_C], 4);
        return true;
    case REEF_OP_ELTWISE: {
        if (!all_positive(a, {REEF_ELT_C, REEF_ELT_INNER})) { n.bad = "a dimension is not positive"; return true; }
        const i64 C = a[REEF_ELT_C], total = C * a[REEF_ELT_INNER];
        n.f32("input", total);
        n.f32("output", total);
        if (a[REEF_ELT_FLAGS] & REEF_ELT_F_B) n.f32("second input", total);
        if (a[REEF_ELT_FLAGS] & REEF_ELT_F_SCALE) n.f32("scale", C);
        if (a[REEF_ELT_FLAGS] & REEF_ELT_F_SHIFT) n.f32("shift", C);
        n.tasks = cdiv(total, 1024);
        return true;
    }
    case REEF_OP_DENSE:
        if (!all_positive(a, {REEF_DENSE_ROWS, REEF_DENSE_IN, REEF_DENSE_OUT})) { n.bad = "a dimension is not positive"; return true; }
        n.f32("input", a[REEF_DENSE_ROWS] * a[REEF_DENSE_IN]);
        n.f32("weights", a[REEF_DENSE_OUT] * a[REEF_DENSE_IN]);
        n.f32("output", a[REEF_DENSE_ROWS] * a[REEF_DENSE_OUT]);
        if (a[REEF_DENSE_FLAGS] & 1) n.f32("bias", a[REEF_DENSE_OUT]);
        n.tasks = cdiv(a[REEF_DENSE_OUT], 4);
        return true;
    case REEF_OP_SOFTMAX:
        if (!all_positive(a, {REEF_SM_ROWS, REEF_SM_COLS})) { n.bad = "a dimension is not positive"; return true; }
        n.f32("input", a[REEF_SM_ROWS] * a[REEF_SM_COLS]);
        n.f32("output", a[REEF_SM_ROWS] * a[REEF_SM_COLS]);
        if (a[REEF_SM_FLAGS] & 1) n.raw("mask", a[REEF_SM_COLS]);
        n.tasks = cdiv(a[REEF_SM_ROWS], 4);
        return true;
    case REEF_OP_LAYERNORM: {
        if (!all_positive(a, {REEF_LN_ROWS, REEF_LN_COLS})) { n.bad = "a dimension is not positive"; return true; }
        const i64 total = a[REEF_LN_ROWS] * a[REEF_LN_COLS];
        n.f32("input", total);
        n.f32("gamma", a[REEF_LN_COLS]);
        n.f32("beta", a[REEF_LN_COLS]);
        n.f32("output", total);
        if (a[REEF_LN_FLAGS] & 1) n.f32("residual", total);
        n.tasks = cdiv(a[REEF_LN_ROWS], 4);
        return true;
    }
    case REEF_OP_BIAS_GELU: {
        if (!all_positive(a, {REEF_GELU_ROWS, REEF_GELU_COLS})) { n.bad = "a dimension is not positive"; return true; }
        const i64 total = a[REEF_GELU_ROWS] * a[REEF_GELU_COLS];
        n.f32("input", total);
        n.f32("output", total);
        if (a[REEF_GELU_FLAGS] & 1) n.f32("bias", a[REEF_GELU_COLS]);
        n.tasks = cdiv(total, 1024);
        return true;
    }
    case REEF_OP_EMBEDDING: {
        if (!all_positive(a, {REEF_EMB_SEQ, REEF_EMB_HIDDEN, REEF_EMB_VOCAB})) { n.bad = "a dimension is not positive"; return true; }
        const i64 total = a[REEF_EMB_SEQ] * a[REEF_EMB_HIDDEN];
        n.raw("token ids", 8 * a[REEF_EMB_SEQ]);
        n.f32("token table", a[REEF_EMB_VOCAB] * a[REEF_EMB_HIDDEN]);
        n.f32("output", total);
        if (a[REEF_EMB_FLAGS] & 1) n.f32("position table", total);
        if (a[REEF_EMB_FLAGS] & 2) n.f32("segment row", a[REEF_EMB_HIDDEN]);
        n.tasks = cdiv(total, 1024);
        return true;
    }
    case REEF_OP_COPY:
        if (a[REEF_COPY_COUNT] <= 0 || a[REEF_COPY_DST_OFF] < 0) { n.bad = "count or offset of the copy is out of range"; return true; }
        n.f32("input", a[REEF_COPY_COUNT]);
        n.f32("output", a[REEF_COPY_DST_OFF] + a[REEF_COPY_COUNT]);
        n.tasks = cdiv(a[REEF_COPY_COUNT], 1024);
        return true;
    case REEF_OP_TRANSPOSE: {
        if (!all_positive(a, {REEF_TR_D0, REEF_TR_D1, REEF_TR_D2})) { n.bad = "a dimension is not positive"; return true; }
        const i64 total = a[REEF_TR_D0] * a[REEF_TR_D1] * a[REEF_TR_D2];
        if (a[REEF_TR_D0] * a[REEF_TR_D1] >= kDivSmallLimit) { n.bad = "4 Mi rows or more"; return true; }
        n.f32("input", total);
        n.f32("output", total);
        if (a[REEF_TR_FLAGS] & 1) n.f32("bias", a[REEF_TR_D1] * a[REEF_TR_D2]);
        n.tasks = cdiv(total, 1024);
        return true;
    }
    case REEF_OP_MOCK_ADD:
    case REEF_OP_MOCK_MULTIPLY:
        // out[task * 128 + t] = a[t] (+|*) b[task * 128 + t]  (resource/mocked_kernel/mocked_kernel.cu:9-27)
        n.f32("a", 128);
        n.f32("b", grid * 128);
        n.f32("out", grid * 128);
        return true;
    default:
        return false;
    }
}

}  // namespace

bool kernel_fits_storages(const Model& m, size_t index, std::string* why) {
    const KernelInfo& ki = m.kernels[index];
    const std::string symbol = ki.name.substr(0, ki.name.find('#'));
    const int op = op_from_symbol(symbol);
    if (op == REEF_OP_NONE) return true;
    const Attrs a{ki.attrs};
    const i64 grid = (i64)ki.launch_params[0] * ki.launch_params[1] * ki.launch_params[2];
    Needs n;
    switch (op) {
    case REEF_OP_CONV2D: conv2d(symbol, a, n); break;
    case REEF_OP_SPLITK_REDUCE: splitk_reduce(a, n); break;
    case REEF_OP_GEMM: gemm(symbol, a, n); break;
    case REEF_OP_ATTENTION: attention(a, n); break;
    default:
        if (!small_op(op, a, grid, n)) return true;
    }
    char buf[512];
    auto fail = [&](const char* msg) {
        if (why) *why = "kernel " + std::to_string(index) + " (" + ki.name + "): " + msg;
        return false;
    };
    if (!n.bad.empty()) return fail(n.bad.c_str());
    if (n.slots.size() != ki.args.size()) {
        std::snprintf(buf, sizeof buf, "its attributes ask for %zu operands, the graph file lists %zu", n.slots.size(),
                      ki.args.size());
        return fail(buf);
    }
    if (n.tasks >= 0 && grid != n.tasks) {
        std::snprintf(buf, sizeof buf, "its attributes ask for %lld workgroups, the graph file launches %lld", n.tasks, grid);
        return fail(buf);
    }
    for (size_t j = 0; j < n.slots.size(); ++j) {
        if (ki.args[j] >= m.storage.size()) return fail("an operand names a storage that does not exist");
        const StorageInfo& s = m.storage[ki.args[j]];
        const i64 have = (i64)(s.size * Model::get_stype_size(s.stype)) - (i64)(ki.arg_offsets.empty() ? 0 : ki.arg_offsets[j]);
        if (n.slots[j].bytes > have) {
            std::snprintf(buf, sizeof buf, "operand %zu (%s) needs %lld bytes, storage %zu (%s) has %lld behind the operand's start",
                          j, n.slots[j].role, n.slots[j].bytes, ki.args[j], s.name.c_str(), have);
            return fail(buf);
        }
    }
    return true;
}

}  // namespace executor
}  // namespace reef
