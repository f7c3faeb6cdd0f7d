/*
 * Device-side boundary of the MI355X REEF build: what a model's code objects
 * (<model>.raw.co, <model>.be.co, <model>.trans.co) export and how the host
 * launches them.  Plain C, shared by the HIP kernels, the C++ executor and the
 * Python model generator (which mirrors the attribute slots below).
 *
 * The reference resolves every graph-JSON `kernels[i].name` with
 * hipModuleGetFunction and binds `kernels[i].args` (storage indices)
 * positionally to the kernel's pointer parameters
 * (src/reef/executor/executor_base.cpp:46-75, 211-223).  Its kernels are TVM
 * output with shapes baked in, one symbol per layer instance.  Here the
 * kernels are hand-written and shape-generic, so one symbol serves every layer
 * of a family and the per-layer shape travels with the launch:
 *
 *   kernels[i].name           entry symbol (REEF_K_* below)
 *   kernels[i].launch_params  [tasks,1,1, 256,1,1]   (logical workgroups x threads)
 *   kernels[i].args           storage indices  -> ReefOpDesc.ptr[j], in order
 *   kernels[i].attrs          int list         -> ReefOpDesc.attr[j], in order
 *                              (added key; the reference parser ignores keys it
 *                               does not look up, src/reef/executor/model.cpp:23-51)
 *
 * Three flavours of every entry, one per code object, as in the reference's
 * model directories (src/reef/server/scheduler.cpp:62-65, src/reef/test/test.cpp:15-22):
 *
 *   raw    K(ReefOpDesc d)
 *          grid = launch_params; replaces the plain TVM kernels.
 *   be     K(ReefBeArgs a)  =  (completion record, int* preempted, int* task_slot, ReefOpDesc d)
 *          replaces script/best_effort_kernel.py:22-29: a workgroup leaves at
 *          once when *preempted != 0, re-polls the flag inside its main loop,
 *          and thread 0 adds 1 to *task_slot only when the workgroup completed.
 *          The completion record (reef_hal.h) lets the launch-window stream the
 *          kernel runs on see it finish without a second device operation: every
 *          workgroup counts itself out as it leaves, preempted or not.
 *   trans  K(ReefDkpArgs a)   and   merge_framework_<n>(ReefDkpArgs a)
 *          replaces the 11-argument dynamic-kernel-padding entry and the
 *          merge_framework_* proxies (script/transform_kernel.py:345-352,
 *          689-718; script/generate_asm_loop.py:189-321): one launch hosts a
 *          real-time side and a best-effort side, each walking its own task
 *          range with a persistent-workgroup loop.
 *
 * Every workgroup has 256 threads (4 wavefronts), 1-D.  A kernel body never
 * reads blockIdx: it receives a logical task index, so any physical workgroup
 * may run any task, which is what makes co-run results bit-identical to solo.
 */
#ifndef REEF_KERNELS_H
#define REEF_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define REEF_WG_THREADS 256
#define REEF_MAX_PTRS 10
#define REEF_MAX_ATTRS 24

typedef struct ReefOpDesc {
    void* ptr[REEF_MAX_PTRS];      /* storages, JSON `args` order */
    int32_t attr[REEF_MAX_ATTRS];  /* JSON `attrs` order */
} ReefOpDesc;

/* Argument block of the best-effort flavour.  The first 32 bytes are the
 * reef_hal_completion of reef_hal.h (all zero: nothing is signalled). */
typedef struct ReefBeArgs {
    uint32_t* done_word;
    uint64_t* exit_ticks;
    uint32_t* exit_count;
    uint32_t seq;
    uint32_t reserved;
    int32_t* preempted;
    int32_t* task_slot;
    ReefOpDesc desc;
} ReefBeArgs;

/* One side of a dynamic-kernel-padding launch
 * (func/layers/task_num/task_offset/param of transform_kernel.py:345-352). */
typedef struct ReefDkpSide {
    int32_t op;           /* REEF_OP_* (replaces the device function pointer) */
    int32_t layers;       /* workgroup layers this side may occupy per virtual CU */
    int32_t task_num;     /* tasks to run in this launch */
    int32_t task_offset;  /* first task */
    ReefOpDesc desc;
} ReefDkpSide;

typedef struct ReefDkpArgs {
    ReefDkpSide l;         /* real-time side  (virtual CUs below the partition) */
    ReefDkpSide r;         /* best-effort side */
    int32_t cu_partition;  /* virtual CUs given to side l, multiple of num_xcds */
    int32_t num_cus;       /* virtual CUs per layer (grid = layers * num_cus) */
    int32_t num_xcds;      /* 8 on MI355X; 1 reproduces the reference's flat mapping */
    int32_t reserved;
    int32_t* task_slot_r;  /* unused, null */
    /* First instruction of each side's own kernel (the reference's func_l / func_r,
     * transform_kernel.py:345-352): read by the merge_framework_<n> proxies only, which jump
     * there; a kernel launched directly ignores them. */
    const void* entry_l;
    const void* entry_r;
} ReefDkpArgs;

/* Op ids for ReefDkpSide.op (order is ABI). */
enum {
    REEF_OP_NONE = 0,
    REEF_OP_CONV2D = 1,
    REEF_OP_SPLITK_REDUCE = 2,
    REEF_OP_DWCONV2D = 3,
    REEF_OP_POOL2D = 4,
    REEF_OP_GLOBAL_AVGPOOL = 5,
    REEF_OP_ELTWISE = 6,
    REEF_OP_DENSE = 7,
    REEF_OP_SOFTMAX = 8,
    REEF_OP_LAYERNORM = 9,
    REEF_OP_BIAS_GELU = 10,
    REEF_OP_EMBEDDING = 11,
    REEF_OP_COPY = 12,
    REEF_OP_TRANSPOSE = 13,
    REEF_OP_GEMM = 14,
    REEF_OP_MOCK_ADD = 15,
    REEF_OP_MOCK_MULTIPLY = 16,
    REEF_OP_ATTENTION = 17,
    REEF_OP_COUNT
};

/* Entry symbols (graph-JSON kernel names). */
#define REEF_K_CONV2D "reef_conv2d"
#define REEF_K_SPLITK_REDUCE "reef_splitk_reduce"
#define REEF_K_DWCONV2D "reef_dwconv2d"
#define REEF_K_POOL2D "reef_pool2d"
#define REEF_K_GLOBAL_AVGPOOL "reef_global_avgpool"
#define REEF_K_ELTWISE "reef_eltwise"
#define REEF_K_DENSE "reef_dense"
#define REEF_K_SOFTMAX "reef_softmax"
#define REEF_K_LAYERNORM "reef_layernorm"
#define REEF_K_BIAS_GELU "reef_bias_gelu"
#define REEF_K_EMBEDDING "reef_embedding"
#define REEF_K_COPY "reef_copy"
#define REEF_K_TRANSPOSE "reef_transpose"
#define REEF_K_GEMM "reef_gemm"
#define REEF_K_ATTENTION "reef_attention"
/* The reference's mocked model (resource/mocked_kernel/mocked_kernel.json)
 * keeps its own names and its (64,1,1)x(4,8,4) launch. */
#define REEF_K_MOCK_ADD "add"
#define REEF_K_MOCK_MULTIPLY "multiply"

/* Activation codes. */
#define REEF_ACT_NONE 0
#define REEF_ACT_RELU 1
#define REEF_ACT_RELU6 2 /* clamp to [0, 6] */
#define REEF_ACT_GELU 3  /* exact erf form, dense/gemm only */

/* ---- reef_conv2d: fp32 implicit-GEMM convolution on MFMA (groups == 1) ----
 * GEMM view: out[M=Cout][N=Ho*Wo] = W[M][K=Cin*kh*kw] x im2col(in)[K][N].
 * ptr: in, W(OIHW), dst, then the optional operands in this order when their
 *      flag bit is set: bias, residual, (scale, shift), (out2, shift2), (workspace, sync).
 * Epilogue: v = acc (+residual) (+bias) (*scale + shift); out = act(v);
 *           with REEF_F_DUAL also out2 = act2(act(v) + shift2[channel]).
 * Split-K (split_k > 1), two forms:
 *   plain : dst is the workspace [split_k][Cout][Ho*Wo]; every split stores its
 *           partial tile and reef_splitk_reduce folds them (the optional operands
 *           then belong to that launch).
 *   REEF_F_FUSED_REDUCE : dst is the output; the workspace holds
 *           [split_k][Cout][Ho*Wo] floats and the sync storage (one per model, named
 *           "reef_sync", int32) holds one counter per output tile starting at
 *           attr SYNC_OFF.  Every split stores its partial, then counts itself on the
 *           tile's counter; the workgroup that arrives last adds the partials in
 *           ascending split order, applies the epilogue and resets the counter.
 *           The sum order is fixed, so the result does not depend on which
 *           workgroup arrives last and equals the plain form bit for bit.
 *           Counters are zero between complete runs of the kernel; after an
 *           interrupted run the host clears the sync storage before the kernel is
 *           run again (HybridExecutor::reset_sync_storage).
 * tasks = split_k * m_tiles * n_tiles;
 * task -> (split = task / (m_tiles*n_tiles), m_tile, n_tile), n fastest. */
enum {
    REEF_CONV_CIN = 0, REEF_CONV_H, REEF_CONV_W, REEF_CONV_COUT, REEF_CONV_HO, REEF_CONV_WO,
    REEF_CONV_KH, REEF_CONV_KW, REEF_CONV_SH, REEF_CONV_SW, REEF_CONV_PH, REEF_CONV_PW,
    REEF_CONV_FLAGS,     /* REEF_F_* */
    REEF_CONV_ACT,       /* REEF_ACT_* */
    REEF_CONV_TILE,      /* REEF_TILE_* */
    REEF_CONV_SPLIT_K,   /* >= 1 */
    REEF_CONV_K_CHUNK,   /* K elements per split, multiple of the tile's BK */
    REEF_CONV_M_TILES, REEF_CONV_N_TILES,
    REEF_CONV_ACT2,      /* activation of the second output (REEF_F_DUAL) */
    REEF_CONV_SYNC_OFF,  /* first counter of this launch inside the sync storage (ints) */
#define REEF_CONV_PROJ REEF_CONV_SYNC_OFF /* REEF_F_PROJ_OUTPUT (a launch without counters): the slot carries the
                                             output channels of the projection behind the depthwise stage */
    REEF_CONV_MODE,      /* REEF_CONV_MODE_*: must match the entry symbol's family */
    REEF_CONV_DST_OFF,   /* element offset added to dst (and out2): channel slice of a concat buffer */
    REEF_CONV_WPACK,     /* pointer slot of the packed copy of the weights (symbols ...d<R>k_ / r9k_), else 0:
                            [ceil(Cout/16)][ceil(Cin/4)][ceil(taps/4)][4 channels][16 rows][4 taps] floats,
                            zero where a row, channel or tap does not exist; the last pointer of the kernel */
    REEF_CONV_NATTR
};
#define REEF_F_BIAS 1
#define REEF_F_RESIDUAL 2
#define REEF_F_AFFINE 4 /* per-channel scale and shift after the sum */
#define REEF_F_DUAL 8   /* second output out2 = act2(out + shift2[channel]) */
#define REEF_F_FUSED_REDUCE 16 /* split-K folded inside the kernel by the last-arriving workgroup */
#define REEF_F_PRE_ACT 32      /* the input is read through relu(in * pre_scale[c] + pre_shift[c]); the two
                                  vectors follow the optional operands (before workspace and counters);
                                  symbols reef_conv2d_p1_<tile>: 1x1 filters, no padding */
#define REEF_F_PAIR_FOLD 64    /* with REEF_F_FUSED_REDUCE and split_k == 2, direct family: the workspace has a third
                                  region of M * N words, zero at rest (the pair slots).  Where every launch on these
                                  buffers runs to completion (plain launches, the real-time side of a padded launch)
                                  the two workgroups of a tile meet there with ONE atomic exchange per output element
                                  instead of partial tile out / count / partial tile in: the first to arrive parks
                                  its value, the second gets it back, adds in split order, finishes the element and
                                  empties the slot.  Best-effort launches, which may be cut short, and the
                                  best-effort side of a padded launch keep the counters. */

#define REEF_F_DW_OUTPUT 128   /* symbols reef_conv2d_xdw_g<G> (G = 2, 4 image rows per tile) and reef_conv2d_xdw2_g2: a 1x1
                                  filter (+ bias, activation ACT) followed by a depthwise 3x3 filter (padding 1, stride
                                  1 resp. 2, + bias, activation ACT2) in one launch; the 1x1 result never leaves the
                                  chip.  ptr: in, W, out, bias, depthwise weights [Cout][9], depthwise bias [Cout].
                                  H, W: the input; HO, WO: the output; SH = SW = the depthwise stride (the 1x1 filter
                                  itself has stride 1).  Spatial tiles as in the row form: G output rows x one
                                  14-column segment; M_TILES = ceil(Cout / 16), N_TILES = ceil(HO / G) * ceil(WO / 14),
                                  TILE = REEF_TILE_R9G2 / R9G4, no split */

/* Loader families of the convolution; the entry symbol carries the family:
 *   reef_conv2d_<tile>      general: im2col gather, needs K % 4 == 0
 *   reef_conv2d_pw_<tile>   pointwise: 1x1, stride 1, no padding, N % 4 == 0, K % 4 == 0
 *   reef_conv2d_u_<tile>    unaligned: im2col gather, any K
 *   reef_conv2d_d<R>_16x<BN>k4  direct: R = kh*kw taps compiled in (1, 3, 7, 9 for BN = 16, 32; 1, 9 for 16x64 and 32x32d4); operands go from memory
 *                           straight into 16x16x4 MFMAs, the four wavefronts split the input
 *                           channels.  d1 needs Cin % 8 == 0 (any stride); K_CHUNK is a multiple
 *                           of R (R > 1) or 8 (d1) and splits K on channel boundaries.
 *   reef_conv2d_r9_g<G>[m2] row form of the direct 3x3 / stride 1 / padding 1 convolution: every input value
 *                           is loaded once per tile and the horizontal taps come from neighbouring lanes. */
#define REEF_F_POOL_OUTPUT 256  /* symbol reef_conv2d_sp7_g2: a 7x7 convolution (stride 2, padding 3, Cin <= 3; + bias,
                                  activation ACT) and the 3x3 max-pool (stride 2, padding 1; + pool shift, activation
                                  ACT2) behind it in one launch.  ptr: in, W, out, bias, then the input shift
                                  (REEF_F_IN_SHIFT) and the pool's shift (REEF_F_POOL_SHIFT).  H, W: the input; HO, WO:
                                  the POOLED output; KH = KW = 7, SH = SW = 2, PH = PW = 3; TILE = REEF_TILE_R9G2;
                                  M_TILES = ceil(Cout / 16), N_TILES = ceil(HO / 2) * ceil(WO / 14); no split. */
#define REEF_F_IN_SHIFT 512    /* with REEF_F_POOL_OUTPUT: the input is read as in + shift[c] inside the image (the
                                  convolution's padding stays 0) */
#define REEF_F_POOL_SHIFT 1024 /* with REEF_F_POOL_OUTPUT: out = act2(maxpool(..) + shift[channel]) */
#define REEF_F_GAP_OUTPUT 2048 /* direct family, 1-tap or multi-tap, no split, N_TILES = 1 (the tile's pixel groups cover
                                  the image): out is [Cout], the global average of what the layer would have written
                                  (bias, residual, scale / shift and activation applied per element first) */
#define REEF_F_PROJ_OUTPUT 4096 /* with REEF_F_DW_OUTPUT, symbols reef_conv2d_sdp_g<G> and reef_conv2d_xdp2_g<G>: a 1x1
                                  projection (+ bias, no activation) behind the depthwise stage in the same launch -- a
                                  whole MobileNetV2 block, for blocks of few channels (COUT = the middle channels <= 32
                                  resp. 96, REEF_CONV_PROJ = P <= 32 output channels; out is [P][HO][WO]).  The front
                                  filter is either the network's 3x3 / stride 2 / padding 1 stem on at most 3 channels
                                  (sdp: KH = KW = 3, SH = SW = 2, PH = PW = 1, depthwise stride 1) or a 1x1 expansion
                                  of at most 16 channels (xdp2: KH = KW = 1, SH = SW = 2 = the depthwise stride; CIN a
                                  multiple of 4, W even).  COUT is a multiple of 4.  ptr:
                                  in, W, out, bias, depthwise weights [COUT][9], depthwise bias [COUT], projection
                                  weights [P][COUT], projection bias [P].  A workgroup holds every channel of its G
                                  output rows x 14 columns: M_TILES = 1, N_TILES = ceil(HO / G) * ceil(WO / 14),
                                  TILE = REEF_TILE_R9G<G>, no split. */
#define REEF_CONV_MODE_GENERAL 0
#define REEF_CONV_MODE_POINTWISE 1
#define REEF_CONV_MODE_UNALIGNED 2
#define REEF_CONV_MODE_DIRECT 3
#define REEF_CONV_MODE_DIRECT_PRE 4   /* direct, 1 tap, with REEF_F_PRE_ACT (reef_conv2d_p1_<tile>) */
#define REEF_CONV_MODE_SP7 7          /* 7x7 stride-2 convolution + 3x3 stride-2 max-pool (reef_conv2d_sp7_g2, REEF_F_POOL_OUTPUT) */
#define REEF_CONV_MODE_XDW 6          /* 1x1 filter + depthwise 3x3 behind it (reef_conv2d_xdw_g<G>, REEF_F_DW_OUTPUT) */
#define REEF_CONV_MODE_BLOCK 8        /* front filter + depthwise 3x3 + 1x1 projection (reef_conv2d_sdp_g<G>, reef_conv2d_xdp2_g<G>,
                                         REEF_F_DW_OUTPUT | REEF_F_PROJ_OUTPUT) */
#define REEF_CONV_MODE_ROWS 5         /* direct, row form: 3x3 / stride 1 / padding 1 (reef_conv2d_r9_g<G>[m2]).
                                         The output tile is 16 (m2: 32) channels x G image rows x one 14-column
                                         segment; N_TILES = ceil(Ho / G) * ceil(Wo / 14), spatial tile index =
                                         row tile * segments + segment.  K_CHUNK a multiple of 144. */

/* Tile configurations: BM x BN output tile per workgroup.  Plain tiles walk K in steps of
 * 32; a "k<n>" tile splits every step of 32*n k values across n wavefronts and sums the n
 * partial tiles inside the workgroup (K_CHUNK is then a multiple of 32*n). */
enum {
    REEF_TILE_128x128 = 0,
    REEF_TILE_128x64 = 1,
    REEF_TILE_64x64 = 2,
    REEF_TILE_128x32 = 3,
    REEF_TILE_32x128 = 4,
    REEF_TILE_64x128 = 5,
    REEF_TILE_32x32k4 = 6,
    REEF_TILE_64x32k2 = 7,
    REEF_TILE_32x64k2 = 8,
    REEF_TILE_16x16k4 = 9,   /* direct family only */
    REEF_TILE_16x32k4 = 10,  /* direct family, 1 and 9 taps */
    REEF_TILE_16x64k4 = 11,  /* direct family, 1 and 9 taps */
    REEF_TILE_32x32d4 = 12,  /* direct family, 1 and 9 taps (symbol suffix 32x32d4) */
    REEF_TILE_R9G1 = 13,     /* row form (REEF_CONV_MODE_ROWS): 16 channels x 1, 2, 4, 7 image rows */
    REEF_TILE_R9G2 = 14,
    REEF_TILE_R9G4 = 15,
    REEF_TILE_R9G7 = 16,
    REEF_TILE_R9G2M2 = 17,   /* 32 channels x 2, 4 image rows */
    REEF_TILE_R9G4M2 = 18,
    REEF_TILE_COUNT
};

/* ---- reef_splitk_reduce: out = act(sum_s ws[s] (+res)(+bias)(*scale+shift)), s ascending ----
 * ptr: ws, out, then optional bias, residual, (scale, shift), (out2, shift2) (same flag order).
 * attr: M, N, split_k, flags, act, act2, dst_off (element offset added to out and out2).   tasks = ceil(M*N / 1024) (4 elements per thread). */
enum { REEF_RED_M = 0, REEF_RED_N, REEF_RED_SPLIT_K, REEF_RED_FLAGS, REEF_RED_ACT, REEF_RED_ACT2,
       REEF_RED_DST_OFF, REEF_RED_NATTR };

/* ---- reef_dwconv2d: depthwise k x k convolution + bias + activation (bandwidth-bound) ----
 * ptr: in, W[C][kh][kw], out, bias(optional by flag).
 * attr: C,H,W,Ho,Wo,kh,kw,sh,sw,ph,pw,flags,act.  tasks = ceil(C*Ho*Wo / 256). */
enum {
    REEF_DW_C = 0, REEF_DW_H, REEF_DW_W, REEF_DW_HO, REEF_DW_WO, REEF_DW_KH, REEF_DW_KW,
    REEF_DW_SH, REEF_DW_SW, REEF_DW_PH, REEF_DW_PW, REEF_DW_FLAGS, REEF_DW_ACT, REEF_DW_NATTR
};

/* ---- reef_pool2d: max / average pooling (+bias +relu) ----
 * ptr: in, out, bias (flags & 1), then pre-scale and pre-shift (flags & REEF_POOL_F_PRE: the input is
 * read as relu(in * scale[c] + shift[c])).  mode 0 max (pads with -FLT_MAX), 1 average.
 * tasks = ceil(C*Ho*Wo / 256). */
#define REEF_POOL_F_PRE 2
enum {
    REEF_POOL_C = 0, REEF_POOL_H, REEF_POOL_W, REEF_POOL_HO, REEF_POOL_WO, REEF_POOL_KH,
    REEF_POOL_KW, REEF_POOL_SH, REEF_POOL_SW, REEF_POOL_PH, REEF_POOL_PW, REEF_POOL_MODE,
    REEF_POOL_COUNT_PAD, REEF_POOL_FLAGS, REEF_POOL_ACT, REEF_POOL_NATTR
};

/* ---- reef_global_avgpool: out[c] = sum(in[c][:]) * (1/HW).  ptr: in, out, then scale and shift
 * (flags & REEF_GAP_F_PRE: the input is read as relu(in * scale[c] + shift[c])).
 * attr: C, HW, flags (absent = 0).  tasks = ceil(C / 4) (one wavefront per channel). */
#define REEF_GAP_F_PRE 1
enum { REEF_GAP_C = 0, REEF_GAP_HW, REEF_GAP_FLAGS, REEF_GAP_NATTR };

/* ---- reef_eltwise: out = act(a (+b) (*scale[c]) (+shift[c])), c = i / inner ----
 * ptr: a, out, then optional b, scale, shift by flag.  attr: C, inner, flags, act.
 * tasks = ceil(C*inner / 1024). */
enum { REEF_ELT_C = 0, REEF_ELT_INNER, REEF_ELT_FLAGS, REEF_ELT_ACT, REEF_ELT_NATTR };
#define REEF_ELT_F_B 1
#define REEF_ELT_F_SCALE 2
#define REEF_ELT_F_SHIFT 4

/* ---- reef_dense: y[r][o] = act(sum_k x[r][k] W[o][k] + b[o]), few rows (GEMV, bandwidth-bound) ----
 * ptr: x, W, y, bias(optional).  attr: rows, in_f, out_f, flags, act.
 * tasks = ceil(out_f / 4) (one wavefront per output neuron). */
enum { REEF_DENSE_ROWS = 0, REEF_DENSE_IN, REEF_DENSE_OUT, REEF_DENSE_FLAGS, REEF_DENSE_ACT, REEF_DENSE_NATTR };

/* ---- reef_softmax: rows x cols, one wavefront per row.  ptr: in, out, mask(optional).
 * attr: rows, cols, flags(bit0 = mask).  tasks = ceil(rows / 4).
 * mask: one byte per column (stype uint1), non-zero = that column counts as -inf in every row:
 * the attention mask the reference applies with a kernel of its own between the scores and the
 * softmax (fused_reshape_cast_broadcast_to_like_where, resource/bert/bert.cu:381-388; the mask
 * itself is resource/bert/bert.json storage[1], zero-filled by fused_full_equal_reshape, :313). */
enum { REEF_SM_ROWS = 0, REEF_SM_COLS, REEF_SM_FLAGS, REEF_SM_NATTR };

/* ---- reef_layernorm: out = LN(x (+res)) * gamma + beta, one wavefront per row ----
 * ptr: x, gamma, beta, out, res(optional).  attr: rows, cols, flags(bit0 = res), eps (float bits).
 * tasks = ceil(rows / 4). */
enum { REEF_LN_ROWS = 0, REEF_LN_COLS, REEF_LN_FLAGS, REEF_LN_EPS_BITS, REEF_LN_NATTR };

/* ---- reef_attention: softmax(alpha Q K^T (masked)) V for every head, one launch ----
 * The three launches of an attention layer (scores, softmax, context: bert.cu:22-271, 3-13,
 * 159-166, 327-337, 381-396) for sequences whose scores fit a workgroup: seq <= 128,
 * head_dim <= 64 and a multiple of 4 (as ld, ldo and the offsets: 128-bit loads).  Q, K and V are column blocks of one [seq][ld] storage
 * (head h at columns off + h * head_dim), the context goes to out[seq][ldo] at columns
 * h * head_dim.  A workgroup takes REEF_AT_ROWS query rows of one head: it holds them, all keys and then
 * all values of the head in LDS, the scores never leave the chip.
 * ptr: qkv, out, mask(optional: one byte per key position, non-zero = -inf).
 * attr: seq, head_dim, heads, ld, ldo, offQ, offK, offV (elements), alpha (float bits), flags
 * (bit0 = mask).  tasks = heads * ceil(seq / REEF_AT_ROWS). */
enum {
    REEF_AT_SEQ = 0, REEF_AT_HEAD_DIM, REEF_AT_HEADS, REEF_AT_LD, REEF_AT_LDO, REEF_AT_OFF_Q,
    REEF_AT_OFF_K, REEF_AT_OFF_V, REEF_AT_ALPHA_BITS, REEF_AT_FLAGS, REEF_AT_NATTR
};
#define REEF_AT_ROWS 8 /* query rows per workgroup: 16 leave too few workgroups, 4 stage the keys and values too often */
#define REEF_AT_MAX_SEQ 128
#define REEF_AT_MAX_HEAD_DIM 64
#define REEF_AT_KV_STRIDE 68 /* floats per staged key / value row: 64 + 4, rows 16-byte aligned */
#define REEF_AT_LDS_BYTES \
    (4 * (REEF_AT_ROWS * REEF_AT_MAX_HEAD_DIM + REEF_AT_MAX_SEQ * REEF_AT_KV_STRIDE + REEF_AT_ROWS * (REEF_AT_MAX_SEQ + 4)))

/* ---- reef_bias_gelu: out = gelu_erf(x + bias[col]).  ptr: x, out, bias(optional).
 * attr: rows, cols, flags.  tasks = ceil(rows*cols / 1024). */
enum { REEF_GELU_ROWS = 0, REEF_GELU_COLS, REEF_GELU_FLAGS, REEF_GELU_NATTR };

/* ---- reef_embedding: out[s][h] = tok[ids[s]][h] (+pos[s][h]) (+seg[h]) ----
 * ptr: ids(int64), tok, out, pos(optional), seg(optional).
 * attr: seq, hidden, flags(bit0 pos, bit1 seg), vocab.  tasks = ceil(seq*hidden/1024). */
enum { REEF_EMB_SEQ = 0, REEF_EMB_HIDDEN, REEF_EMB_FLAGS, REEF_EMB_VOCAB, REEF_EMB_NATTR };

/* ---- reef_copy: out[dst_off + i] = in[i].  ptr: in, out.  attr: count, dst_off.
 * tasks = ceil(count / 1024). */
enum { REEF_COPY_COUNT = 0, REEF_COPY_DST_OFF, REEF_COPY_NATTR };

/* ---- reef_transpose: in [d0][d1][d2] -> out [d1][d0][d2] (+bias over (d1,d2)) ----
 * ptr: in, out, bias(optional).  attr: d0, d1, d2, flags.  tasks = ceil(d0*d1*d2/1024). */
enum { REEF_TR_D0 = 0, REEF_TR_D1, REEF_TR_D2, REEF_TR_FLAGS, REEF_TR_NATTR };

/* ---- reef_gemm_nt_<tile> / reef_gemm_ntd_<tile> / reef_gemm_nn_<tile>: batched fp32 GEMM on MFMA ----
 * nt: trans_b = 1 (K, lda, ldb and the batch strides must be multiples of 4);
 * ntd: trans_b = 1, operands straight from memory into 16x16x4 MFMAs (tiles 16x16k4, 16x32k4,
 *      32x32d4; K a multiple of 8, lda, ldb and the batch strides multiples of 4);
 * nn: trans_b = 0 (K and lda multiples of 4).
 * C[b][m][n] = act(alpha * sum_k A[b][m][k] * B(b,k,n) (+bias[n])) (+R[b][m][n])
 * trans_b = 1: B stored [b][n][k] (dense layers, Q.K^T); 0: [b][k][n] (P.V).
 * R (REEF_GEMM_F_RES): a residual laid out as C is (ldc, offC, strideC), added after the activation.
 * ptr: A, B, C, bias (optional), R (optional).
 * attr: batch, M, N, K, trans_b, flags, act, alpha (float bits), tile, m_tiles, n_tiles,
 *       lda, ldb, ldc, strideA, strideB, strideC (elements), then offA, offB, offC: where the
 *       first matrix starts inside its storage, in elements (absent = 0; multiples of 4 like the
 *       strides) -- several operands can share one storage, e.g. Q, K and V as column blocks of
 *       one [tokens][3 * hidden] projection.
 * tasks = batch * m_tiles * n_tiles.
 *
 * reef_gemm_ntl_<tile> (staged tiles, trans_b = 1, batch 1, flags has REEF_GEMM_F_LN): the product
 * behind a LayerNorm of the rows of A,
 *   A'[m][k] = (A[m][k] - mean[m]) / sqrt(var[m] + eps) * gamma[k] + beta[k]
 * (mean and variance over the K columns of the row), C = act(alpha * A' x W^T (+bias)) (+R), computed
 * as  alpha * (rstd[m] * (sum_k A[m][k] Wg[n][k] - mean[m] c1[n]) + c2[n])  from three tensors derived
 * from the parameters: Wg[n][k] = gamma[k] W[n][k], c1[n] = sum_k Wg[n][k], c2[n] = sum_k beta[k] W[n][k].
 * A and A' are [M][K] with leading dimension lda and no offset; K <= 65536.
 * ptr: A, Wg, C, bias (optional), R (optional), c1, c2, gamma, beta, A' (REEF_GEMM_F_LN_OUT: the
 * normalised rows are written as well, a share by every workgroup of a row block).  The storage
 * of Wg is named <name of W's storage>gk; W itself stays a storage of the model.
 * attr: as above, then eps (float bits). */
#define REEF_GEMM_F_BIAS 1
#define REEF_GEMM_F_LN 2
#define REEF_GEMM_F_LN_OUT 4
#define REEF_GEMM_F_RES 8
#define REEF_GEMM_F_PAIR_FOLD 16
/* K split across workgroups (reef_gemm_ntd_<tile>, batch 1; attrs split_k > 1, k_chunk a multiple
 * of 128): tasks = split_k * m_tiles * n_tiles, the split_k workgroups of a tile neighbours in
 * the task order.  The partial tiles meet inside the launch as those of the direct convolutions
 * do: ptr gets two more operands behind the optional ones, a workspace of split_k regions of
 * M x N floats and the model's arrival counters (sync_off: first counter of this launch, one per
 * output tile); with REEF_GEMM_F_PAIR_FOLD (split_k = 2) the workspace has a third region, the
 * pair slots, zero at rest, and launches that always run to completion exchange through them. */
enum {
    REEF_GEMM_BATCH = 0, REEF_GEMM_M, REEF_GEMM_N, REEF_GEMM_K, REEF_GEMM_TRANS_B,
    REEF_GEMM_FLAGS, REEF_GEMM_ACT, REEF_GEMM_ALPHA_BITS, REEF_GEMM_TILE, REEF_GEMM_M_TILES,
    REEF_GEMM_N_TILES, REEF_GEMM_LDA, REEF_GEMM_LDB, REEF_GEMM_LDC, REEF_GEMM_STRIDE_A,
    REEF_GEMM_STRIDE_B, REEF_GEMM_STRIDE_C, REEF_GEMM_OFF_A, REEF_GEMM_OFF_B, REEF_GEMM_OFF_C,
    REEF_GEMM_NATTR,
    REEF_GEMM_LN_EPS_BITS = REEF_GEMM_NATTR,     /* reef_gemm_ntl_* only */
    REEF_GEMM_SPLIT_K, REEF_GEMM_K_CHUNK, REEF_GEMM_SYNC_OFF      /* absent or 0: no split */
};

/* ---- add / multiply (the reference's mocked model): ptr: a, b, out; no attrs ---- */

#ifdef __cplusplus
}
#endif
#endif /* REEF_KERNELS_H */
