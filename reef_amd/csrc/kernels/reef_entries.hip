// Entry points of the REEF code objects for gfx950.  This one source is
// compiled three times (REEF_FLAVOUR = 0 raw, 1 be, 2 trans) into
// reef_kernels.{raw,be,trans}.co, the three code objects a model directory
// carries (src/reef/server/scheduler.cpp:62-65; raw.co is used by the
// reference's tests only, src/reef/test/test.cpp:19).
//
//   raw    K(ReefOpDesc)                               plain launch, task = blockIdx.x
//   be     K(int* preempted, int* task_slot, ReefOpDesc)
//          script/best_effort_kernel.py:22-29 restated: leave at once when the
//          flag is set, poll it again inside long bodies, count completed
//          workgroups in *task_slot.
//   trans  K(ReefDkpArgs) and merge_framework_<n>(ReefDkpArgs)
//          script/generate_asm_loop.py:227-321 / transform_kernel.py:423-478
//          restated: pick the side from the virtual CU id, then walk that
//          side's task range with a persistent-workgroup loop.  The virtual CU
//          id is two-level on MI355X (xcd = cu % 8, slot = cu / 8) so both
//          sides get the same share of every XCD and of every XCD's L2.
#include "reef_bw_ops.hpp"
#include "reef_mma.hpp"

#ifndef REEF_FLAVOUR
#error "compile with -DREEF_FLAVOUR=0|1|2"
#endif

using namespace reef_dev;

namespace {

// ---- op functors: LDS need + body ------------------------------------------
template <class T, int MODE = CONV_GENERAL>
struct OpConv {
    static constexpr int LDS = T::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_body<T, MODE>(d, task, smem, p);
    }
};
template <int R, int TN = 1, int TM = 1, bool PRE = false>
struct OpConvDirect {
    static constexpr int LDS = TileD16<TN, TM>::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_direct_body<R, TN, TM, PRE>(d, task, smem, p);
    }
};
template <class T, bool TRANS_B>
struct OpGemm {
    static constexpr int LDS = T::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return gemm_body<T, TRANS_B>(d, task, smem, p);
    }
};
template <int TM, int TN>
struct OpGemmNtDirect {
    static constexpr int LDS = TileD16<TN, TM>::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return gemm_nt_direct_body<TM, TN>(d, task, smem, p);
    }
};
#define REEF_SIMPLE_OP(STRUCT, CALL)                                                            \
    struct STRUCT {                                                                             \
        static constexpr int LDS = 0;                                                           \
        template <class P>                                                                      \
        static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char*, const P&) { \
            CALL(d, task);                                                                      \
            return true;                                                                        \
        }                                                                                       \
    };
REEF_SIMPLE_OP(OpSplitKReduce, splitk_reduce_body<8>)
REEF_SIMPLE_OP(OpDwConv, dwconv2d_body)
REEF_SIMPLE_OP(OpPool, pool2d_body)
REEF_SIMPLE_OP(OpGap, global_avgpool_body)
REEF_SIMPLE_OP(OpEltwise, eltwise_body)
REEF_SIMPLE_OP(OpDense, dense_body)
REEF_SIMPLE_OP(OpSoftmax, softmax_body)
REEF_SIMPLE_OP(OpLayerNorm, layernorm_body)
REEF_SIMPLE_OP(OpBiasGelu, bias_gelu_body)
REEF_SIMPLE_OP(OpEmbedding, embedding_body)
REEF_SIMPLE_OP(OpCopy, copy_body)
REEF_SIMPLE_OP(OpTranspose, transpose_body)

// The mocked kernels keep the reference's 128 logical threads per block.
template <bool MUL>
struct OpMocked {
    static constexpr int LDS = 0;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char*, const P&) {
        const int t = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y;
        if (t < 128) mocked_body<MUL>(d, task, t);
        return true;
    }
};

// The launch arguments are read in place from the kernarg segment (constant
// address space, scalar loads).  Going through the by-value parameter instead
// makes the compiler copy the structs to scratch as soon as a side or an
// optional-operand slot is selected at run time.
template <class T>
__device__ __forceinline__ const T& kernarg_at(int byte_offset) {
    const char* base = (const char*)__builtin_amdgcn_kernarg_segment_ptr();
    return *(const T*)(base + byte_offset);
}

#if REEF_FLAVOUR == 2
// Side selection and first task of this workgroup.  Returns false when the
// workgroup has nothing to do.
struct DkpWalk {
    bool right;
    int idx, step, end;
};
__device__ __forceinline__ bool dkp_walk(const ReefDkpArgs& a, DkpWalk& w) {
    const int C = a.num_cus, X = a.num_xcds;
    const int b = blockIdx.x;
    const int layer = b / C, cu = b - layer * C;
    const int xcd = cu % X, slot = cu / X;
    const int rt_slots = a.cu_partition / X;
    int span, cu_idx, layers, task_num, task_offset;
    if (slot < rt_slots) {
        w.right = false;
        span = rt_slots * X;
        cu_idx = slot * X + xcd;
        layers = a.l.layers; task_num = a.l.task_num; task_offset = a.l.task_offset;
    } else {
        w.right = true;
        span = C - rt_slots * X;
        cu_idx = (slot - rt_slots) * X + xcd;
        layers = a.r.layers; task_num = a.r.task_num; task_offset = a.r.task_offset;
    }
    if (layer >= layers) return false;
    w.idx = span * layer + cu_idx + task_offset;
    w.step = layers * span;
    w.end = task_offset + task_num;
    return w.idx < w.end;
}
#endif

}  // namespace

// ---- entry generators ---------------------------------------------------------
#define REEF_COMMA ,
#if REEF_FLAVOUR == 0
#define REEF_ENTRY(NAME, OP)                                                          \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS) NAME(ReefOpDesc) {  \
        __shared__ __align__(16) char smem[OP::LDS > 0 ? OP::LDS : 16];               \
        OP::run(kernarg_at<ReefOpDesc>(0), (int)blockIdx.x, smem, NoPoll{});          \
    }
#elif REEF_FLAVOUR == 1
#define REEF_ENTRY(NAME, OP)                                                              \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS)                         \
    NAME(int* preempted, int* task_slot, ReefOpDesc) {                                    \
        __shared__ __align__(16) char smem[OP::LDS > 0 ? OP::LDS : 16];                   \
        __shared__ int s_pre;                                                             \
        const int t = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y; \
        FlagPoll poll{preempted};                                                         \
        if (t == 0) s_pre = poll.load();                                                  \
        __syncthreads();                                                                  \
        if (s_pre) return;                                                                \
        const bool done = OP::run(kernarg_at<ReefOpDesc>(16), (int)blockIdx.x, smem, poll); \
        if (done && t == 0) atomicAdd(task_slot, 1);                                      \
    }
#else
#define REEF_ENTRY(NAME, OP)                                                           \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS) NAME(ReefDkpArgs) {  \
        __shared__ __align__(16) char smem[OP::LDS > 0 ? OP::LDS : 16];                \
        const ReefDkpArgs& a = kernarg_at<ReefDkpArgs>(0);                             \
        DkpWalk w;                                                                     \
        if (!dkp_walk(a, w)) return;                                                   \
        const ReefDkpSide& side = w.right ? a.r : a.l;                                 \
        for (int i = w.idx; i < w.end; i += w.step) {                                  \
            OP::run(side.desc, i, smem, NoPoll{});                                     \
            __syncthreads();                                                           \
        }                                                                              \
    }
#endif

REEF_ENTRY(reef_conv2d_128x128, OpConv<Tile128x128>)
REEF_ENTRY(reef_conv2d_128x64, OpConv<Tile128x64>)
REEF_ENTRY(reef_conv2d_64x64, OpConv<Tile64x64>)
REEF_ENTRY(reef_conv2d_128x32, OpConv<Tile128x32>)
REEF_ENTRY(reef_conv2d_32x128, OpConv<Tile32x128>)
REEF_ENTRY(reef_conv2d_64x128, OpConv<Tile64x128>)
REEF_ENTRY(reef_conv2d_32x32k4, OpConv<Tile32x32k4>)
REEF_ENTRY(reef_conv2d_64x32k2, OpConv<Tile64x32k2>)
REEF_ENTRY(reef_conv2d_32x64k2, OpConv<Tile32x64k2>)
REEF_ENTRY(reef_conv2d_pw_128x128, OpConv<Tile128x128 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_128x64, OpConv<Tile128x64 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_64x64, OpConv<Tile64x64 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_128x32, OpConv<Tile128x32 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_32x128, OpConv<Tile32x128 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_64x128, OpConv<Tile64x128 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_32x32k4, OpConv<Tile32x32k4 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_64x32k2, OpConv<Tile64x32k2 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_pw_32x64k2, OpConv<Tile32x64k2 REEF_COMMA CONV_POINTWISE>)
REEF_ENTRY(reef_conv2d_u_128x128, OpConv<Tile128x128 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_128x64, OpConv<Tile128x64 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_64x64, OpConv<Tile64x64 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_128x32, OpConv<Tile128x32 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_32x128, OpConv<Tile32x128 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_64x128, OpConv<Tile64x128 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_32x32k4, OpConv<Tile32x32k4 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_64x32k2, OpConv<Tile64x32k2 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_u_32x64k2, OpConv<Tile32x64k2 REEF_COMMA CONV_UNALIGNED>)
REEF_ENTRY(reef_conv2d_d1_16x16k4, OpConvDirect<1>)
REEF_ENTRY(reef_conv2d_d3_16x16k4, OpConvDirect<3>)
REEF_ENTRY(reef_conv2d_d7_16x16k4, OpConvDirect<7>)
REEF_ENTRY(reef_conv2d_d9_16x16k4, OpConvDirect<9>)
REEF_ENTRY(reef_conv2d_d1_16x32k4, OpConvDirect<1 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d9_16x32k4, OpConvDirect<9 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d1_16x64k4, OpConvDirect<1 REEF_COMMA 4>)
REEF_ENTRY(reef_conv2d_d9_16x64k4, OpConvDirect<9 REEF_COMMA 4>)
REEF_ENTRY(reef_conv2d_d3_16x32k4, OpConvDirect<3 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d7_16x32k4, OpConvDirect<7 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_p1_16x16k4, OpConvDirect<1 REEF_COMMA 1 REEF_COMMA 1 REEF_COMMA true>)
REEF_ENTRY(reef_conv2d_p1_16x32k4, OpConvDirect<1 REEF_COMMA 2 REEF_COMMA 1 REEF_COMMA true>)
REEF_ENTRY(reef_conv2d_p1_32x32d4, OpConvDirect<1 REEF_COMMA 2 REEF_COMMA 2 REEF_COMMA true>)
REEF_ENTRY(reef_conv2d_d1_32x32d4, OpConvDirect<1 REEF_COMMA 2 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d9_32x32d4, OpConvDirect<9 REEF_COMMA 2 REEF_COMMA 2>)
REEF_ENTRY(reef_gemm_nt_128x128, OpGemm<Tile128x128 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_64x64, OpGemm<Tile64x64 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_32x128, OpGemm<Tile32x128 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_32x32k4, OpGemm<Tile32x32k4 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_64x32k2, OpGemm<Tile64x32k2 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_ntd_16x16k4, OpGemmNtDirect<1 REEF_COMMA 1>)
REEF_ENTRY(reef_gemm_ntd_16x32k4, OpGemmNtDirect<1 REEF_COMMA 2>)
REEF_ENTRY(reef_gemm_ntd_32x32d4, OpGemmNtDirect<2 REEF_COMMA 2>)
REEF_ENTRY(reef_gemm_nn_128x128, OpGemm<Tile128x128 REEF_COMMA false>)
REEF_ENTRY(reef_gemm_nn_64x64, OpGemm<Tile64x64 REEF_COMMA false>)
REEF_ENTRY(reef_gemm_nn_32x128, OpGemm<Tile32x128 REEF_COMMA false>)
REEF_ENTRY(reef_gemm_nn_32x32k4, OpGemm<Tile32x32k4 REEF_COMMA false>)
REEF_ENTRY(reef_gemm_nn_64x32k2, OpGemm<Tile64x32k2 REEF_COMMA false>)
REEF_ENTRY(reef_splitk_reduce, OpSplitKReduce)
REEF_ENTRY(reef_dwconv2d, OpDwConv)
REEF_ENTRY(reef_pool2d, OpPool)
REEF_ENTRY(reef_global_avgpool, OpGap)
REEF_ENTRY(reef_eltwise, OpEltwise)
REEF_ENTRY(reef_dense, OpDense)
REEF_ENTRY(reef_softmax, OpSoftmax)
REEF_ENTRY(reef_layernorm, OpLayerNorm)
REEF_ENTRY(reef_bias_gelu, OpBiasGelu)
REEF_ENTRY(reef_embedding, OpEmbedding)
REEF_ENTRY(reef_copy, OpCopy)
REEF_ENTRY(reef_transpose, OpTranspose)
REEF_ENTRY(add, OpMocked<false>)
REEF_ENTRY(multiply, OpMocked<true>)

#if REEF_FLAVOUR == 2
// ---- merge_framework_<n>: two different ops in one launch ------------------------
// The reference's proxies jump to a device function pointer per side
// (script/transform_kernel.py:689-718) and exist in ten variants whose register
// budgets are patched to the gfx906 occupancy classes
// (script/replace_register_usage.py:33-59).  Here the side carries an op id and
// the proxy switches into the inlined body; the variants are the gfx950
// occupancy classes that matter for this kernel set, <n> = wavefronts per SIMD:
//   merge_framework_8  bandwidth-bound ops only                          (<= 64 registers)
//   merge_framework_3  + conv (general, pointwise) tiles 64x64 / 128x32,
//                        direct family with 1 and 9 taps, 16x16 and 16x32    (<= 168)
//   merge_framework_2  + conv (general, pointwise) tile 128x64 and the
//                        wave-split-K tiles                                   (<= 256)
// Kernels outside these sets (the other tiles, the unaligned-K convolution, GEMM)
// are never merged: they run single-sided through their own entry.
// LDS is dynamic (the host passes the larger of the two sides' needs, as
// src/reef/server/scheduler.cpp:643-649 does).
namespace {
template <int LEVEL>
__device__ __forceinline__ void run_op(const ReefDkpSide& s, int task, char* smem) {
    const ReefOpDesc& d = s.desc;
    const NoPoll np{};
    switch (s.op) {
        case REEF_OP_CONV2D:
            if (LEVEL >= 1) {
                const int tile = d.attr[REEF_CONV_TILE];
                if (d.attr[REEF_CONV_MODE] == REEF_CONV_MODE_DIRECT) {
                    const int taps = d.attr[REEF_CONV_KH] * d.attr[REEF_CONV_KW];
                    if (tile == REEF_TILE_16x16k4) {
                        if (taps == 1) OpConvDirect<1>::run(d, task, smem, np);
                        else if (taps == 9) OpConvDirect<9>::run(d, task, smem, np);
                    } else if (tile == REEF_TILE_16x32k4) {
                        if (taps == 1) OpConvDirect<1, 2>::run(d, task, smem, np);
                        else if (taps == 9) OpConvDirect<9, 2>::run(d, task, smem, np);
                    }
                } else if (d.attr[REEF_CONV_MODE] == CONV_POINTWISE) {
                    if (tile == REEF_TILE_64x64) OpConv<Tile64x64, CONV_POINTWISE>::run(d, task, smem, np);
                    else if (tile == REEF_TILE_128x32) OpConv<Tile128x32, CONV_POINTWISE>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_32x32k4) OpConv<Tile32x32k4, CONV_POINTWISE>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_64x32k2) OpConv<Tile64x32k2, CONV_POINTWISE>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_32x64k2) OpConv<Tile32x64k2, CONV_POINTWISE>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_128x64) OpConv<Tile128x64, CONV_POINTWISE>::run(d, task, smem, np);
                } else if (d.attr[REEF_CONV_MODE] == CONV_GENERAL) {
                    if (tile == REEF_TILE_64x64) OpConv<Tile64x64, CONV_GENERAL>::run(d, task, smem, np);
                    else if (tile == REEF_TILE_128x32) OpConv<Tile128x32, CONV_GENERAL>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_128x64) OpConv<Tile128x64, CONV_GENERAL>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_32x32k4) OpConv<Tile32x32k4, CONV_GENERAL>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_64x32k2) OpConv<Tile64x32k2, CONV_GENERAL>::run(d, task, smem, np);
                    else if (LEVEL >= 2 && tile == REEF_TILE_32x64k2) OpConv<Tile32x64k2, CONV_GENERAL>::run(d, task, smem, np);
                }
            }
            break;
        case REEF_OP_SPLITK_REDUCE:
            // fewer partial loads in flight where the class allows 64 registers only
            if (LEVEL == 0) splitk_reduce_body<4>(d, task);
            else splitk_reduce_body<8>(d, task);
            break;
        case REEF_OP_DWCONV2D: dwconv2d_body(d, task); break;
        case REEF_OP_POOL2D: pool2d_body(d, task); break;
        case REEF_OP_GLOBAL_AVGPOOL: global_avgpool_body(d, task); break;
        case REEF_OP_ELTWISE: eltwise_body(d, task); break;
        case REEF_OP_DENSE: dense_body(d, task); break;
        case REEF_OP_SOFTMAX: softmax_body(d, task); break;
        case REEF_OP_LAYERNORM: layernorm_body(d, task); break;
        case REEF_OP_BIAS_GELU: bias_gelu_body(d, task); break;
        case REEF_OP_EMBEDDING: embedding_body(d, task); break;
        case REEF_OP_COPY: copy_body(d, task); break;
        case REEF_OP_TRANSPOSE: transpose_body(d, task); break;
        case REEF_OP_MOCK_ADD: if (threadIdx.x < 128) mocked_body<false>(d, task, threadIdx.x); break;
        case REEF_OP_MOCK_MULTIPLY: if (threadIdx.x < 128) mocked_body<true>(d, task, threadIdx.x); break;
        default: break;
    }
}
}  // namespace

#define REEF_PROXY(N, LEVEL)                                                                \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS)                           \
    __attribute__((amdgpu_waves_per_eu(N, N))) merge_framework_##N(ReefDkpArgs) {           \
        extern __shared__ __align__(16) char dyn_smem[];                                    \
        const ReefDkpArgs& a = kernarg_at<ReefDkpArgs>(0);                                  \
        DkpWalk w;                                                                          \
        if (!dkp_walk(a, w)) return;                                                        \
        const ReefDkpSide& side = w.right ? a.r : a.l;                                      \
        int* slot = w.right ? a.task_slot_r : nullptr;                                      \
        for (int i = w.idx; i < w.end; i += w.step) {                                       \
            run_op<LEVEL>(side, i, dyn_smem);                                               \
            __syncthreads();                                                                \
            if (slot && threadIdx.x == 0) atomicAdd(slot, 1);                               \
        }                                                                                   \
    }
REEF_PROXY(8, 0)
REEF_PROXY(3, 1)
REEF_PROXY(2, 2)
#endif
