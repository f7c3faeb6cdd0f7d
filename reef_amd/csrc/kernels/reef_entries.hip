// Entry points of the REEF code objects for gfx950.  This one source is
// compiled three times (REEF_FLAVOUR = 0 raw, 1 be, 2 trans) into
// reef_kernels.{raw,be,trans}.co, the three code objects a model directory
// carries (src/reef/server/scheduler.cpp:62-65; raw.co is used by the
// reference's tests only, src/reef/test/test.cpp:19).
//
//   raw    K(ReefOpDesc)                               plain launch, task = blockIdx.x
//   be     K(ReefBeArgs) = (completion record, int* preempted, int* task_slot, ReefOpDesc)
//          script/best_effort_kernel.py:22-29 restated: leave at once when the
//          flag is set, poll it again inside long bodies, count completed
//          workgroups in *task_slot; the last workgroup to leave tells the
//          launch-window stream that the kernel is done.
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
template <int R, int TN = 1, int TM = 1, bool PRE = false, bool ROWS = false, bool PACKED = false>
struct OpConvDirect {
    static constexpr int LDS = TileD16<TN, TM>::LDS_BYTES;
    static constexpr bool CHECKS_FLAG_ITSELF = true;   // the body makes the wrapper's first flag check
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_direct_body<R, TN, TM, PRE, ROWS, PACKED>(d, task, smem, p);
    }
};
// the same with the weights read from their packed copy
template <int R, int TN = 1, int TM = 1>
using OpConvDirectK = OpConvDirect<R, TN, TM, false, false, true>;
template <int G, int TM = 1>
using OpConvRowsK = OpConvDirect<9, G, TM, false, true, true>;
// row form of the 3x3 convolution: G image rows x one 14-column segment per workgroup
template <int G, int TM = 1>
using OpConvRows = OpConvDirect<9, G, TM, false, true>;
// 1x1 convolution and the depthwise 3x3 convolution (stride S) behind it in one launch
template <int G, int S = 1>
struct OpConvXdw {
    static constexpr int LDS = TileXdw<G, S>::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_xdw_body<G, S>(d, task, smem, p);
    }
};
// front filter (STEM: 3x3 / stride 2 on the image, else a 1x1 expansion), depthwise 3x3 (stride S) and 1x1
// projection in one launch, every channel in one workgroup
template <int G, int S, bool STEM, int MT, int KC>
struct OpConvBlock {
    static constexpr int LDS = TileBlk<G, S, STEM, MT, KC>::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_block_body<G, S, STEM, MT, KC>(d, task, smem, p);
    }
};
// 7x7 stride-2 convolution and the 3x3 stride-2 max-pool behind it in one launch
struct OpConvStemPool {
    static constexpr int LDS = TileSp7::LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return conv2d_stem_pool_body(d, task, smem, p);
    }
};
template <class T, bool TRANS_B, bool LN_A = false>
struct OpGemm {
    static constexpr int LDS = T::LDS_BYTES + (LN_A ? 2 * T::BM * 4 : 0);   // + mean, rstd of the tile's rows
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P& p) {
        return gemm_body<T, TRANS_B, LN_A>(d, task, smem, p);
    }
};
template <int TM, int TN>
struct OpGemmNtDirect {
    static constexpr int LDS = TileD16<TN, TM>::LDS_BYTES;
    static constexpr bool CHECKS_FLAG_ITSELF = true;
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
struct OpAttention {
    static constexpr int LDS = REEF_AT_LDS_BYTES;
    template <class P>
    static __device__ __forceinline__ bool run(const ReefOpDesc& d, int task, char* smem, const P&) {
        attention_body(d, task, smem);
        return true;
    }
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
#if REEF_FLAVOUR == 2
        const int t = threadIdx.x;   // the padding flavour is launched with a flat workgroup
#else
        const int t = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y;
#endif
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

// Touches every 64-byte line of the argument block at once and waits for them together.
// The block was written by the host a moment ago and is in no cache: a kernel that reads its
// attributes, then (depending on them) its pointers, then (depending on the flags) its optional
// operands takes one trip to memory per line it touches for the first time, one after the
// other -- 0.8 us each, measured -- before it can issue its first load.  After this call the
// lines are in the scalar cache and those reads cost a cache hit.  The loaded words themselves
// are not used; the wait is part of the statement, so no register is written behind the
// compiler's back.
// Only words of the block itself are read: one every 64 bytes from its start, and its last
// word (the block need not start on a line boundary, so its tail may lie on a line of its
// own).  An offset that would fall behind the block is moved onto the last word.
template <int BYTES, int I>
struct KernargWord {
    static constexpr int value = I * 64 + 4 <= BYTES ? I * 64 : BYTES - 4;
    static_assert(value >= 0 && value + 4 <= BYTES && value % 4 == 0, "reads inside the argument block only");
};
template <int BYTES>
__device__ __forceinline__ void kernarg_warm() {
    const char* base = (const char*)__builtin_amdgcn_kernarg_segment_ptr();
    static_assert(BYTES >= 4 && BYTES % 4 == 0 && BYTES <= 512, "argument blocks are whole words, at most 512 bytes");
    int t0, t1, t2, t3, t4, t5, t6, t7, t8;
#define REEF_KW(I) "n"(KernargWord<BYTES, I>::value)
    if (BYTES <= 256)
        asm volatile("s_load_dword %0, %5, %6\n\ts_load_dword %1, %5, %7\n\ts_load_dword %2, %5, %8\n\t"
                     "s_load_dword %3, %5, %9\n\ts_load_dword %4, %5, %10\n\ts_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4)
                     : "s"(base), REEF_KW(0), REEF_KW(1), REEF_KW(2), REEF_KW(3), "n"(BYTES - 4) : "memory");
    else
        asm volatile("s_load_dword %0, %9, %10\n\ts_load_dword %1, %9, %11\n\ts_load_dword %2, %9, %12\n\t"
                     "s_load_dword %3, %9, %13\n\ts_load_dword %4, %9, %14\n\ts_load_dword %5, %9, %15\n\t"
                     "s_load_dword %6, %9, %16\n\ts_load_dword %7, %9, %17\n\ts_load_dword %8, %9, %18\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6), "=&s"(t7),
                       "=&s"(t8)
                     : "s"(base), REEF_KW(0), REEF_KW(1), REEF_KW(2), REEF_KW(3), REEF_KW(4), REEF_KW(5),
                       REEF_KW(6), REEF_KW(7), "n"(BYTES - 4) : "memory");
#undef REEF_KW
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
    const int layer = div_small(b, C), cu = b - layer * C;
    const int slot = div_small(cu, X), xcd = cu - slot * X;
    const int rt_slots = div_small(a.cu_partition, X);
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
        kernarg_warm<sizeof(ReefOpDesc)>();                                           \
        OP::run(kernarg_at<ReefOpDesc>(0), (int)blockIdx.x, smem, NoPoll{true});      \
    }
#elif REEF_FLAVOUR == 1
namespace {
// A best-effort workgroup counts itself out as it leaves (finished or preempted).  The last
// one of the launch puts the counter back to zero for the next launch on the stream, stores
// the device clock and then the launch's sequence number where the host sees them.  All with
// ordinary vector stores whose scope travels on the instruction; the clock is acknowledged
// before the sequence number is sent.
__device__ __forceinline__ void be_signal_exit(const ReefBeArgs& a, int t) {
    if (a.done_word == nullptr) return;   // not on a launch-window stream
    __syncthreads();                      // every thread of the workgroup is past its work
    if (t != 0) return;
    const unsigned total = gridDim.x * gridDim.y * gridDim.z;
    const unsigned old = __hip_atomic_fetch_add(a.exit_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old != total - 1) return;
    __hip_atomic_store(a.exit_count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(a.exit_ticks, (uint64_t)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __hip_atomic_store(a.done_word, a.seq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
}  // namespace
namespace {
// Ops whose body makes the first flag check of a best-effort workgroup itself, at a point where
// its loads are already under way (the direct families); for all others the wrapper makes it.
template <class OP, class = void>
struct ChecksFlagItself { static constexpr bool value = false; };
template <class OP>
struct ChecksFlagItself<OP, decltype((void)OP::CHECKS_FLAG_ITSELF)> { static constexpr bool value = OP::CHECKS_FLAG_ITSELF; };
}  // namespace
#define REEF_ENTRY(NAME, OP)                                                              \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS) NAME(ReefBeArgs) {      \
        __shared__ __align__(16) char smem[OP::LDS > 0 ? OP::LDS : 16];                   \
        __shared__ int s_pre;                                                             \
        kernarg_warm<sizeof(ReefBeArgs)>();                                               \
        const ReefBeArgs& a = kernarg_at<ReefBeArgs>(0);                                  \
        const int t = threadIdx.x + threadIdx.y * blockDim.x + threadIdx.z * blockDim.x * blockDim.y; \
        FlagPoll poll{a.preempted};                                                       \
        bool done = false;                                                                \
        if (ChecksFlagItself<OP>::value) {                                                \
            done = OP::run(a.desc, (int)blockIdx.x, smem, poll);                          \
        } else {                                                                          \
            if (t == 0) s_pre = poll.load();                                              \
            __syncthreads();                                                              \
            if (!s_pre) done = OP::run(a.desc, (int)blockIdx.x, smem, poll);              \
        }                                                                                 \
        if (done && t == 0) atomicAdd(a.task_slot, 1);                                    \
        be_signal_exit(a, t);                                                             \
    }
#else
// Every entry also publishes the address of its first instruction in a device variable
// <name>_entry: what the reference reads out of the kernel descriptor on the host
// (GPUConfig::get_kernel_address, src/reef/executor/hip/hip_impl.cpp:16-32) and passes to its
// proxies as func_l / func_r.  A merge_framework_<n> proxy jumps there.
#define REEF_ENTRY(NAME, OP)                                                           \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS) NAME(ReefDkpArgs) {  \
        __shared__ __align__(16) char smem[OP::LDS > 0 ? OP::LDS : 16];                \
        kernarg_warm<sizeof(ReefDkpArgs)>();                                           \
        const ReefDkpArgs& a = kernarg_at<ReefDkpArgs>(0);                             \
        DkpWalk w;                                                                     \
        if (!dkp_walk(a, w)) return;                                                   \
        const ReefDkpSide& side = w.right ? a.r : a.l;                                 \
        for (int i = w.idx; i < w.end; i += w.step) {                                  \
            OP::run(side.desc, i, smem, NoPoll{!w.right});                             \
            __syncthreads();                                                           \
        }                                                                              \
    }                                                                                  \
    extern "C" __device__ __attribute__((used)) void* const NAME##_entry = (void*)NAME;
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
REEF_ENTRY(reef_conv2d_r9_g1, OpConvRows<1>)
REEF_ENTRY(reef_conv2d_r9_g2, OpConvRows<2>)
REEF_ENTRY(reef_conv2d_r9_g4, OpConvRows<4>)
REEF_ENTRY(reef_conv2d_r9_g7, OpConvRows<7>)
REEF_ENTRY(reef_conv2d_r9_g2m2, OpConvRows<2 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_r9_g4m2, OpConvRows<4 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_r9k_g1, OpConvRowsK<1>)
REEF_ENTRY(reef_conv2d_r9k_g2, OpConvRowsK<2>)
REEF_ENTRY(reef_conv2d_r9k_g4, OpConvRowsK<4>)
REEF_ENTRY(reef_conv2d_d9k_16x16k4, OpConvDirectK<9>)
REEF_ENTRY(reef_conv2d_d9k_16x32k4, OpConvDirectK<9 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d9k_32x32d4, OpConvDirectK<9 REEF_COMMA 2 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d3k_16x16k4, OpConvDirectK<3>)
REEF_ENTRY(reef_conv2d_d3k_16x32k4, OpConvDirectK<3 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d25_16x16k4, OpConvDirect<25>)
REEF_ENTRY(reef_conv2d_d25_16x32k4, OpConvDirect<25 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d25k_16x16k4, OpConvDirectK<25>)
REEF_ENTRY(reef_conv2d_d25k_16x32k4, OpConvDirectK<25 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_d7k_16x16k4, OpConvDirectK<7>)
REEF_ENTRY(reef_conv2d_d7k_16x32k4, OpConvDirectK<7 REEF_COMMA 2>)
REEF_ENTRY(reef_conv2d_xdw_g2, OpConvXdw<2>)
REEF_ENTRY(reef_conv2d_xdw_g4, OpConvXdw<4>)
REEF_ENTRY(reef_conv2d_sp7_g2, OpConvStemPool)
REEF_ENTRY(reef_conv2d_sdp_g2, OpConvBlock<2 REEF_COMMA 1 REEF_COMMA true REEF_COMMA 2 REEF_COMMA 1>)
REEF_ENTRY(reef_conv2d_sdp_g4, OpConvBlock<4 REEF_COMMA 1 REEF_COMMA true REEF_COMMA 2 REEF_COMMA 1>)
REEF_ENTRY(reef_conv2d_xdp2_g1, OpConvBlock<1 REEF_COMMA 2 REEF_COMMA false REEF_COMMA 6 REEF_COMMA 4>)
REEF_ENTRY(reef_conv2d_xdp2_g2, OpConvBlock<2 REEF_COMMA 2 REEF_COMMA false REEF_COMMA 6 REEF_COMMA 4>)
REEF_ENTRY(reef_conv2d_xdw2_g2, OpConvXdw<2 REEF_COMMA 2>)
REEF_ENTRY(reef_gemm_nt_128x128, OpGemm<Tile128x128 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_64x64, OpGemm<Tile64x64 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_32x128, OpGemm<Tile32x128 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_32x32k4, OpGemm<Tile32x32k4 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_nt_64x32k2, OpGemm<Tile64x32k2 REEF_COMMA true>)
REEF_ENTRY(reef_gemm_ntl_32x32k4, OpGemm<Tile32x32k4 REEF_COMMA true REEF_COMMA true>)
REEF_ENTRY(reef_gemm_ntl_64x32k2, OpGemm<Tile64x32k2 REEF_COMMA true REEF_COMMA true>)
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
REEF_ENTRY(reef_attention, OpAttention)
REEF_ENTRY(reef_embedding, OpEmbedding)
REEF_ENTRY(reef_copy, OpCopy)
REEF_ENTRY(reef_transpose, OpTranspose)
REEF_ENTRY(add, OpMocked<false>)
REEF_ENTRY(multiply, OpMocked<true>)

#if REEF_FLAVOUR == 2
// ---- merge_framework_<n>: two different kernels in one launch ---------------------------
// As in the reference (script/transform_kernel.py:689-718) a proxy is a trampoline: it finds
// the side of its workgroup and jumps to the first instruction of that side's own kernel,
// whose address the host passes in (entry_l / entry_r, the reference's func_l / func_r).  The
// kernel then runs exactly as if it had been launched directly: it reads the same argument
// block, finds the same side and walks that side's tasks.  Any two kernels of this code object
// can share a launch that way, and each runs the very code of its solo launch.
//
// What makes the jump legal is that a proxy starts its wavefronts in the state every kernel
// here expects: argument block address in s[0:1], workgroup id in s2, packed work-item id in
// v0, no other preloaded registers, no scratch, the same floating-point mode (all kernels are
// built from this one source with one set of flags, none uses blockIdx.y/z or hidden
// arguments), and LDS from offset 0 (the launch passes the larger static need of the two
// sides as dynamic LDS, src/reef/server/scheduler.cpp:643-649).  The proxy's own kernel
// descriptor fixes the register file of the launch, so, like the reference's ten variants
// whose register counts are patched to the gfx906 occupancy classes
// (script/replace_register_usage.py:33-59), there is one proxy per gfx950 register class:
// <n> wavefronts per SIMD = 512 / n unified registers, split into V architectural VGPRs (the
// accumulation registers start behind them) and A accumulation registers.  The counts are
// claimed by naming the last register of each kind as clobbered.  The host picks the class
// with the most wavefronts whose V and A hold both kernels (TransExecutor::select_proxy).
//
//   proxy                 V    A   unified  wavefronts/SIMD
//   merge_framework_8     64    0     64    8   bandwidth-bound kernels
//   merge_framework_5     96    0     96    5
//   merge_framework_4     96   32    128    4
//   merge_framework_3    136   32    168    3   direct / row convolutions, 64x64 and 128x32 staged tiles
//   merge_framework_3b   152   16    168    3
//   merge_framework_2    192   64    256    2   wide tiles
//   merge_framework_2b   224   32    256    2
//   merge_framework_2c   128  128    256    2
//   merge_framework_1    256  256    512    1   everything else
#define REEF_PROXY(NAME, LAST_V, LAST_A_CLOBBER)                                             \
    extern "C" __global__ void __launch_bounds__(REEF_WG_THREADS) NAME(ReefDkpArgs) {        \
        kernarg_warm<sizeof(ReefDkpArgs)>();                                                 \
        const ReefDkpArgs& a = kernarg_at<ReefDkpArgs>(0);                                   \
        const void* kernarg = __builtin_amdgcn_kernarg_segment_ptr();                        \
        const unsigned wg = __builtin_amdgcn_workgroup_id_x();                               \
        const unsigned tid = __builtin_amdgcn_workitem_id_x();                               \
        const int C = a.num_cus, X = a.num_xcds;                                             \
        const int cu = (int)wg - div_small((int)wg, C) * C;                                  \
        const bool right = div_small(cu, X) >= div_small(a.cu_partition, X);   /* the side test of dkp_walk */ \
        const void* target = right ? a.entry_r : a.entry_l;                                  \
        asm volatile("s_setpc_b64 %3"                                                        \
                     :                                                                       \
                     : "{s[0:1]}"(kernarg), "{s2}"(wg), "{v0}"(tid), "s"(target)             \
                     : "s99", "vcc", LAST_V LAST_A_CLOBBER, "memory");                       \
        __builtin_unreachable();                                                             \
    }
REEF_PROXY(merge_framework_8, "v63", )
REEF_PROXY(merge_framework_5, "v95", )
REEF_PROXY(merge_framework_4, "v95", REEF_COMMA "a31")
REEF_PROXY(merge_framework_3, "v135", REEF_COMMA "a31")
REEF_PROXY(merge_framework_3b, "v151", REEF_COMMA "a15")
REEF_PROXY(merge_framework_2, "v191", REEF_COMMA "a63")
REEF_PROXY(merge_framework_2b, "v223", REEF_COMMA "a31")
REEF_PROXY(merge_framework_2c, "v127", REEF_COMMA "a127")
REEF_PROXY(merge_framework_1, "v255", REEF_COMMA "a255")
#endif
