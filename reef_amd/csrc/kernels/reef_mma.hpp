// fp32 implicit-GEMM convolution and batched GEMM on the gfx950 matrix cores.
//
// Replaces the reference's generated direct-convolution kernels
// (resource/resnet152/resnet152.cu:35-4786, families fused_nn_conv2d[_add]
// [_add][_multiply_add][_nn_relu]) and batch_matmul kernels
// (resource/bert/bert.cu:22-271), which stage tiles in LDS and issue scalar
// __ocml_fma_f32.  Here a 256-thread workgroup (4 wavefronts) owns a BM x BN
// output tile and walks K in steps of 32 with v_mfma_f32_32x32x2f32:
//
//   out[M][N] = A[M][K] x B[K][N]
//   conv : A = weights OIHW viewed as [Cout][Cin*kh*kw]  (K contiguous)
//          B = im2col(input)[k=(c,ky,kx)][n=(y,x)]        (gathered on the fly)
//   gemm : A = [M][K] row-major; B = [N][K] (trans_b) or [K][N]
//
// LDS staging, double-buffered, one barrier per K step:
//   A tile  [BM][36]   (row = m, 32 k values + 4 pad floats)  -> the MFMA A
//           fragment of a lane (m, h) is ONE ds_read_b128 of k = 8j+4h .. +3.
//   B tile  [32][BN]   (row = k)                               -> four ds_read_b32.
//   (trans_b GEMM stores B like A and reads it with ds_read_b128.)
// The MFMA sums its two k slots, so any k -> slot assignment is legal as long
// as A and B agree; slot h of MFMA t inside group j carries k = 8j + 4h + t.
//
// Accumulator layout of v_mfma_f32_32x32x2f32 (16 floats per lane):
//   element r of lane l  ->  row = 8*(r/4) + 4*(l/32) + r%4,  col = l%32.
#pragma once
#include "reef_common.hpp"

namespace reef_dev {

// KW_ > 1 splits K across wavefronts: the workgroup stages 32 * KW k values per
// step, wavefront kw of a (row, column) group multiplies the kw-th 32 of them, and
// the KW partial tiles are summed through LDS after the loop (always in the order
// kw = 0, 1, ..).  A batch-1 layer has far fewer output tiles than the device has
// matrix pipes; this puts all four pipes of a CU on one small tile without a
// second kernel to fold partial sums.
template <int WGM_, int WGN_, int TM_, int TN_, int DEPTH_, int KW_ = 1>
struct Tile {
    static constexpr int WGM = WGM_, WGN = WGN_, TM = TM_, TN = TN_, KW = KW_;
    static constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32, BK = 32 * KW;
    // K steps whose global loads are in flight at once.  A batch-1 layer gives a
    // workgroup only a handful of K steps, each shorter than one trip to memory, so
    // the loads of several steps have to be outstanding together.
    static constexpr int DEPTH = DEPTH_;
    static_assert(DEPTH_ % 2 == 0, "the LDS buffer of a step is picked by the stage's parity");
    static constexpr int LDA = BK + 4;
    static constexpr int A_FLOATS = BM * LDA;
    static constexpr int BK_FLOATS = BK * BN;   // B tile, k-major
    static constexpr int BN_FLOATS = BN * LDA;  // B tile, n-major (trans_b GEMM)
    static constexpr int B_FLOATS = BN_FLOATS > BK_FLOATS ? BN_FLOATS : BK_FLOATS;
    static constexpr int LDS_BYTES = 2 * (A_FLOATS + B_FLOATS) * 4 + 16;
    static constexpr int RPW = 16 / KW;  // accumulator rows-of-lanes each wavefront finishes
    static_assert(WGM * WGN * KW == 4, "four wavefronts per workgroup");
    static_assert(KW == 1 || 4 * TM * TN * 16 * 64 <= 2 * (A_FLOATS + B_FLOATS),
                  "the partial tiles are exchanged through the staging buffers");
};

typedef Tile<2, 2, 2, 2, 2> Tile128x128;
typedef Tile<2, 2, 2, 1, 2> Tile128x64;
typedef Tile<2, 2, 1, 1, 2> Tile64x64;
typedef Tile<4, 1, 1, 1, 2> Tile128x32;
typedef Tile<1, 4, 1, 1, 2> Tile32x128;
typedef Tile<2, 2, 1, 2, 2> Tile64x128;
typedef Tile<1, 1, 1, 1, 2, 4> Tile32x32k4;
typedef Tile<2, 1, 1, 1, 2, 2> Tile64x32k2;
typedef Tile<1, 2, 1, 1, 2, 2> Tile32x64k2;

// All tile loads are buffer loads: an element outside the tensor or outside this launch's K
// range (row >= M, k >= k_end, a padding tap) is addressed at kOutside and comes back as 0, so
// a K step's loads issue back to back with one compare-and-select per load and nothing to
// patch up afterwards.

// ---- A tile: rows of a K-contiguous matrix -------------------------------
// VEC: rows are 16-byte aligned at every k that is a multiple of 4 (K % 4 == 0).
// LN (reef_gemm_ntl_*): the rows go into LDS as they are; on the way every thread adds what it
// loads to per-row sums of (a - p) and (a - p)^2 around a pivot p (element 0 of the row), from
// which gemm_body makes the row's mean and variance once the K loop has seen the whole row.
template <class T, bool VEC, bool LN = false>
struct ALoader {
    static constexpr int TPR = T::BK / 4;          // threads (float4s) per tile row
    static constexpr int RPP = kThreads / TPR;     // rows per pass
    static constexpr int NV = T::BM / RPP;         // float4 per thread per tile
    static_assert(NV >= 1, "tile shorter than one pass");
    static_assert(!LN || VEC, "the LayerNorm form loads whole float4s");
    struct Regs { f32x4 v[NV]; float in; };     // in (LN): 1 for a float4 inside K, 0 for one outside
    rsrc_t rs;
    unsigned rowoff[NV];    // byte offset of the row (kOutside when the row is outside M)
    int k;                  // k of this thread's float4 in the next tile
    int k_end;
    // LN only
    float pivot[LN ? NV : 1], s1[LN ? NV : 1], s2[LN ? NV : 1];
    __device__ __forceinline__ void init_ln() {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            pivot[LN ? i : 0] = buf_load(rs, rowoff[i]);
            s1[LN ? i : 0] = s2[LN ? i : 0] = 0.0f;
        }
    }

    // `bytes`: size of the matrix from `a` on
    __device__ __forceinline__ void init(const float* a, unsigned bytes, int lda, int m0, int M,
                                         int k_begin, int k_end_) {
        const int tid = threadIdx.x;
        rs = make_rsrc(a, bytes);
        k_end = k_end_;
        k = k_begin + (tid % TPR) * 4;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int row = m0 + tid / TPR + RPP * i;
            rowoff[i] = row < M ? (unsigned)row * (unsigned)lda * 4u : kOutside;
        }
    }
    __device__ __forceinline__ void load(Regs& r) {
        if (VEC) {
            // k and k_end are multiples of 4 here: the float4 is inside or outside as a whole
            const unsigned koff = k < k_end ? (unsigned)k * 4u : kOutside;
#pragma unroll
            for (int i = 0; i < NV; ++i) r.v[i] = buf_load4(rs, rowoff[i] + koff);
            if (LN) r.in = k < k_end ? 1.0f : 0.0f;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const unsigned koff = k + e < k_end ? (unsigned)(k + e) * 4u : kOutside;
#pragma unroll
                for (int i = 0; i < NV; ++i) r.v[i][e] = buf_load(rs, rowoff[i] + koff);
            }
        }
        k += T::BK;
    }
    __device__ __forceinline__ void store(const Regs& r, float* As) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            if (LN) {
                // no branch in here: a branch between a stage's loads and its LDS stores makes the wait
                // for that stage a wait for every outstanding load, the next stage's included
                const float pv = pivot[LN ? i : 0] * r.in;     // a float4 outside K was loaded as zeros: 0 - 0
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float dl = r.v[i][e] - pv;
                    s1[LN ? i : 0] += dl;
                    s2[LN ? i : 0] = fmaf(dl, dl, s2[LN ? i : 0]);
                }
            }
            *(f32x4*)(As + (tid / TPR + RPP * i) * T::LDA + (tid % TPR) * 4) = r.v[i];
        }
    }
};

// ---- B tile for convolution: im2col gather, one n per thread --------------
// Thread (n, row group): n = tid % BN fixed for the whole kernel, k rows
// tid / BN + RS * i.  For BN >= 64 a wavefront works on one k row at a time, so
// the (channel, ky, kx) decode of the row and its carries live in scalar
// registers; per lane only the padding test (two precomputed bit masks) and one
// offset add remain.
template <class T>
struct Im2colLoader {
    static constexpr int RS = kThreads / T::BN;  // k rows covered per pass
    static constexpr int NR = T::BK / RS;        // rows per thread per tile
    static constexpr bool UNIFORM = T::BN >= 64; // one k row per wavefront
    struct Regs { float v[NR]; };
    rsrc_t rs;
    int HW, W, kh, kw;
    unsigned ymask, xmask;  // bit ky / kx: that tap is inside the image for this thread's pixel
    int soff;               // iy0 * W + ix0 of this thread's pixel (may be negative)
    int k, k_end, c, ky, kx;
    int dkx, dky, dc;

    __device__ __forceinline__ void init(const float* in_, const int* a, int n0, int N, int k_begin,
                                         int k_end_) {
        const int tid = threadIdx.x;
        const int H = a[REEF_CONV_H];
        W = a[REEF_CONV_W];
        HW = H * W;
        rs = make_rsrc(in_, (unsigned)a[REEF_CONV_CIN] * (unsigned)HW * 4u);
        kh = a[REEF_CONV_KH];
        kw = a[REEF_CONV_KW];
        const int Wo = a[REEF_CONV_WO];
        const int n = n0 + (tid & (T::BN - 1));
        const int y = div_small(n, Wo), x = n - y * Wo;
        const int iy0 = y * a[REEF_CONV_SH] - a[REEF_CONV_PH];
        const int ix0 = x * a[REEF_CONV_SW] - a[REEF_CONV_PW];
        soff = iy0 * W + ix0;
        ymask = xmask = 0;
        if (n < N) {
            for (int t = 0; t < kh; ++t) ymask |= ((unsigned)(iy0 + t) < (unsigned)H ? 1u : 0u) << t;
            for (int t = 0; t < kw; ++t) xmask |= ((unsigned)(ix0 + t) < (unsigned)W ? 1u : 0u) << t;
        }
        k_end = k_end_;
        int row0 = tid / T::BN;
        if (UNIFORM) row0 = __builtin_amdgcn_readfirstlane(row0);
        k = k_begin + row0;
        const int khw = kh * kw;
        c = div_small(k, khw);
        const int r = k - c * khw;
        ky = div_small(r, kw);
        kx = r - ky * kw;
        const int t = div_small(RS, kw);
        dkx = RS - t * kw;
        dc = div_small(t, kh);
        dky = t - dc * kh;
    }
    __device__ __forceinline__ void load(Regs& r) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const bool ok = (k < k_end) && (((ymask >> ky) & (xmask >> kx) & 1u) != 0);
            r.v[i] = buf_load(rs, ok ? (unsigned)(c * HW + ky * W + kx + soff) * 4u : kOutside);
            // advance (c, ky, kx) by RS rows, mixed radix (kh, kw), without branches
            k += RS;
            kx += dkx;
            const int cx = kx >= kw ? 1 : 0;
            kx -= kw & -cx;
            ky += dky + cx;
            const int cy = ky >= kh ? 1 : 0;
            ky -= kh & -cy;
            c += dc + cy;
        }
    }
    __device__ __forceinline__ void store(const Regs& r, float* Bs) const {
        const int tid = threadIdx.x;
        const int nl = tid & (T::BN - 1), kr0 = tid / T::BN;
#pragma unroll
        for (int i = 0; i < NR; ++i) Bs[(kr0 + RS * i) * T::BN + nl] = r.v[i];
    }
};

// ---- B tile for pointwise convolution (1x1, stride 1, no padding, N % 4 == 0) ----
// The im2col matrix is the input itself, [K = Cin][N = H*W] row-major: 128-bit
// loads along n, 128-bit LDS stores, one offset add per K step.
template <class T>
struct PointwiseLoader {
    static constexpr int C4 = T::BN / 4;                 // float4 per tile row
    static constexpr int NF = T::BK * C4 / kThreads;     // float4 per thread per tile
    static constexpr int RSTEP = kThreads / C4;          // rows between a thread's float4s
    static_assert(NF >= 1, "tile narrower than one pass");
    struct Regs { f32x4 v[NF]; };
    rsrc_t rs;
    unsigned off;   // byte offset of this thread's first float4 in the next tile
    unsigned step;  // RSTEP rows in bytes
    unsigned tile;  // BK rows in bytes
    int k, k_end;

    // K = all rows of the matrix (the buffer ends there), k_end = this launch's last row + 1
    __device__ __forceinline__ void init(const float* in_, int n0, int N, int K, int k_begin, int k_end_) {
        const int tid = threadIdx.x;
        rs = make_rsrc(in_, (unsigned)K * (unsigned)N * 4u);
        const int row = tid / C4, col = (tid % C4) * 4;
        k = k_begin + row;
        k_end = k_end_;
        // a column past N stays outside for every row
        off = n0 + col < N ? ((unsigned)k * (unsigned)N + (unsigned)(n0 + col)) * 4u : kOutside;
        step = (unsigned)RSTEP * (unsigned)N * 4u;
        tile = (unsigned)T::BK * (unsigned)N * 4u;
    }
    __device__ __forceinline__ void load(Regs& r) {
#pragma unroll
        for (int i = 0; i < NF; ++i)
            r.v[i] = buf_load4(rs, (k + RSTEP * i) < k_end ? off + step * i : kOutside);
        // (an offset that started at kOutside stays outside: the rows of a tensor below 1 GiB do
        // not carry it around the 32-bit range)
        off += tile;
        k += T::BK;
    }
    __device__ __forceinline__ void store(const Regs& r, float* Bs) const {
        const int tid = threadIdx.x;
        const int row = tid / C4, col = (tid % C4) * 4;
#pragma unroll
        for (int i = 0; i < NF; ++i) *(f32x4*)(Bs + (row + RSTEP * i) * T::BN + col) = r.v[i];
    }
};

// ---- B tile for GEMM with B stored [K][N] (n contiguous) -------------------
template <class T>
struct BknLoader {
    static constexpr int RS = kThreads / T::BN;
    static constexpr int NR = T::BK / RS;
    struct Regs { float v[NR]; };
    rsrc_t rs;
    unsigned noff;   // byte offset of this thread's column (kOutside when it is past N)
    unsigned ldb4;   // row pitch in bytes
    int k, k_end;
    __device__ __forceinline__ void init(const float* b, unsigned bytes, int ldb, int n0, int N,
                                         int k_begin, int k_end_) {
        const int tid = threadIdx.x;
        rs = make_rsrc(b, bytes);
        const int n = n0 + (tid & (T::BN - 1));
        noff = n < N ? (unsigned)n * 4u : kOutside;
        ldb4 = (unsigned)ldb * 4u;
        k = k_begin + tid / T::BN;
        k_end = k_end_;
    }
    __device__ __forceinline__ void load(Regs& r) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            r.v[i] = buf_load(rs, k < k_end ? (unsigned)k * ldb4 + noff : kOutside);
            k += RS;
        }
    }
    __device__ __forceinline__ void store(const Regs& r, float* Bs) const {
        const int tid = threadIdx.x;
        const int nl = tid & (T::BN - 1), kr0 = tid / T::BN;
#pragma unroll
        for (int i = 0; i < NR; ++i) Bs[(kr0 + RS * i) * T::BN + nl] = r.v[i];
    }
};

// ---- which part of the tile a wavefront owns ---------------------------------
// Wavefronts are numbered (group, kw): the KW wavefronts of a group share one
// TM*32 x TN*32 block of the tile and split the k values of every step.
template <class T>
struct WaveGeom {
    int wk, wm0, wn0;
    __device__ __forceinline__ WaveGeom() {
        const int wave = threadIdx.x >> 6;
        wk = wave % T::KW;
        const int g = wave / T::KW;
        wm0 = (g / T::WGN) * (T::TM * 32);
        wn0 = (g % T::WGN) * (T::TN * 32);
    }
};

// After the K loop: the values this wavefront writes out.  res[tm][tn][rr] is
// accumulator element r = r0 + rr of the lane (row = 8*(r/4) + 4*(lane/32) + r%4,
// col = lane%32).  With KW == 1 that is the wavefront's own accumulator (r0 = 0, all
// 16 elements); otherwise the KW partial tiles of the group go through LDS, are
// summed in the order kw = 0, 1, .., and each wavefront keeps 16/KW elements, so
// the epilogue is spread over all wavefronts too.
template <class T>
__device__ __forceinline__ int finish_tile(const f32x16 (&acc)[T::TM][T::TN],
                                           float (&res)[T::TM][T::TN][T::RPW], float* smem) {
    if (T::KW == 1) {
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int r = 0; r < T::RPW; ++r) res[tm][tn][r] = acc[tm][tn][r];
        return 0;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();  // every wavefront is done reading the staged tiles
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                smem[(((wave * T::TM + tm) * T::TN + tn) * 16 + r) * 64 + lane] = acc[tm][tn][r];
    __syncthreads();
    const int wk = wave % T::KW, first = wave - wk;
    const int r0 = wk * T::RPW;
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int rr = 0; rr < T::RPW; ++rr) {
                float v = smem[(((first * T::TM + tm) * T::TN + tn) * 16 + r0 + rr) * 64 + lane];
#pragma unroll
                for (int s = 1; s < T::KW; ++s)
                    v += smem[((((first + s) * T::TM + tm) * T::TN + tn) * 16 + r0 + rr) * 64 + lane];
                res[tm][tn][rr] = v;
            }
    return r0;
}

// ---- the MFMA inner product over one staged K step -------------------------
template <class T, bool B_NMAJOR>
__device__ __forceinline__ void mma_step(const float* As, const float* Bs, f32x16 (&acc)[T::TM][T::TN],
                                         int wm0, int wn0, int wk0) {
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    As += wk0;                                   // this wavefront's 32 k values of the step
    Bs += B_NMAJOR ? wk0 : wk0 * T::BN;
    // All operand fragments of the K step are fetched from LDS first, then the 16 x
    // TM x TN MFMAs issue back to back: one LDS round trip per step is exposed
    // instead of one per group of four MFMAs.
    f32x4 af[4][T::TM];
    f32x4 bf[4][T::TN];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
            af[j][tm] = *(const f32x4*)(As + (wm0 + tm * 32 + l32) * T::LDA + 8 * j + 4 * h);
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            if (B_NMAJOR) {
                bf[j][tn] = *(const f32x4*)(Bs + (wn0 + tn * 32 + l32) * T::LDA + 8 * j + 4 * h);
            } else {
                const float* bp = Bs + (8 * j + 4 * h) * T::BN + wn0 + tn * 32 + l32;
                bf[j][tn].x = bp[0];
                bf[j][tn].y = bp[T::BN];
                bf[j][tn].z = bp[2 * T::BN];
                bf[j][tn].w = bp[3 * T::BN];
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < T::TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[j][tm][t], bf[j][tn][t],
                                                                       acc[tm][tn], 0, 0, 0);
}

// K loop shared by conv and GEMM.  Global loads run DEPTH steps ahead of the
// matrix cores (register staging), LDS is double-buffered, one barrier per step:
//   step it:  regs[it % DEPTH] -> LDS[it & 1];  issue loads of step it + DEPTH;
//             barrier;  MFMAs on LDS[it & 1]
// The barrier of step it also proves every wavefront finished the MFMAs of step
// it - 1, whose LDS buffer step it + 1 overwrites.
// Returns false when the preemption flag was seen.  The whole workgroup leaves
// together: thread 0 reads the flag one step ahead (the load overlaps the MFMAs)
// and publishes it through LDS before the step's barrier.
template <class T, bool B_NMAJOR, class LA, class LB, class Poll>
__device__ __forceinline__ bool k_loop(LA& la, LB& lb, int nk, float* smem, f32x16 (&acc)[T::TM][T::TN],
                                       const Poll& poll) {
    constexpr int D = T::DEPTH;
    float* As = smem;
    float* Bs = smem + 2 * T::A_FLOATS;
    int* sflag = (int*)(smem + 2 * (T::A_FLOATS + T::B_FLOATS));
    const WaveGeom<T> wg;
    const int wm0 = wg.wm0, wn0 = wg.wn0, wk0 = wg.wk * 32;
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

    typename LA::Regs ra[D];
    typename LB::Regs rb[D];
    if (Poll::enabled && threadIdx.x == 0) *sflag = 0;
    // Loads past the last K step are issued too: the loaders mask them (k >= k_end)
    // to a stand-in address, which keeps the steady state free of branches.
#pragma unroll
    for (int s = 0; s < D; ++s) {
        la.load(ra[s]);
        lb.load(rb[s]);
        // Keep the stages' loads in this order: loads come back in the order they were issued, and the
        // wait in front of a stage's LDS stores counts the loads issued after it.  If the compiler moves
        // stage 1's loads in front of stage 0's here, the loop's first wait has to be a wait for
        // everything, and since the loop has one wait for both ways into it, so has every later one.
        asm volatile("" ::: "memory");
    }
    int pf = 0;
    int it = 0;
    for (;;) {
#pragma unroll
        for (int s = 0; s < D; ++s) {
            if (it >= nk) return true;
            const int cur = s & 1;  // D is even, so step parity == stage parity
            la.store(ra[s], As + cur * T::A_FLOATS);
            lb.store(rb[s], Bs + cur * T::B_FLOATS);
            if (Poll::enabled && threadIdx.x == 0) {
                if (pf) *sflag = 1;
                pf = poll.load();
            }
            __syncthreads();
            if (Poll::enabled && *sflag) return false;
            // refill this stage next to the MFMAs: the address arithmetic of the
            // loads fills the issue slots the dependent MFMA chain leaves free
            la.load(ra[s]);
            lb.load(rb[s]);
            mma_step<T, B_NMAJOR>(As + cur * T::A_FLOATS, Bs + cur * T::B_FLOATS, acc, wm0, wn0, wk0);
            ++it;
        }
    }
}

// ---- task -> tile order that keeps neighbours on one XCD ---------------------
// The dispatcher hands workgroup j to XCD j % 8 and every XCD has its own L2.  Tiles
// are numbered (split, m tile, n tile) row-major, so neighbours in that order share
// weight rows and input columns; handing XCD x the x-th CONTIGUOUS eighth of the
// order (instead of every eighth tile) lets one L2 fetch those once for all of them.
// Without it a 32-row weight tile used by seven column tiles is fetched by seven L2s.
// A bijection on [0, total): chunk x holds total/8 tiles, plus one if x < total % 8.
__device__ __forceinline__ int xcd_chunked(int task, int total) {
    constexpr int X = 8;
    const int x = task % X, l = task / X;
    const int base = total / X, r = total - base * X;
    return x * base + min(x, r) + l;
}

// ---- reef_conv2d ------------------------------------------------------------
// MODE selects the tile loaders, one K loop per kernel symbol:
//   CONV_GENERAL    im2col gather, 128-bit weight loads        (K % 4 == 0)
//   CONV_POINTWISE  1x1 / stride 1 / no padding / N % 4 == 0:  128-bit loads on both operands
//   CONV_UNALIGNED  im2col gather, element-wise weight loads    (any K; the 7x7x3 stem)
enum { CONV_GENERAL = 0, CONV_POINTWISE = 1, CONV_UNALIGNED = 2 };

// Epilogue operands of a convolution as buffers.  Optional operands follow the three fixed
// pointers in flag order (bias, residual, scale + shift, second output + its shift).  A
// per-channel vector is `channels` floats long and a full tensor `MN` floats, so an offset
// computed for a row >= M falls outside by itself; only a column >= N has to be turned into
// kOutside by the caller (it would land in the next row).
struct ConvEpilogue {
    rsrc_t out, out2, res, bias, scale, shift, shift2;
    bool has_res, has_bias, has_affine, has_dual;
    int act, act2;
    int next;         // first pointer slot after the optional operands
    unsigned doff4;   // byte offset of this layer's slice inside the output tensor(s)
    __device__ __forceinline__ void init(const ReefOpDesc& d, int flags, int act_, int act2_, int M,
                                         unsigned MN4, unsigned doff4_) {
        int p = 3;
        const unsigned M4 = (unsigned)M * 4u;
        doff4 = doff4_;
        out = make_rsrc(d.ptr[2], doff4 + MN4);
        has_bias = flags & REEF_F_BIAS;
        has_res = flags & REEF_F_RESIDUAL;
        has_affine = flags & REEF_F_AFFINE;
        has_dual = flags & REEF_F_DUAL;
        bias = res = scale = shift = out2 = shift2 = out;
        if (has_bias) bias = make_rsrc(d.ptr[p++], M4);
        if (has_res) res = make_rsrc(d.ptr[p++], MN4);
        if (has_affine) {
            scale = make_rsrc(d.ptr[p], M4);
            shift = make_rsrc(d.ptr[p + 1], M4);
            p += 2;
        }
        if (has_dual) {
            out2 = make_rsrc(d.ptr[p], doff4 + MN4);
            shift2 = make_rsrc(d.ptr[p + 1], M4);
            p += 2;
        }
        act = act_;
        act2 = act2_;
        next = p;
    }
    // off = (m * N + n) * 4 or outside; m4 = m * 4.  v = acc; v += residual; v += bias;
    // v = fma(v, scale, shift); act  -- then out2 = act2(out + shift2).
    // the layer's value for one output element
    __device__ __forceinline__ float value(float v, unsigned m4, float resv, float biasv) const {
        if (has_res) v = v + resv;
        if (has_bias) v = v + biasv;
        if (has_affine) v = fmaf(v, buf_load(scale, m4), buf_load(shift, m4));
        return act_apply(v, act);
    }
    __device__ __forceinline__ void finish(float v, unsigned off, unsigned m4, float resv, float biasv,
                                           float sh2v) const {
        const float o = value(v, m4, resv, biasv);
        buf_store(out, off + doff4, o);
        if (has_dual) buf_store(out2, off + doff4, act_apply(o + sh2v, act2));
    }
};

template <class T, int MODE, class Poll>
__device__ __forceinline__ bool conv2d_body(const ReefOpDesc& d_in, int task, char* smem_raw,
                                            const Poll& poll) {
  int M, N, split_k, split, rem, m0, n0;
  float* smem = (float*)smem_raw;
  f32x16 acc[T::TM][T::TN];
  // wave-split-K tiles leave each wavefront only 16/KW accumulator elements to write
  // out: few enough to fetch their bias / residual / second shift ahead of the K loop
  constexpr bool EARLY = T::KW > 1;
  constexpr int ER = EARLY ? T::RPW : 1;
  float e_bias[T::TM][ER], e_sh2[T::TM][ER], e_res[T::TM][T::TN][ER];
  const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
  const WaveGeom<T> wg;
  const int r0 = wg.wk * T::RPW;   // first accumulator element this wavefront writes out
  {
    const ReefOpDesc& d = d_in;
    const int* a = d.attr;
    M = a[REEF_CONV_COUT];
    N = a[REEF_CONV_HO] * a[REEF_CONV_WO];
    const int K = a[REEF_CONV_CIN] * a[REEF_CONV_KH] * a[REEF_CONV_KW];
    split_k = a[REEF_CONV_SPLIT_K];
    const int k_chunk = a[REEF_CONV_K_CHUNK];
    const int n_tiles = a[REEF_CONV_N_TILES];
    const int tiles = a[REEF_CONV_M_TILES] * n_tiles;
    task = xcd_chunked(task, tiles * split_k);
    split = div_small(task, tiles);
    rem = task - split * tiles;
    const int mt = div_small(rem, n_tiles), nt = rem - mt * n_tiles;
    m0 = mt * T::BM;
    n0 = nt * T::BN;
    const int k_begin = split * k_chunk;
    const int k_end = min(K, k_begin + k_chunk);
    const int nk = (k_end - k_begin + T::BK - 1) / T::BK;

    if (EARLY) {
        // Epilogue operands of the few outputs this wavefront will write: issued now, used
        // after the K loop.
        if (split_k == 1) {
            ConvEpilogue ep;
            ep.init(d, a[REEF_CONV_FLAGS], 0, 0, M, (unsigned)M * (unsigned)N * 4u, 0);
#pragma unroll
            for (int tm = 0; tm < T::TM; ++tm) {
                const unsigned mb = (unsigned)(m0 + wg.wm0 + tm * 32 + 4 * h + 8 * (r0 >> 2));
#pragma unroll
                for (int rr = 0; rr < T::RPW; ++rr) {
                    const unsigned m = mb + 8 * (rr >> 2) + (rr & 3);
                    e_bias[tm][rr] = ep.has_bias ? buf_load(ep.bias, m * 4u) : 0.0f;
                    e_sh2[tm][rr] = ep.has_dual ? buf_load(ep.shift2, m * 4u) : 0.0f;
#pragma unroll
                    for (int tn = 0; tn < T::TN; ++tn) {
                        const unsigned n = (unsigned)(n0 + wg.wn0 + tn * 32 + l32);
                        e_res[tm][tn][rr] = ep.has_res ? buf_load(ep.res, (m * (unsigned)N + n) * 4u) : 0.0f;
                    }
                }
            }
        }
        asm volatile("" ::: "memory");  // keeps the loads above the K loop
    }

    bool ok;
    if (MODE == CONV_POINTWISE) {
        ALoader<T, true> la;
        PointwiseLoader<T> lp;
        la.init((const float*)d.ptr[1], (unsigned)M * (unsigned)K * 4u, K, m0, M, k_begin, k_end);
        lp.init((const float*)d.ptr[0], n0, N, K, k_begin, k_end);
        ok = k_loop<T, false>(la, lp, nk, smem, acc, poll);
    } else {
        Im2colLoader<T> lb;
        lb.init((const float*)d.ptr[0], a, n0, N, k_begin, k_end);
        ALoader<T, MODE == CONV_GENERAL> la;
        la.init((const float*)d.ptr[1], (unsigned)M * (unsigned)K * 4u, K, m0, M, k_begin, k_end);
        ok = k_loop<T, false>(la, lb, nk, smem, acc, poll);
    }
    if (!ok) return false;
  }
    float res[T::TM][T::TN][T::RPW];
    finish_tile<T>(acc, res, smem);

    // Everything the epilogue needs is re-read from the argument block here, so the
    // K loop does not carry the epilogue's pointers in scalar registers.
    const ReefOpDesc* dp = &d_in;
    asm volatile("" : "+s"(dp));
    const ReefOpDesc& d = *dp;
    const int* a = d.attr;
    const int flags = a[REEF_CONV_FLAGS];
    const unsigned MN4 = (unsigned)M * (unsigned)N * 4u;
    const unsigned row4 = (unsigned)N * 4u;
    const bool fused = split_k > 1 && (flags & REEF_F_FUSED_REDUCE);

    if (!fused) {
        // One pass over this wavefront's outputs.  Offsets are 32-bit byte offsets built from a
        // per-lane base plus compile-time row steps; a column past N makes the base kOutside, a
        // row past M runs off the end of the buffer: no compares per element.
        const bool to_ws = split_k > 1;   // plain split-K: partial tile to the workspace
        ConvEpilogue ep;
        rsrc_t ws;
        if (to_ws) ws = make_rsrc((const float*)d.ptr[2] + (size_t)split * M * N, MN4);
        else ep.init(d, flags, a[REEF_CONV_ACT], a[REEF_CONV_ACT2], M, MN4, (unsigned)a[REEF_CONV_DST_OFF] * 4u);
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm) {
            const unsigned mb = (unsigned)(m0 + wg.wm0 + tm * 32 + 4 * h + 8 * (r0 >> 2));
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn) {
                const unsigned n = (unsigned)(n0 + wg.wn0 + tn * 32 + l32);
                const unsigned base = n < (unsigned)N ? (mb * (unsigned)N + n) * 4u : kOutside;
#pragma unroll
                for (int rr = 0; rr < T::RPW; ++rr) {
                    const unsigned c = 8 * (rr >> 2) + (rr & 3);
                    const unsigned off = base + c * row4;
                    const float v = res[tm][tn][rr];
                    if (to_ws) {
                        buf_store(ws, off, v);
                    } else {
                        const unsigned m4 = (mb + c) * 4u;
                        if (EARLY) {
                            ep.finish(v, off, m4, e_res[tm][tn][rr], e_bias[tm][rr], e_sh2[tm][rr]);
                        } else {
                            ep.finish(v, off, m4, ep.has_res ? buf_load(ep.res, off) : 0.0f,
                                      ep.has_bias ? buf_load(ep.bias, m4) : 0.0f,
                                      ep.has_dual ? buf_load(ep.shift2, m4) : 0.0f);
                        }
                    }
                }
            }
        }
        return true;
    }

    // fused split-K: store the partial, count in, the last arrival folds all partials in
    // ascending split order (fixed order => same bits whoever is last)
    const int wm0 = wg.wm0, wn0 = wg.wn0;
    const size_t MN = (size_t)M * N;
    float* dst = (float*)d.ptr[2] + a[REEF_CONV_DST_OFF];
    Epilogue ep;
    ep.unpack(d, 3, flags, a[REEF_CONV_ACT], a[REEF_CONV_ACT2]);
    if (ep.out2) ep.out2 += a[REEF_CONV_DST_OFF];
    {
        float* ws = (float*)d.ptr[ep.next];
        int* counters = (int*)d.ptr[ep.next + 1] + a[REEF_CONV_SYNC_OFF];
        int* s_last = (int*)(smem + 2 * (T::A_FLOATS + T::B_FLOATS)) + 1;
        float* part = ws + (size_t)split * MN;
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn) {
                const int n = n0 + wn0 + tn * 32 + l32;
#pragma unroll
                for (int rr = 0; rr < T::RPW; ++rr) {
                    const int r = r0 + rr;
                    const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < M && n < N) store_agent(part + (size_t)m * N + n, res[tm][tn][rr]);
                }
            }
        // Every store of this workgroup has completed at device scope before it counts in.  The
        // stores carry device scope themselves, so they are complete once acknowledged: each
        // lane waits for its own (a workgroup-scope fence alone does not wait for outstanding
        // stores on this target), then the barrier collects all lanes.
        partial_stores_done();
        __syncthreads();
        if (threadIdx.x == 0) {
            const int old = __hip_atomic_fetch_add(&counters[rem], 1, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
            *s_last = (old == split_k - 1);
        }
        __syncthreads();
        if (!*s_last) return true;
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn) {
                const int n = n0 + wn0 + tn * 32 + l32;
#pragma unroll
                for (int rr = 0; rr < T::RPW; ++rr) {
                    const int r = r0 + rr;
                    const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < M && n < N) {
                        const size_t idx = (size_t)m * N + n;
                        // loads of eight partials in flight together, sums in ascending s
                        float v = 0.0f;
                        for (int s0 = 0; s0 < split_k; s0 += 8) {
                            float p[8];
#pragma unroll
                            for (int j = 0; j < 8; ++j)
                                p[j] = load_agent(ws + (size_t)min(s0 + j, split_k - 1) * MN + idx);
#pragma unroll
                            for (int j = 0; j < 8; ++j)
                                if (s0 + j < split_k) v = (s0 + j == 0) ? p[j] : v + p[j];
                        }
                        ep.store(dst, v, m, idx);
                    }
                }
            }
        if (threadIdx.x == 0)  // ready for the next run
            __hip_atomic_store(&counters[rem], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return true;
    }
}

// ---- reef_conv2d_d<R>: operands straight from memory into the matrix cores ----------------
// A batch-1 layer is latency bound: every weight is used once per inference, so each K step of
// the tiled kernels above waits a full memory round trip (global -> registers -> LDS -> barrier).
// This family removes the staging.  A workgroup owns a 16 TM x 16 TN output tile (16 x 16 in the
// basic form) and its four wavefronts split the input channels; v_mfma_f32_16x16x4f32 takes one
// A value (row = lane % 16, k = lane / 16) and one B value (column = lane % 16, k = lane / 16)
// per lane, which a lane can load directly:
//   R > 1 (R = kh * kw taps): k slot kq = lane / 16 is input channel c + kq; the lane loads the
//          R contiguous weights W[m][c + kq][0..R) and the R taps in[c + kq][iy(t)][ix(t)] of
//          its output pixel; MFMA t multiplies tap t of four channels.  Tap offsets and their
//          padding validity are fixed per lane for the whole kernel.
//   R = 1: k slot kq covers eight channels c + 8 kq .. + 8: two 128-bit weight loads and eight
//          pixel loads; MFMA j multiplies channel j of each slot.  Any stride.
// No LDS and no barrier inside the K loop, so NS steps of loads are in flight per wavefront
// (a wavefront may have 63 vector-memory instructions outstanding; NS steps are up to 60 of
// them).  The four partial tiles are summed through LDS in wavefront order and thread t writes
// output element (t / 16, t % 16) of every 16 x 16 sub-tile, so stores are 64-byte runs along a row.  The sum order over k differs from
// the tiled kernels (it is fixed, so results are reproducible run to run).
template <int TN_, int TM_ = 1>
struct TileD16 {
    static constexpr int TN = TN_;      // 16-pixel column groups per workgroup
    static constexpr int TM = TM_;      // 16-row groups per workgroup: the tile is 16 TM x 16 TN
    static constexpr int BM = 16 * TM, BN = 16 * TN;
    static constexpr int PART = 320;    // floats per 16 x 16 partial tile in LDS (256 + row-group skew)
    static constexpr int SUBS = TM * TN;
    static constexpr int LDS_BYTES = 4 * SUBS * PART * 4 + 16;
};

template <int R, int TN, int TM = 1, bool PRE = false, bool ROWS = false>
struct DirectGeom {
    // channels per k slot and step.  1-tap filters: 4 -- a 128-bit load of weights per lane and step.
    // (8 halves the steps, but a step is also the unit in which loads and MFMAs alternate: with 4,
    // same process, ResNet-152 -2 %, Inception-v3 -1.4 %, MobileNetV2 -4.7 %, DenseNet-201 -2.4 %;
    // with 2 the weights come as 32-bit loads and ResNet-152 is 5-12 % slower.)
    static constexpr int CPL = R == 1 ? 4 : 1;
    static constexpr int RC = R * CPL;           // A values per lane and step (x TN B values and MFMAs)
    static constexpr int STEP_C = 16 * CPL;      // channels a workgroup consumes per step
    // B values a lane loads per step: every tap of every pixel group, or (row form) one value
    // per input row of the tile
    static constexpr int NB = ROWS ? TN + 2 : TN * RC;
    // vector-memory instructions per step (PRE: two 128-bit loads each of input scale and shift)
    static constexpr int LOADS = TM * ((RC / 4) + (RC % 4)) + NB + (PRE ? 2 * (RC / 4) : 0);
    // Steps of loads in flight per wavefront.  All of them are issued before the first MFMA, and a
    // wavefront that is still issuing loads multiplies nothing: with 8 steps ahead (all of a 14x14
    // row-form layer at a split of two) cycle stamps showed 4600 cycles of issue, then 6600 of K loop
    // whose MFMAs alone need 4600.  Fewer steps ahead start the MFMAs while the later loads are
    // still being issued behind them.  Picked per family by timing whole networks with the code
    // objects side by side in one process (ResNet-152 1.180 -> 1.102 ms, DenseNet-201 1.26 -> 1.18):
    //   row form 4 (3: +1.8 %, 5 and 6: +2.3 % on ResNet-152), d1 16x32 2 (3: +3.2 %), d1 16x16 and
    //   p1 16x16 3 (2 to 5 within 0.5 %), d9 16x16 3 (2, 4 the same); the others 40 loads' worth, at
    //   least 2 and at most 4.  (Steps of 1-tap filters are 64 channels.)
    static constexpr int NS_GEN = 40 / LOADS < 2 ? 2 : (40 / LOADS > 4 ? 4 : 40 / LOADS);
    static constexpr int NS = ROWS ? 4
                            : (R == 1 && TN == 1 && TM == 1) ? 3
                            : (R == 1 && TN == 2 && TM == 1 && !PRE) ? 2
                            : (R == 9 && TN == 1 && TM == 1) ? 3
                            : NS_GEN;
};

// Row form (ROWS; 3x3 filters, stride 1, padding 1; symbols reef_conv2d_r9_g<G>[m2]): the tile is
// G image rows x one 14-column segment of the output.  Pixel group g is image row y0 + g and the
// 16 lanes of a k slot are the columns of the segment: lanes 0..13 hold columns x0 .. x0 + 13,
// lane 14 the column right of the segment and lane 15 the column left of it (zero outside the
// image).  A lane loads ONE value per input row y0 - 1 .. y0 + G of its channel; the three
// horizontal taps of a row are that value (kx = 1) and its rotations by one lane within the
// 16-lane row (kx = 0: from lane - 1, lane 0 from lane 15; kx = 2: from lane + 1, lane 13 from
// lane 14), the three vertical taps are the rows g, g + 1, g + 2.  Every input value is fetched
// once per tile instead of once per tap: G + 2 loads per step instead of 9 G, so the loads of
// up to eight K steps are in flight per wavefront.  Lanes 14 and 15 compute columns nobody
// stores.  Same sum order over k as the tap form (channel-major steps, taps in filter order).
constexpr int kRowSeg = 14;
__device__ __forceinline__ float lane_from_left(float v) {   // lane i <- lane (i - 1) mod 16 of its row
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xF, 0xF, false));
}
__device__ __forceinline__ float lane_from_right(float v) {  // lane i <- lane (i + 1) mod 16 of its row
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x12F, 0xF, 0xF, false));
}

// TN > 1 widens the tile along the pixels: every weight value a lane has loaded is multiplied
// with TN pixel groups, so the weight rows -- the larger, cold operand -- are streamed by a
// TN-th of the workgroups.  TM > 1 does the same along the output channels for the input values.
// What a CU can pull from memory per microsecond is what bounds these kernels at batch 1 (a lone workgroup on an idle device takes as long as 208 of them), so fewer,
// wider tiles are combined with a split of K across workgroups to keep every CU busy with a
// shorter stream; REEF_F_FUSED_REDUCE then folds the split inside this launch: a workgroup
// stores its partial tile, counts itself in, and the last one to arrive for a tile adds the
// partial tiles in ascending split order (fixed order, so the result does not depend on who is
// last) and runs the epilogue.
//
// PRE (1-tap kernels only, symbols reef_conv2d_p1_*): the layer reads its input through a
// per-channel scale, shift and ReLU -- the pre-activation of a DenseNet layer, which cannot be
// folded into the producing convolution because every consumer of the concatenation has its own.
// The eight input values a lane loads per step are eight consecutive channels, so their scales
// and shifts are two 128-bit loads each; a channel past the split loads scale = shift = 0 and
// contributes relu(0) = 0.  REEF_F_PRE_ACT; the two vectors follow the optional epilogue operands.
//
// PACKED (filters with several taps; symbols reef_conv2d_d<R>k_* / reef_conv2d_r9k_*): the weights
// are read from a copy laid out for these loads instead of from OIHW, where the R taps of one
// (row, channel) are R * 4 bytes that start at any multiple of 4 and the 16 rows of a tile lie
// K * 4 bytes apart (a 128-bit load of a wavefront then touches some forty cache lines and most
// of its lanes are misaligned).  The copy is [Cout / 16][Cin / 4][taps / 4][k slot][row][4 taps]
// (zero-padded to whole groups): the 64 lanes of a wavefront read 1 KiB contiguous, aligned, per
// group of four taps.  Measured on the 3x3 layers of ResNet-152: 1.4 us less per launch.  The
// model generator writes the copy as a parameter of its own; attr WPACK names its pointer slot.
template <int R, int TN, int TM, bool PRE, bool ROWS, bool PACKED, class Poll>
__device__ __forceinline__ bool conv2d_direct_body(const ReefOpDesc& d_in, int task, char* smem_raw,
                                                   const Poll& poll) {
    static_assert(!PRE || R == 1, "the pre-activation form exists for 1-tap filters only");
    static_assert(!ROWS || R == 9, "the row form exists for 3x3 filters only");
    static_assert(!PACKED || R > 1, "1-tap filters are read from OIHW as they are");
    typedef DirectGeom<R, TN, TM, PRE, ROWS> G;
    typedef TileD16<TN, TM> TD;
    constexpr int RC = G::RC, NS = G::NS;
    float* smem = (float*)smem_raw;
    int* sflag = (int*)(smem + 4 * TD::SUBS * TD::PART);
    const ReefOpDesc& d = d_in;
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, i16 = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int M = a[REEF_CONV_COUT], C = a[REEF_CONV_CIN];
    const int H = a[REEF_CONV_H], W = a[REEF_CONV_W], Wo = a[REEF_CONV_WO];
    const int N = a[REEF_CONV_HO] * Wo;
    const int K = C * R;
    const int split_k = a[REEF_CONV_SPLIT_K];
    const int n_tiles = a[REEF_CONV_N_TILES];
    const int tiles = a[REEF_CONV_M_TILES] * n_tiles;
    const int flags = a[REEF_CONV_FLAGS];
    const bool fused = split_k > 1 && (flags & REEF_F_FUSED_REDUCE);
    const bool to_ws = split_k > 1 && !fused;   // plain split-K: partial tile to the workspace
    task = xcd_chunked(task, tiles * split_k);
    // Folded split: the workgroups of one tile are neighbours in the task order, so they run on
    // one XCD and meet in its L2; otherwise split-major like the staged tiles.
    const int q_split = div_small(task, fused ? split_k : tiles);
    const int split = fused ? task - q_split * split_k : q_split;
    const int rem = fused ? q_split : task - split * tiles;
    const int mt = div_small(rem, n_tiles), nt = rem - mt * n_tiles;
    const int m0 = mt * TD::BM, n0 = nt * TD::BN;
    // row form: spatial tile nt -> (row tile, column segment)
    const int segs = ROWS ? (W + kRowSeg - 1) / kRowSeg : 1;
    const int q_seg = ROWS ? div_small(nt, segs) : 0;
    const int y0 = ROWS ? q_seg * TN : 0;
    const int x0 = ROWS ? (nt - q_seg * segs) * kRowSeg : 0;
    const int c_chunk = a[REEF_CONV_K_CHUNK] / R;
    const int cb = split * c_chunk;
    const int ce = min(C, cb + c_chunk);
    const int nsteps = (ce - cb + G::STEP_C - 1) / G::STEP_C;
    const unsigned HW4 = (unsigned)(H * W) * 4u;
    const unsigned MN4 = (unsigned)M * (unsigned)N * 4u;

    // epilogue operands of the TM x TN output elements this thread writes (element (h, g): row
    // 16 h + t / 16, column 16 g + t % 16 of the tile), fetched ahead of the K loop
    const int orow = threadIdx.x >> 4, ocol = threadIdx.x & 15;
    unsigned om[TM], ooff[TM][TN];
#pragma unroll
    for (int h = 0; h < TM; ++h) {
        om[h] = (unsigned)(m0 + 16 * h + orow);
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            if (ROWS) {
                const bool ok = ocol < kRowSeg && x0 + ocol < W && y0 + g < H;
                ooff[h][g] = ok ? (om[h] * (unsigned)N + (unsigned)((y0 + g) * W + x0 + ocol)) * 4u : kOutside;
            } else {
                const unsigned on = (unsigned)(n0 + 16 * g + ocol);
                ooff[h][g] = on < (unsigned)N ? (om[h] * (unsigned)N + on) * 4u : kOutside;
            }
        }
    }
    // Pointer slot behind the optional epilogue operands (known from the flags alone): the
    // epilogue itself is set up further down, after the first loads of the K loop are on their
    // way -- its operands are needed last.
    const int ep_next = to_ws ? 3
                              : 3 + ((flags & REEF_F_BIAS) ? 1 : 0) + ((flags & REEF_F_RESIDUAL) ? 1 : 0) +
                                    ((flags & REEF_F_AFFINE) ? 2 : 0) + ((flags & REEF_F_DUAL) ? 2 : 0);
    // per-lane operand offsets
    const rsrc_t rs_a = make_rsrc(d.ptr[1], (unsigned)M * (unsigned)K * 4u);
    const rsrc_t rs_b = make_rsrc(d.ptr[0], (unsigned)C * HW4);
    const int lane_c = cb + (wave * 4 + kq) * G::CPL;     // first channel of this lane's k slot
    constexpr int G4 = (R + 3) / 4;                 // groups of four taps in the packed copy
    const unsigned C4 = (unsigned)(C + 3) / 4u;
    const rsrc_t rs_ap = make_rsrc(d.ptr[PACKED ? a[REEF_CONV_WPACK] : 1],
                                   PACKED ? (unsigned)((M + 15) / 16) * C4 * (unsigned)G4 * 1024u
                                          : (unsigned)M * (unsigned)K * 4u);
    unsigned va[TM];
#pragma unroll
    for (int h = 0; h < TM; ++h)
        va[h] = PACKED ? (((unsigned)(m0 / 16 + h) * C4 + (unsigned)(cb / 4 + wave)) * (unsigned)G4) * 1024u
                             + (unsigned)lane * 16u
                       : ((unsigned)(m0 + 16 * h + i16) * (unsigned)K + (unsigned)(lane_c * R)) * 4u;
    // steps this lane's k slot stays inside the channel range of the split
    const int lane_steps = lane_c < ce ? (ce - lane_c + G::STEP_C - 1) / G::STEP_C : 0;

    constexpr int NB = G::NB;
    float ra[NS][TM][RC], rb[NS][NB];
    float rps[NS][PRE ? RC : 1], rpt[NS][PRE ? RC : 1];
    auto load_a = [&](int s, int step) {
        // offsets are below kOutside (a power of two), so or-ing it in moves them outside
        const unsigned outm = step < lane_steps ? 0u : kOutside;
        const unsigned sa = PACKED ? (unsigned)step * (unsigned)(4 * G4) * 1024u      // uniform
                                   : (unsigned)step * (unsigned)(G::STEP_C * R) * 4u;
        if (PACKED) {
#pragma unroll
            for (int h = 0; h < TM; ++h) {
                const unsigned oa = va[h] | outm;
#pragma unroll
                for (int q = 0; q < G4; ++q) {
                    if (R - 4 * q == 1) {
                        ra[s][h][4 * q] = __builtin_bit_cast(
                            float, __builtin_amdgcn_raw_buffer_load_b32(rs_ap, (int)(oa + 1024u * q), (int)sa, 0));
                    } else {
                        const f32x4 v = __builtin_bit_cast(
                            f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_ap, (int)(oa + 1024u * q), (int)sa, 0));
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (4 * q + e < RC) ra[s][h][4 * q + e] = v[e];
                    }
                }
            }
        } else
#pragma unroll
        for (int h = 0; h < TM; ++h) {
            const unsigned oa = va[h] | outm;
#pragma unroll
            for (int q = 0; q < RC / 4; ++q) {
                const f32x4 v = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, (int)(oa + 16u * q), (int)sa, 0));
                ra[s][h][4 * q] = v[0]; ra[s][h][4 * q + 1] = v[1];
                ra[s][h][4 * q + 2] = v[2]; ra[s][h][4 * q + 3] = v[3];
            }
#pragma unroll
            for (int q = RC / 4 * 4; q < RC; ++q)
                ra[s][h][q] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(rs_a, (int)(oa + 4u * q), (int)sa, 0));
        }
    };
    // The weights first -- the cold stream, and their offsets need nothing of the pixel
    // decode -- for all NS steps; the input offsets are worked out while those are on
    // their way.  (The waits the compiler places count loads in issue order, whatever it is.)
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        load_a(s, s);
        asm volatile("" ::: "memory");
    }
    unsigned vb[ROWS ? TN + 2 : TN][ROWS ? 1 : R];
    if (ROWS) {
        // one value per input row: column of this lane (lane 15: left of the segment)
        const int ix = i16 == 15 ? x0 - 1 : x0 + i16;
#pragma unroll
        for (int r = 0; r < TN + 2; ++r) {
            const int iy = y0 - 1 + r;
            const bool ok = (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
            vb[ROWS ? r : 0][0] = ok ? (unsigned)(iy * W + ix) * 4u + (unsigned)lane_c * HW4 : kOutside;
        }
    } else {
        const int kw_ = a[REEF_CONV_KW];
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            const int n = n0 + 16 * g + i16;
            const int oy = div_small(n, Wo), ox = n - oy * Wo;
#pragma unroll
            for (int t = 0; t < R; ++t) {
                const int ky = R == 1 ? 0 : div_small(t, kw_), kx = t - ky * kw_;
                const int iy = oy * a[REEF_CONV_SH] + ky - a[REEF_CONV_PH];
                const int ix = ox * a[REEF_CONV_SW] + kx - a[REEF_CONV_PW];
                const bool ok = n < N && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
                vb[ROWS ? 0 : g][ROWS ? 0 : t] = ok ? (unsigned)(iy * W + ix) * 4u + (unsigned)lane_c * HW4 : kOutside;
            }
        }
    }
    // operands that follow the optional epilogue operands: (pre-activation scale, shift), then
    // (workspace, arrival counters) of a folded split
    const int aux = ep_next + (PRE ? 2 : 0);
    const rsrc_t rs_ps = make_rsrc(d.ptr[PRE ? ep_next : 0], (unsigned)C * 4u);
    const rsrc_t rs_pt = make_rsrc(d.ptr[PRE ? ep_next + 1 : 0], (unsigned)C * 4u);
    const unsigned vpre = (unsigned)lane_c * 4u;

    auto load_b = [&](int s, int step) {
        const unsigned outm = step < lane_steps ? 0u : kOutside;
        const unsigned sb = (unsigned)step * (unsigned)G::STEP_C * HW4;         // uniform
        if (PRE) {
            const unsigned op = vpre | outm;
            const unsigned sp = (unsigned)step * (unsigned)G::STEP_C * 4u;   // uniform
#pragma unroll
            for (int q = 0; q < RC / 4; ++q) {
                const f32x4 sc = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_ps, (int)(op + 16u * q), (int)sp, 0));
                const f32x4 sh = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_pt, (int)(op + 16u * q), (int)sp, 0));
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    rps[s][PRE ? 4 * q + e : 0] = sc[e];
                    rpt[s][PRE ? 4 * q + e : 0] = sh[e];
                }
            }
        }
        if (ROWS) {
#pragma unroll
            for (int r = 0; r < NB; ++r)
                rb[s][r] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(rs_b, (int)(vb[ROWS ? r : 0][0] | outm), (int)sb, 0));
        } else {
#pragma unroll
            for (int g = 0; g < TN; ++g)
#pragma unroll
                for (int q = 0; q < RC; ++q) {
                    // R > 1: tap q of the slot's channel; R == 1: channel q of the slot
                    const unsigned ob = (R > 1 ? vb[ROWS ? 0 : g][ROWS ? 0 : q] : vb[ROWS ? 0 : g][0]) | outm;
                    const unsigned sq = R > 1 ? sb : sb + (unsigned)q * HW4;
                    rb[s][ROWS ? 0 : g * RC + q] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(rs_b, (int)ob, (int)sq, 0));
                }
        }
    };
    auto load_step = [&](int s, int step) {
        load_a(s, step);
        load_b(s, step);
    };
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        load_b(s, s);
        asm volatile("" ::: "memory");
    }

    // epilogue operands of this thread's output elements, behind the first K steps' loads
    ConvEpilogue ep;
    ep.next = 3;   // plain split-K launches carry no epilogue operands
    float e_bias[TM], e_sh2[TM], e_res[TM][TN];
#pragma unroll
    for (int h = 0; h < TM; ++h) {
        e_bias[h] = e_sh2[h] = 0.0f;
#pragma unroll
        for (int g = 0; g < TN; ++g) e_res[h][g] = 0.0f;
    }
    if (!to_ws) {
        ep.init(d, flags, a[REEF_CONV_ACT], a[REEF_CONV_ACT2], M, MN4, (unsigned)a[REEF_CONV_DST_OFF] * 4u);
#pragma unroll
        for (int h = 0; h < TM; ++h) {
            if (ep.has_bias) e_bias[h] = buf_load(ep.bias, om[h] * 4u);
            if (ep.has_dual) e_sh2[h] = buf_load(ep.shift2, om[h] * 4u);
            if (ep.has_res) {
#pragma unroll
                for (int g = 0; g < TN; ++g) e_res[h][g] = buf_load(ep.res, ooff[h][g]);
            }
        }
    }

    if (Poll::enabled) {
        // The flag check every best-effort workgroup makes before it does anything
        // (script/best_effort_kernel.py:22-29) is made here, with the first loads of the K loop
        // already on their way: its trip to memory hides behind theirs instead of standing in
        // front of them.  A workgroup that finds the flag raised has only read.
        if (threadIdx.x == 0) *sflag = poll.load();
        __syncthreads();
        if (*sflag) return false;
    }

    // Whole groups of NS steps with no condition inside (a loop with per-step conditions gets
    // reordered around the loads), then the remaining steps, whose loads are already under way.
    // Two accumulators per pixel group, so consecutive MFMAs never depend on each other.
    f32x4 acc[TM][TN][2];
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            acc[h][g][0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            acc[h][g][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    auto mma_stage = [&](int s) {
        if (ROWS) {
            // taps of input row r: the loaded value and its two neighbours within the 16-lane row
            float bt[NB][3];
#pragma unroll
            for (int r = 0; r < NB; ++r) {
                bt[r][0] = lane_from_left(rb[s][r]);
                bt[r][1] = rb[s][r];
                bt[r][2] = lane_from_right(rb[s][r]);
            }
#pragma unroll
            for (int q = 0; q < RC; ++q)
#pragma unroll
                for (int h = 0; h < TM; ++h)
#pragma unroll
                    for (int g = 0; g < TN; ++g)
                        acc[h][g][q & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            ra[s][h][q], bt[ROWS ? g + q / 3 : 0][q % 3], acc[h][g][q & 1], 0, 0, 0);
            return;
        }
        if (PRE) {
#pragma unroll
            for (int g = 0; g < TN; ++g)
#pragma unroll
                for (int q = 0; q < RC; ++q)
                    rb[s][ROWS ? 0 : g * RC + q] = fmaxf(fmaf(rb[s][ROWS ? 0 : g * RC + q], rps[s][PRE ? q : 0], rpt[s][PRE ? q : 0]), 0.0f);
        }
#pragma unroll
        for (int q = 0; q < RC; ++q)
#pragma unroll
            for (int h = 0; h < TM; ++h)
#pragma unroll
                for (int g = 0; g < TN; ++g)
                    acc[h][g][q & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[s][h][q], rb[s][ROWS ? 0 : g * RC + q],
                                                                            acc[h][g][q & 1], 0, 0, 0);
    };
    int pf = 0;
    int it = 0;
    bool left = false;
    // (groups whose refills all exist; the last whole group follows with the refills the remaining
    // steps need and no others: a load outside the buffer brings nothing but still takes its turn in
    // the vector-memory pipe, and a group of them cost a layer with nsteps == NS 1700 cycles)
    for (; it + 2 * NS <= nsteps; it += NS) {
        if (Poll::enabled) {
            // the flag is read one group ahead; a wavefront that sees it tells the others
            // through LDS and all of them leave after the barrier below
            if (pf) {
                *sflag = 1;
                left = true;
                break;
            }
            pf = poll.load();
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            mma_stage(s);
            load_step(s, it + s + NS);
            // keeps each step's refill behind its own MFMAs instead of at the end of the group
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (!left && it + NS <= nsteps) {
        if (Poll::enabled && pf) {
            *sflag = 1;
            left = true;
        } else {
            if (Poll::enabled) pf = poll.load();
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                mma_stage(s);
                if (it + s + NS < nsteps) load_step(s, it + s + NS);
                __builtin_amdgcn_sched_barrier(0);
            }
            it += NS;
        }
    }
    if (!left) {
#pragma unroll
        for (int s = 0; s < NS - 1; ++s)
            if (it + s < nsteps) mma_stage(s);
    }

    // partial tiles of this wavefront -> LDS; element j of a lane is row 4 * (lane / 16) + j.
    // Each group of four rows is skewed by 16 floats so the four k slots write to different banks.
    float* part = smem + wave * (TD::SUBS * TD::PART);
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                part[(h * TN + g) * TD::PART + (5 * kq + j) * 16 + i16] = acc[h][g][0][j] + acc[h][g][1][j];
    __syncthreads();
    if (Poll::enabled && *sflag) return false;
    const float* mine = smem + threadIdx.x + (threadIdx.x >> 6) * 16;
    constexpr int WSTRIDE = TD::SUBS * TD::PART;   // one wavefront's partial tiles
    float v[TM][TN];
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            const float* e = mine + (h * TN + g) * TD::PART;
            v[h][g] = ((e[0] + e[WSTRIDE]) + e[2 * WSTRIDE]) + e[3 * WSTRIDE];
        }
    if (to_ws) {
        const rsrc_t ws = make_rsrc((const float*)d.ptr[2] + (size_t)split * M * N, MN4);
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g) buf_store(ws, ooff[h][g], v[h][g]);
        return true;
    }
    if (!fused) {
        if (flags & REEF_F_GAP_OUTPUT) {
            // The global average of the layer's output instead of the output (a classifier's last
            // convolution): one pixel tile covers the image, so the 16 lanes of an output row hold
            // the whole row between them.  out[m] = sum over the pixels / N, pixels in ascending order
            // within a lane, lanes folded pairwise.
#pragma unroll
            for (int h = 0; h < TM; ++h) {
                float s = 0.0f;
#pragma unroll
                for (int g = 0; g < TN; ++g)
                    if (ooff[h][g] != kOutside) s += ep.value(v[h][g], om[h] * 4u, e_res[h][g], e_bias[h]);
#pragma unroll
                for (int o = 1; o < 16; o <<= 1) s += __shfl_xor(s, o, 64);
                if ((threadIdx.x & 15) == 0 && om[h] < (unsigned)M) buf_store(ep.out, om[h] * 4u, s * (1.0f / (float)N));
            }
            return true;
        }
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g)
                ep.finish(v[h][g], ooff[h][g], om[h] * 4u, e_res[h][g], e_bias[h], e_sh2[h]);
        return true;
    }

    // split-K folded inside the launch
    const size_t MN = (size_t)M * N;
    float* ws = (float*)d.ptr[aux];
    if (split_k == 2 && (flags & REEF_F_PAIR_FOLD) && poll.pair_fold_ok()) {
        // One exchange per output element.  A value is parked with its sign bit flipped: a sum
        // of products that starts from +0 is never -0, so a parked value is never the empty
        // slot's 0 (and a -0 is parked as +0, should one ever come).
        unsigned* slots = (unsigned*)(ws + 2 * MN);
        unsigned got[TM][TN];
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g) {
                got[h][g] = 0;
                if (ooff[h][g] != kOutside && om[h] < (unsigned)M) {
                    unsigned mine = __float_as_uint(v[h][g]) ^ 0x80000000u;
                    mine = mine ? mine : 0x80000000u;
                    got[h][g] = __hip_atomic_exchange(&slots[ooff[h][g] >> 2], mine, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g)
                if (got[h][g] != 0) {   // second to arrive: the other half is here
                    const float other = __uint_as_float(got[h][g] ^ 0x80000000u);
                    const float sum = split == 0 ? v[h][g] + other : other + v[h][g];   // split order
                    ep.finish(sum, ooff[h][g], om[h] * 4u, e_res[h][g], e_bias[h], e_sh2[h]);
                    __hip_atomic_store(&slots[ooff[h][g] >> 2], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        return true;
    }
    int* counters = (int*)d.ptr[aux + 1] + a[REEF_CONV_SYNC_OFF];
    int* s_last = sflag + 1;
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g)
            if (ooff[h][g] != kOutside && om[h] < (unsigned)M)
                store_agent(ws + (size_t)split * MN + (ooff[h][g] >> 2), v[h][g]);
    // every store of this workgroup has completed at device scope before it counts in
    partial_stores_done();
    __syncthreads();
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(&counters[rem], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_last = (old == split_k - 1);
    }
    __syncthreads();
    if (!*s_last) return true;
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            if (ooff[h][g] != kOutside && om[h] < (unsigned)M) {
                const float* src = ws + (ooff[h][g] >> 2);
                float sum = 0.0f;
                for (int s0 = 0; s0 < split_k; s0 += 4) {
                    float p[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) p[j] = load_agent(src + (size_t)min(s0 + j, split_k - 1) * MN);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (s0 + j < split_k) sum = (s0 + j == 0) ? p[j] : sum + p[j];
                }
                ep.finish(sum, ooff[h][g], om[h] * 4u, e_res[h][g], e_bias[h], e_sh2[h]);
            }
        }
    if (threadIdx.x == 0)  // ready for the next run
        __hip_atomic_store(&counters[rem], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// ---- reef_conv2d_xdw[2]_g<G>: 1x1 convolution, then depthwise 3x3, in one launch --------------
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ f32x2 buf_load2(rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_off, 0, 0));
}

// The front half of a MobileNetV2 block: expand (1x1 filter, + bias, activation) and the depthwise
// 3x3 filter (padding 1, stride S = 1 or 2, + bias, activation) that follows it.  As two launches
// the expanded tensor -- six times the block's input, the largest tensor of the network -- is
// written and read back; here it never leaves the chip.  The depthwise stage is channel-local, so
// a workgroup owns 16 channels x G image rows x one 14-column segment of the OUTPUT and needs the
// 1x1 result of the same 16 channels on the rows and columns its taps touch: it forms that
// itself.  The input has few channels (K = 16..160 for 96..960 expanded channels), so what
// neighbouring tiles compute twice is a fraction of a small product, and no workgroup waits for
// another.
//   phase 0  CK input channels at a time: the input patch into LDS as [pixel][channel] (every
//            value loaded once, by one thread), the tile's weight rows as [row][channel] (128-bit
//            loads), all loads of a thread on their way before its first store.
//            S = 1: pixel group r is image row y0 - 1 + r (G + 2 of them); lanes 0..13 of a group
//            are the segment's columns, lane 14 the column right of it, lane 15 the column left.
//            S = 2: input rows 2 y0 - 1 + r (2 G + 1 of them), each as two groups: the even
//            columns 2 x (lanes 0..13 = the segment's x) and the odd columns 2 x + 1 (lane 15:
//            column 2 x0 - 1, left of the segment).
//   phase 1  the 1x1 result on the matrix cores, both operands 128-bit LDS reads: k slot
//            (s, lane / 16) of a chunk's MFMAs stands for channel (lane / 16) * (chunk / 4) + s, so
//            what a lane multiplies is contiguous.  The wavefronts split the pixel groups, each
//            sums over all channels: nobody adds partial sums.  + bias, activation; positions
//            outside the image become 0 (the depthwise stage's padding) -> E in LDS.
//   phase 2  thread t = (channel t / 16, column t % 16) forms its G outputs from E: a value per
//            row (two for S = 2) from LDS, the neighbouring columns from the neighbouring lanes
//            (the sixteen threads of a channel are one row of lanes); taps in filter order, then
//            the bias, then the activation, as the depthwise kernel does.
// ptr: in [Cin][H][W], W [Cout][Cin], out [Cout][Ho][Wo], bias [Cout], depthwise weights [Cout][9],
// depthwise bias [Cout].  attr: H, W the input (and the 1x1 result), HO, WO the output, SH = SW =
// S (the 1x1 filter itself has stride 1), ACT the 1x1 layer's activation, ACT2 the depthwise
// stage's, flags REEF_F_BIAS | REEF_F_DW_OUTPUT, M_TILES = ceil(Cout / 16), N_TILES = ceil(Ho / G)
// * ceil(Wo / 14), no split.  tasks = M_TILES * N_TILES.
template <int G, int S = 1>
struct TileXdw {
    static constexpr int R = S == 1 ? G + 2 : 2 * G + 1;    // rows of the 1x1 result a tile needs
    static constexpr int NG = R * S;                         // pixel groups of 16 lanes: S per row
    static constexpr int GW = (NG + 3) / 4;                  // pixel groups per wavefront at most
    // input channels staged at a time: what the network's layers of the tile's kind have
    static constexpr int CK = S == 2 ? 96 : G == 4 ? 64 : 160;
    static constexpr int PS = CK + 4;                        // floats per pixel of the patch and per weight row (4 mod 32: banks)
    // floats per channel of E [channel][pixel]: 20 mod 32, so that the 4 x 16 values a wavefront writes
    // (channels 4 apart) and the 4 x 16 it reads (consecutive channels) each meet every bank twice
    static constexpr int ESTRIDE = NG * 16 + (NG % 2 == 0 ? 20 : 4);
    static constexpr int O_W = NG * 16 * PS, O_E = O_W + 16 * PS;
    static constexpr int LDS_BYTES = (O_E + 16 * ESTRIDE) * 4 + 16;
    static_assert(CK % 16 == 0 && PS % 32 == 4, "chunks are whole 16-channel steps");
};

template <int G, int S, class Poll>
__device__ __forceinline__ bool conv2d_xdw_body(const ReefOpDesc& d, int task, char* smem_raw, const Poll&) {
    typedef TileXdw<G, S> T;
    constexpr int R = T::R, NG = T::NG, GW = T::GW, JM = T::CK / 16;
    float* smem = (float*)smem_raw;
    float* Wl = smem + T::O_W;
    float* E = smem + T::O_E;
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, i16 = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int C = a[REEF_CONV_CIN], H = a[REEF_CONV_H], W = a[REEF_CONV_W], M = a[REEF_CONV_COUT];
    const int Ho = a[REEF_CONV_HO], Wo = a[REEF_CONV_WO];
    const int m_tiles = a[REEF_CONV_M_TILES], n_tiles = a[REEF_CONV_N_TILES];
    // the tiles of one pixel tile (all channel tiles) are neighbours in the order: they read the
    // same input, and a contiguous piece of the order runs on one XCD
    task = xcd_chunked(task, m_tiles * n_tiles);
    const int nt = div_small(task, m_tiles), mt = task - nt * m_tiles;
    const int segs = (Wo + kRowSeg - 1) / kRowSeg;
    const int q_seg = div_small(nt, segs);
    const int y0 = q_seg * G, x0 = (nt - q_seg * segs) * kRowSeg;     // first output row and column
    const int m0 = mt * 16;
    const int HW = H * W;

    // roles: phase 0 thread = (channel or weight row t / 16, column t % 16); phase 2 the same
    const int row = threadIdx.x >> 4, col = threadIdx.x & 15;
    const unsigned ch = (unsigned)(m0 + row);
    const rsrc_t rs_a = make_rsrc(d.ptr[1], (unsigned)M * (unsigned)C * 4u);
    const rsrc_t rs_b = make_rsrc(d.ptr[0], (unsigned)C * (unsigned)HW * 4u);
    const rsrc_t rs_bias = make_rsrc(d.ptr[3], (unsigned)M * 4u);
    const rsrc_t rs_dw = make_rsrc(d.ptr[4], (unsigned)M * 36u);
    const rsrc_t rs_db = make_rsrc(d.ptr[5], (unsigned)M * 4u);

    // Image column that lane / column c of pixel group (r, p) stands for.  S = 1: the segment's
    // columns, lane 14 right of it, lane 15 left of it.  S = 2, p = 0: even columns 2 x; p = 1:
    // odd columns 2 x + 1, lane 15 the odd column left of the segment; lanes nobody reads: none.
    auto image_col = [&](int c, int p) -> int {
        if (S == 1) return c == 15 ? x0 - 1 : x0 + c;
        if (p == 0) return c < kRowSeg ? 2 * (x0 + c) : -1;
        return c == 15 ? 2 * x0 - 1 : c < kRowSeg ? 2 * (x0 + c) + 1 : -1;
    };
    // activation without a branch per element: clamp to [0, hi], or the value itself
    auto activate = [](float v, int act) -> float {
        const float hi = act == REEF_ACT_RELU6 ? 6.0f : __builtin_inff();
        const float c = fminf(fmaxf(v, 0.0f), hi);
        return act == REEF_ACT_NONE ? v : c;
    };

    // what the later phases need from memory, on its way from the start
    float wdw[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) wdw[t] = buf_load(rs_dw, ch * 36u + 4u * t);
    const float bdw = buf_load(rs_db, ch * 4u);
    float bexs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) bexs[j] = buf_load(rs_bias, (unsigned)(m0 + 4 * kq + j) * 4u);

    // the wavefront's pixel groups (one that does not exist: the last one again, result dropped)
    int gcl[GW];
#pragma unroll
    for (int u = 0; u < GW; ++u) gcl[u] = min(wave + 4 * u, NG - 1);
    f32x4 acc[GW][4];
#pragma unroll
    for (int u = 0; u < GW; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[u][e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    for (int c0 = 0; c0 < C; c0 += T::CK) {
        const int nq = (min(C - c0, T::CK) + 15) >> 4;          // 16-channel steps of this chunk
        if (c0 > 0) __syncthreads();                            // the previous chunk has been multiplied
        // ---- phase 0
        {
            float v[JM][NG];
            f32x4 vw[(JM + 3) / 4];
#pragma unroll
            for (int i = 0; i < (JM + 3) / 4; ++i) {
                const int c = c0 + 4 * col + 64 * i;
                const bool ok = 4 * col + 64 * i < 16 * nq && c < C && ch < (unsigned)M;
                vw[i] = buf_load4(rs_a, ok ? (ch * (unsigned)C + (unsigned)c) * 4u : kOutside);
            }
#pragma unroll
            for (int j = 0; j < JM; ++j) {
                if (j < nq) {
                    const int c = c0 + row + 16 * j;
                    const bool c_ok = c < C;
                    const unsigned cbase = (unsigned)(c * HW) * 4u;
                    if (S == 2 && !(W & 1)) {
                        // an even column and the odd one right of it in one 64-bit load; lane 15 fetches
                        // the pair left of the segment for its odd column, lane 14 has nothing to fetch
#pragma unroll
                        for (int r = 0; r < R; ++r) {
                            const int iy = y0 * S - 1 + r, ix = col == 15 ? 2 * x0 - 2 : 2 * (x0 + col);
                            const bool ok = c_ok && col != 14 && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
                            const f32x2 p2 = buf_load2(rs_b, ok ? cbase + (unsigned)(iy * W + ix) * 4u : kOutside);
                            v[j][2 * r] = col < kRowSeg ? p2[0] : 0.0f;
                            v[j][2 * r + 1] = p2[1];
                        }
                    } else {
#pragma unroll
                        for (int g = 0; g < NG; ++g) {
                            const int r = g / S, p = g % S;
                            const int iy = y0 * S - 1 + r, ix = image_col(col, p);
                            const bool ok = c_ok && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
                            v[j][g] = buf_load(rs_b, ok ? cbase + (unsigned)(iy * W + ix) * 4u : kOutside);
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < (JM + 3) / 4; ++i)
                if (4 * col + 64 * i < 16 * nq) *(f32x4*)(Wl + row * T::PS + 4 * col + 64 * i) = vw[i];
#pragma unroll
            for (int j = 0; j < JM; ++j) {
                if (j < nq) {
#pragma unroll
                    for (int g = 0; g < NG; ++g) smem[(g * 16 + col) * T::PS + row + 16 * j] = v[j][g];
                }
            }
        }
        __syncthreads();

        // ---- phase 1: the chunk's MFMAs, the operands of step q + 1 read while step q multiplies
        {
            const float* wa = Wl + i16 * T::PS + kq * 4 * nq;
            const float* pb[GW];
#pragma unroll
            for (int u = 0; u < GW; ++u) pb[u] = smem + (gcl[u] * 16 + i16) * T::PS + kq * 4 * nq;
            f32x4 a_cur = *(const f32x4*)wa, b_cur[GW];
#pragma unroll
            for (int u = 0; u < GW; ++u) b_cur[u] = *(const f32x4*)pb[u];
            for (int q = 0; q < nq; ++q) {
                const int qn = min(q + 1, nq - 1);
                const f32x4 a_nxt = *(const f32x4*)(wa + 4 * qn);
                f32x4 b_nxt[GW];
#pragma unroll
                for (int u = 0; u < GW; ++u) b_nxt[u] = *(const f32x4*)(pb[u] + 4 * qn);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int u = 0; u < GW; ++u)
                        acc[u][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[e], b_cur[u][e], acc[u][e], 0, 0, 0);
                a_cur = a_nxt;
#pragma unroll
                for (int u = 0; u < GW; ++u) b_cur[u] = b_nxt[u];
            }
        }
    }

    // + bias, activation, 0 outside the image -> E
    const int act = a[REEF_CONV_ACT], act2 = a[REEF_CONV_ACT2];
#pragma unroll
    for (int u = 0; u < GW; ++u) {
        const int g = wave + 4 * u;
        if (g < NG) {
            const int r = g / S, p = g - r * S;
            const int my = y0 * S - 1 + r, mx = image_col(i16, p);
            const bool inside = (unsigned)my < (unsigned)H && (unsigned)mx < (unsigned)W;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float v = activate(((acc[u][0][j] + acc[u][1][j]) + (acc[u][2][j] + acc[u][3][j])) + bexs[j], act);
                E[(4 * kq + j) * T::ESTRIDE + g * 16 + i16] = inside ? v : 0.0f;
            }
        }
    }
    __syncthreads();

    // ---- phase 2: the depthwise stage from E
    const rsrc_t rs_o = make_rsrc(d.ptr[2], (unsigned)M * (unsigned)(Ho * Wo) * 4u);
    const float* Ec = E + row * T::ESTRIDE;
    float e[R][3];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        if (S == 1) {
            e[rr][1] = Ec[rr * 16 + col];
        } else {
            e[rr][1] = Ec[(2 * rr) * 16 + col];         // 2 x
            e[rr][2] = Ec[(2 * rr + 1) * 16 + col];     // 2 x + 1
        }
    }
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        if (S == 1) {
            e[rr][0] = lane_from_left(e[rr][1]);
            e[rr][2] = lane_from_right(e[rr][1]);
        } else {
            e[rr][0] = lane_from_left(e[rr][2]);        // the odd column left of 2 x
        }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float s = 0.0f;
#pragma unroll
        for (int t = 0; t < 9; ++t) s = fmaf(e[S * g + t / 3][t % 3], wdw[t], s);
        const bool ok = col < kRowSeg && x0 + col < Wo && y0 + g < Ho && ch < (unsigned)M;
        buf_store(rs_o, ok ? (ch * (unsigned)(Ho * Wo) + (unsigned)((y0 + g) * Wo + x0 + col)) * 4u : kOutside,
                  activate(s + bdw, act2));
    }
    return true;
}

// ---- reef_conv2d_sdp_g<G> / reef_conv2d_xdp2_g<G>: a whole MobileNetV2 block in one launch -------
// front filter (+ bias, activation) -> depthwise 3x3 filter (padding 1, + bias, activation) -> 1x1
// projection (+ bias, linear), for the blocks at the head of the network, whose images are large
// and whose channels are few: every tensor between the three layers is several times the block's
// input or output (32 and 96 channels at 112 x 112 against 3 in and 16 or 24 out), and with so
// few channels a workgroup can hold ALL of them for its pixels.  A workgroup owns G output rows x
// one 14-column segment x every channel; nothing is split, nobody waits for anybody.
//   STEM   the front filter is the network's first layer: 3x3, stride 2, padding 1 on at most 3
//          channels (K = 27: what neighbouring tiles compute twice costs nothing); the depthwise
//          stage has stride 1.
//   !STEM  the front filter is a 1x1 expansion of at most 4 KC channels; the depthwise stage has
//          stride S.
//   phase 0  the input patch and the parameters of the first two layers into LDS, all loads of a
//            thread on their way before its first store (zero where the image or a channel ends).
//   phase 1  the front filter on the matrix cores, operands from LDS; pixel groups as in
//            reef_conv2d_xdw (S = 1: group r = row y0 - 1 + r of the front filter's result, lanes
//            0..13 the segment's columns, lane 14 the column right of it, lane 15 the one left;
//            S = 2: rows 2 y0 - 1 + r as an even-column and an odd-column group).  + bias,
//            activation, 0 outside the image (the depthwise padding) -> E in LDS.  The wavefronts
//            share the (channel tile, pixel group) pairs.
//   phase 2  thread (channel, column) forms the depthwise outputs of its G rows, a channel tile
//            at a time, taps in filter order, then bias and activation -> D in LDS.
//   phase 3  the projection on the matrix cores from D, its weights waiting in registers since the
//            kernel's start, + bias, store.
// ptr: in [Cin][H][W], front weights [Cmid][Cin][KH][KW], out [P][Ho][Wo], front bias [Cmid],
// depthwise weights [Cmid][9], depthwise bias [Cmid], projection weights [P][Cmid], projection
// bias [P].  attr: COUT = Cmid (<= 16 MT), REEF_CONV_PROJ = P (<= 32); H, W the input; HO, WO the
// output; KH = KW = 3, SH = SW = 2, PH = PW = 1 (STEM: the front filter's) or KH = KW = 1, SH = SW
// = S, PH = PW = 0 (the depthwise stride, as for reef_conv2d_xdw); ACT, ACT2 the front filter's
// and the depthwise stage's activation; flags REEF_F_BIAS | REEF_F_DW_OUTPUT | REEF_F_PROJ_OUTPUT;
// M_TILES = 1, N_TILES = ceil(Ho / G) * ceil(Wo / 14) = tasks.
template <int G, int S, bool STEM, int MT, int KC>
struct TileBlk {
    static constexpr int R = S == 1 ? G + 2 : 2 * G + 1;    // rows of the front filter's result a tile needs
    static constexpr int NG = R * S;                         // pixel groups of 16 lanes: S per row
    static constexpr int CM = MT * 16, CP = 32;              // most middle channels, most output channels
    // k slot (s, lane / 16) of an MFMA stands for tap resp. channel (lane / 16) * KF + s in phase 1 and
    // for channel (lane / 16) * KP + s in phase 3: what a lane multiplies is contiguous in memory
    static constexpr int KF = STEM ? 7 : KC, KP = MT * 4;
    static constexpr int WFS = STEM ? 36 : 4 * KC + 4;       // floats per channel of the front weights ([lane / 16][KF], 4 mod 32: banks)
    static constexpr int PR = 2 * R + 1, PCS = 36;           // STEM: patch rows per channel, row stride (33 columns)
    static constexpr int PS = 4 * KC + 4;                    // !STEM: floats per pixel of the input patch [pixel][channel]
    static constexpr int PATCH = STEM ? 3 * PR * PCS : NG * 16 * PS;
    // floats per channel of E [channel][pixel]: 20 mod 32, so that the 4 x 16 values a wavefront writes
    // (channels 4 apart) and the 4 x 16 it reads (consecutive channels) each meet every bank twice
    static constexpr int ESTRIDE = NG * 16 + (NG % 2 == 0 ? 20 : 4);
    static constexpr int DPS = CM + 4;                       // floats per pixel of D [pixel][channel]
    static constexpr int MH = MT / 2, GH = NG / 2;           // phase 1: a wavefront's channel tiles x pixel groups
    // LDS map (floats; every block starts on 16 bytes)
    static constexpr int O_WF = PATCH, O_BF = O_WF + CM * WFS, O_WD = O_BF + CM, O_BD = O_WD + CM * 9;
    static constexpr int O_BP = O_BD + CM, O_E = O_BP + CP, O_D = O_E + CM * ESTRIDE;
    static constexpr int FLOATS = O_D + G * 16 * DPS;
    static constexpr int LDS_BYTES = FLOATS * 4 + 16;
    static_assert(MT % 2 == 0 && NG % 2 == 0, "the wavefronts share phase 1 as 2 x 2 rectangles");
    static_assert(STEM || (KC == 4 && S == 2), "the expansion form: sixteen input channels, depthwise stride 2");
    static_assert(MT % 2 == 0 && CM * 9 / 4 <= kThreads && CM <= kThreads, "phase 0 and 2 take the channels in these steps");
};

// One segment of phase 0: COUNT floats of LDS at dst, float i from byte offset src(i) of the
// buffer (kOutside: 0).  Loads first, stores second.
template <int COUNT, class F>
__device__ __forceinline__ void blk_stage_load(float (&v)[(COUNT + kThreads - 1) / kThreads], const rsrc_t& rs, F src) {
#pragma unroll
    for (int i = 0; i < (COUNT + kThreads - 1) / kThreads; ++i) {
        const int idx = (int)threadIdx.x + kThreads * i;
        v[i] = buf_load(rs, idx < COUNT ? src(idx) : kOutside);
    }
}
template <int COUNT>
__device__ __forceinline__ void blk_stage_store(const float (&v)[(COUNT + kThreads - 1) / kThreads], float* dst) {
#pragma unroll
    for (int i = 0; i < (COUNT + kThreads - 1) / kThreads; ++i) {
        const int idx = (int)threadIdx.x + kThreads * i;
        if (idx < COUNT) dst[idx] = v[i];
    }
}

template <int G, int S, bool STEM, int MT, int KC, class Poll>
__device__ __forceinline__ bool conv2d_block_body(const ReefOpDesc& d, int task, char* smem_raw, const Poll&) {
    typedef TileBlk<G, S, STEM, MT, KC> T;
    constexpr int R = T::R, NG = T::NG, KF = T::KF, KP = T::KP;
    static_assert(!STEM || S == 1, "the stem form has a stride-1 depthwise stage");
    float* smem = (float*)smem_raw;
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, i16 = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int C = a[REEF_CONV_CIN], H = a[REEF_CONV_H], W = a[REEF_CONV_W], M = a[REEF_CONV_COUT];
    const int Ho = a[REEF_CONV_HO], Wo = a[REEF_CONV_WO], P = a[REEF_CONV_PROJ];
    const int Hm = STEM ? Ho : H, Wm = STEM ? Wo : W;            // the front filter's result
    task = xcd_chunked(task, a[REEF_CONV_N_TILES]);
    const int segs = (Wo + kRowSeg - 1) / kRowSeg;
    const int q_seg = div_small(task, segs);
    const int y0 = q_seg * G, x0 = (task - q_seg * segs) * kRowSeg;     // first output row and column

    // column of the front filter's result that lane / column c of pixel group (r, p) stands for
    auto image_col = [&](int c, int p) -> int {
        if (S == 1) return c == 15 ? x0 - 1 : x0 + c;
        if (p == 0) return c < kRowSeg ? 2 * (x0 + c) : -1;
        return c == 15 ? 2 * x0 - 1 : c < kRowSeg ? 2 * (x0 + c) + 1 : -1;
    };
    // activation without a branch per element: clamp to [0, hi], or the value itself
    auto activate = [](float v, int act) -> float {
        const float hi = act == REEF_ACT_RELU6 ? 6.0f : __builtin_inff();
        const float c = fminf(fmaxf(v, 0.0f), hi);
        return act == REEF_ACT_NONE ? v : c;
    };

    // The projection's weights go from memory straight into the registers of the wavefront that
    // multiplies with them (row i16 of output tile pt, channels kq KP .. + KP - 1: 128-bit loads; the
    // channel count is a multiple of 4), on their way from the first instruction on: phase 3 is the
    // last to need anything.
    const int npairs3 = ((P + 15) >> 4) * G;
    const rsrc_t rs_wp = make_rsrc(d.ptr[6], (unsigned)P * (unsigned)M * 4u);
    f32x4 wp[KP / 4];
    auto load_wp = [&](int pr) {
        const unsigned prow = (unsigned)((pr / G) * 16 + i16);
#pragma unroll
        for (int q = 0; q < KP / 4; ++q) {
            const int ch0 = kq * KP + 4 * q;
            wp[q] = buf_load4(rs_wp, (prow < (unsigned)P && ch0 < M) ? (prow * (unsigned)M + (unsigned)ch0) * 4u : kOutside);
        }
    };
    if (wave < npairs3) load_wp(wave);

    // ---- phase 0.  Channels, rows and columns that do not exist are staged as zeros, so the phases
    // below run over the compiled sizes whatever the layer's.
    {
        const rsrc_t rs_in = make_rsrc(d.ptr[0], (unsigned)C * (unsigned)(H * W) * 4u);
        const rsrc_t rs_wf = make_rsrc(d.ptr[1], (unsigned)M * (unsigned)C * (STEM ? 36u : 4u));
        const rsrc_t rs_bf = make_rsrc(d.ptr[3], (unsigned)M * 4u);
        const rsrc_t rs_wd = make_rsrc(d.ptr[4], (unsigned)M * 36u);
        const rsrc_t rs_bd = make_rsrc(d.ptr[5], (unsigned)M * 4u);
        const rsrc_t rs_bp = make_rsrc(d.ptr[7], (unsigned)P * 4u);
        const int t = (int)threadIdx.x;
        // depthwise weights: a copy, four floats a thread; the three bias vectors
        const f32x4 v_wd = buf_load4(rs_wd, t < T::CM * 9 / 4 ? (unsigned)t * 16u : kOutside);
        const float v_bf = buf_load(rs_bf, t < T::CM ? (unsigned)t * 4u : kOutside);
        const float v_bd = buf_load(rs_bd, t < T::CM ? (unsigned)t * 4u : kOutside);
        const float v_bp = buf_load(rs_bp, t < T::CP ? (unsigned)t * 4u : kOutside);
        if constexpr (STEM) {
            constexpr int N_WF = T::CM * T::WFS;
            float v_in[(T::PATCH + kThreads - 1) / kThreads], v_wf[(N_WF + kThreads - 1) / kThreads];
            const int iy0 = 2 * y0 - 3, ix0 = 2 * x0 - 3;            // the patch's first input row and column
            const int K = 9 * C;
            blk_stage_load<T::PATCH>(v_in, rs_in, [&](int idx) -> unsigned {
                const int c = idx / (T::PR * T::PCS), rem = idx - c * (T::PR * T::PCS);
                const int row = rem / T::PCS, colp = rem - row * T::PCS;
                const int iy = iy0 + row, ix = ix0 + colp;
                const bool ok = c < C && colp < 33 && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
                return ok ? (unsigned)(c * H * W + iy * W + ix) * 4u : kOutside;
            });
            blk_stage_load<N_WF>(v_wf, rs_wf, [&](int idx) -> unsigned {
                // [middle channel][lane / 16][8]: tap (lane / 16) * 7 + s of the 9 Cin, s < 7
                const int m = idx / T::WFS, q = idx - m * T::WFS;
                const int k = (q >> 3) * KF + (q & 7);
                const bool ok = m < M && q < 32 && (q & 7) < KF && k < K;
                return ok ? (unsigned)(m * K + k) * 4u : kOutside;
            });
            blk_stage_store<T::PATCH>(v_in, smem);
            blk_stage_store<N_WF>(v_wf, smem + T::O_WF);
        } else {
            // the patch: thread = (input channel, column); a 64-bit load brings an even column and
            // the odd one right of it (W is even).  Lane 15 fetches the pair left of the segment
            // for its odd column; lane 14 has nothing to fetch.
            const int c = t >> 4, l = t & 15;
            f32x2 v_in[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int iy = y0 * S - 1 + r, ix = l == 15 ? 2 * x0 - 2 : 2 * (x0 + l);
                const bool ok = c < C && l != 14 && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
                v_in[r] = buf_load2(rs_in, ok ? (unsigned)(c * H * W + iy * W + ix) * 4u : kOutside);
            }
            // the front weights: thread = (middle channel of 64, four input channels), 128-bit loads
            constexpr int NWF = (T::CM + 63) / 64;
            f32x4 v_wf[NWF];
#pragma unroll
            for (int i = 0; i < NWF; ++i) {
                const int m = (t >> 2) + 64 * i, k0 = 4 * (t & 3);
                v_wf[i] = buf_load4(rs_wf, (m < M && k0 < C) ? (unsigned)(m * C + k0) * 4u : kOutside);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                smem[((2 * r) * 16 + l) * T::PS + c] = l < kRowSeg ? v_in[r][0] : 0.0f;
                smem[((2 * r + 1) * 16 + l) * T::PS + c] = v_in[r][1];
            }
#pragma unroll
            for (int i = 0; i < NWF; ++i) {
                const int m = (t >> 2) + 64 * i;
                if (m < T::CM) *(f32x4*)(smem + T::O_WF + m * T::WFS + 4 * (t & 3)) = v_wf[i];
            }
        }
        if (t < T::CM * 9 / 4) *(f32x4*)(smem + T::O_WD + 4 * t) = v_wd;
        if (t < T::CM) { smem[T::O_BF + t] = v_bf; smem[T::O_BD + t] = v_bd; }
        if (t < T::CP) smem[T::O_BP + t] = v_bp;
    }
    __syncthreads();

    // ---- phase 1: E = act(front filter + bias), 0 outside the image
    const int act = a[REEF_CONV_ACT], act2 = a[REEF_CONV_ACT2];
    float* E = smem + T::O_E;
    int poff[STEM ? KF : 1];       // STEM: where tap kq * 7 + s sits in the patch, relative to tap 0
    if constexpr (STEM) {
#pragma unroll
        for (int s = 0; s < KF; ++s) {
            const int k = min(kq * KF + s, 26);      // (the 28th tap does not exist: its weight is 0)
            const int c = k / 9, ky = (k - 9 * c) / 3, kx = k - 9 * c - 3 * ky;
            poff[s] = (c * T::PR + ky) * T::PCS + kx;
        }
    }
    {
        // a wavefront takes MH channel tiles x GH pixel groups: every operand read once, then per
        // channel tile the MFMAs of its GH groups (2 GH independent sums) and their results
        const int mtb = (wave & 1) * T::MH, gb = (wave >> 1) * T::GH;
        float ra[T::MH][STEM ? 8 : KF], rb[T::GH][KF];
        f32x4 bias[T::MH];
#pragma unroll
        for (int m = 0; m < T::MH; ++m) {
            const float* wa = smem + T::O_WF + ((mtb + m) * 16 + i16) * T::WFS + kq * (STEM ? 8 : KF);
            const f32x4 w0 = *(const f32x4*)wa;
#pragma unroll
            for (int e = 0; e < 4; ++e) ra[m][e] = w0[e];
            if constexpr (STEM) {
                const f32x4 w1 = *(const f32x4*)(wa + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) ra[m][4 + e] = w1[e];
            }
            bias[m] = *(const f32x4*)(smem + T::O_BF + (mtb + m) * 16 + 4 * kq);
        }
#pragma unroll
        for (int b = 0; b < T::GH; ++b) {
            const int g = gb + b;
            if constexpr (STEM) {
                // the lane's column of the result is patch column 2 ((i16 + 1) mod 16) of filter column 0
                const float* pb = smem + 2 * g * T::PCS + 2 * ((i16 + 1) & 15);
#pragma unroll
                for (int s = 0; s < KF; ++s) rb[b][s] = pb[poff[s]];
            } else {
                const f32x4 b0 = *(const f32x4*)(smem + (g * 16 + i16) * T::PS + 4 * kq);
#pragma unroll
                for (int e = 0; e < 4; ++e) rb[b][e] = b0[e];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < T::MH; ++m) {
            f32x4 acc[T::GH][2];
#pragma unroll
            for (int b = 0; b < T::GH; ++b) acc[b][0] = acc[b][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int s = 0; s < KF; ++s)
#pragma unroll
                for (int b = 0; b < T::GH; ++b)
                    acc[b][s & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[m][s], rb[b][s], acc[b][s & 1], 0, 0, 0);
#pragma unroll
            for (int b = 0; b < T::GH; ++b) {
                const int g = gb + b, r = g / S, p = g - r * S;
                const int my = y0 * S - 1 + r, mx = image_col(i16, p);
                const bool inside = (unsigned)my < (unsigned)Hm && (unsigned)mx < (unsigned)Wm;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float v = activate((acc[b][0][j] + acc[b][1][j]) + bias[m][j], act);
                    E[((mtb + m) * 16 + 4 * kq + j) * T::ESTRIDE + g * 16 + i16] = inside ? v : 0.0f;
                }
            }
        }
    }
    __syncthreads();

    // ---- phase 2: D = act2(depthwise(E) + bias), two channel tiles at a time: every value a thread
    // needs read once, then its outputs formed, then stored
    float* D = smem + T::O_D;
    {
        const int row = threadIdx.x >> 4, col = threadIdx.x & 15;
#pragma unroll
        for (int mt0 = 0; mt0 < MT; mt0 += 2) {
            float wdw[2][9], bdw[2], e[2][R][3];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int ch = (mt0 + h) * 16 + row;
#pragma unroll
                for (int tp = 0; tp < 9; ++tp) wdw[h][tp] = smem[T::O_WD + ch * 9 + tp];
                bdw[h] = smem[T::O_BD + ch];
                const float* Ec = E + ch * T::ESTRIDE;
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    // the sixteen threads of a channel are one row of lanes: neighbours come from there
                    if (S == 1) {
                        e[h][rr][1] = Ec[rr * 16 + col];
                    } else {
                        e[h][rr][1] = Ec[(2 * rr) * 16 + col];         // 2 x
                        e[h][rr][2] = Ec[(2 * rr + 1) * 16 + col];     // 2 x + 1
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    if (S == 1) {
                        e[h][rr][0] = lane_from_left(e[h][rr][1]);
                        e[h][rr][2] = lane_from_right(e[h][rr][1]);
                    } else {
                        e[h][rr][0] = lane_from_left(e[h][rr][2]);     // the odd column left of 2 x
                    }
                }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int ch = (mt0 + h) * 16 + row;
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    float s = 0.0f;
#pragma unroll
                    for (int tp = 0; tp < 9; ++tp) s = fmaf(e[h][S * g + tp / 3][tp % 3], wdw[h][tp], s);
                    D[(g * 16 + col) * T::DPS + ch] = activate(s + bdw[h], act2);
                }
            }
        }
    }
    __syncthreads();

    // ---- phase 3: out = projection(D) + bias
    const rsrc_t rs_o = make_rsrc(d.ptr[2], (unsigned)P * (unsigned)(Ho * Wo) * 4u);
    for (int pr = wave; pr < npairs3; pr += 4) {
        if (pr != wave) load_wp(pr);
        const int pt = pr / G, g = pr - pt * G;
        const float* db = D + (g * 16 + i16) * T::DPS + kq * KP;
        f32x4 rb[KP / 4];
#pragma unroll
        for (int q = 0; q < KP / 4; ++q) rb[q] = *(const f32x4*)(db + 4 * q);
        const f32x4 bias = *(const f32x4*)(smem + T::O_BP + pt * 16 + 4 * kq);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 acc[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[q] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int q = 0; q < KP / 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(wp[q][e], rb[q][e], acc[e], 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int ch = pt * 16 + 4 * kq + j;
            const bool ok = i16 < kRowSeg && x0 + i16 < Wo && y0 + g < Ho && ch < P;
            buf_store(rs_o, ok ? ((unsigned)ch * (unsigned)(Ho * Wo) + (unsigned)((y0 + g) * Wo + x0 + i16)) * 4u : kOutside,
                      ((acc[0][j] + acc[1][j]) + (acc[2][j] + acc[3][j])) + bias[j]);
        }
    }
    return true;
}

// ---- reef_conv2d_sp7_g2: the stem of a ResNet / DenseNet in one launch ------------------------
// in (+ a per-channel shift) -> 7x7 convolution, stride 2, padding 3, + bias, activation ->
// 3x3 max-pool, stride 2, padding 1 (+ a per-channel shift, activation).  As launches of their own
// the three are 3.5 + 16.6 + 4.3 us on a 224 x 224 image, and the 64 x 112 x 112 tensor between
// convolution and pool (3.2 MB) is written to be read once.  The convolution has K = 147: cheap to
// compute again, and the pool is local to a channel -- the case of reef_conv2d_xdw: a workgroup
// owns 16 channels x 2 pooled rows x 14 pooled columns and forms the 5 x 29 convolution results
// its windows touch itself (1.3 x the convolution's work in total); no workgroup waits for another.
//   phase 0  the 15 x 63 input patch of every channel into LDS (zero outside the image: the
//            convolution's padding; the input shift applies inside the image only, as it does
//            when the shift is a launch of its own in front of a zero-padding convolution).
//   phase 1  the convolution on the matrix cores: pixel group (r, c) is convolution row
//            2 py0 - 1 + r and columns 2 px0 - 1 + 16 c + lane.  The taps are taken in the order
//            (channel, ky, kx) with kx counted to 8 (the eighth weight is 0): MFMA s of a group
//            covers filter row s / 2 and taps kx = 4 (s % 2) + lane / 16, so the weight's and the
//            patch value's addresses are the lane's base plus a constant of s -- no index
//            arithmetic, nothing to keep in registers.
//            The wavefronts split the ten groups, so nobody adds partial sums.  + bias,
//            activation; a position outside the convolution's output counts as -FLT_MAX (the
//            pool's padding) -> E in LDS.
//   phase 2  thread (channel, pooled column) takes the maximum of its 3 x 3 windows for the two
//            pooled rows, adds the pool's shift, applies its activation, stores.
// ptr: in [Cin][H][W] (Cin <= 3), W [Cout][Cin][7][7], out [Cout][Ho][Wo] (pooled), bias [Cout],
// then the input shift [Cin] (REEF_F_IN_SHIFT) and the pool's shift [Cout] (REEF_F_POOL_SHIFT).
// attr: H, W of the input; Ho, Wo of the POOLED output; M_TILES = ceil(Cout / 16),
// N_TILES = ceil(Ho / 2) * ceil(Wo / 14); ACT the convolution's, ACT2 the pool's activation.
struct TileSp7 {
    static constexpr int G = 2, CR = 2 * G + 1, NG = 2 * CR;       // pooled rows; convolution rows; pixel groups
    static constexpr int PR = 2 * CR + 5, PC = 64, CMAX = 3;       // patch rows, row stride, channels
    static constexpr int STEPS = CMAX * 7 * 2;                     // 42 MFMAs per group: two per filter row
    static constexpr int ESTRIDE = CR * 32 + 1;                    // floats per channel of E
    static constexpr int PATCH = CMAX * PR * PC, EFLOATS = 16 * ESTRIDE + 32;
    static constexpr int WFLOATS = 16 * CMAX * 49;                 // the tile's weight rows
    static constexpr int LDS_BYTES = (PATCH + EFLOATS + WFLOATS) * 4 + 16;
};

template <class Poll>
__device__ __forceinline__ bool conv2d_stem_pool_body(const ReefOpDesc& d, int task, char* smem_raw, const Poll&) {
    typedef TileSp7 T;
    float* patch = (float*)smem_raw;
    float* E = patch + T::PATCH;
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, i16 = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int C = a[REEF_CONV_CIN], H = a[REEF_CONV_H], W = a[REEF_CONV_W], M = a[REEF_CONV_COUT];
    const int Ho = a[REEF_CONV_HO], Wo = a[REEF_CONV_WO];
    const int Hc = (H - 1) / 2 + 1, Wc = (W - 1) / 2 + 1;          // the convolution's output: (H + 6 - 7) / 2 + 1
    const int flags = a[REEF_CONV_FLAGS];
    const int m_tiles = a[REEF_CONV_M_TILES], n_tiles = a[REEF_CONV_N_TILES];
    task = xcd_chunked(task, m_tiles * n_tiles);
    const int nt = div_small(task, m_tiles), mt = task - nt * m_tiles;
    const int segs = (Wo + kRowSeg - 1) / kRowSeg;
    const int q_seg = div_small(nt, segs);
    const int py0 = q_seg * T::G, px0 = (nt - q_seg * segs) * kRowSeg;
    const int m0 = mt * 16;
    const int K = C * 49;
    int p = 4;
    const float* in_shift = (flags & REEF_F_IN_SHIFT) ? (const float*)d.ptr[p++] : nullptr;
    const float* pool_shift = (flags & REEF_F_POOL_SHIFT) ? (const float*)d.ptr[p++] : nullptr;

    // the tile's sixteen weight rows into LDS as they are (contiguous in memory; every value loaded
    // once by one thread -- as 42 loads per lane in each of the four wavefronts they took longer than
    // the convolution itself)
    const rsrc_t rs_w = make_rsrc(d.ptr[1], (unsigned)M * (unsigned)K * 4u);
    float* WL = E + T::EFLOATS;
    constexpr int WSHARE = (T::WFLOATS + kThreads - 1) / kThreads;
    float wv[WSHARE];
#pragma unroll
    for (int i = 0; i < WSHARE; ++i) {
        const int idx = (int)threadIdx.x + kThreads * i;
        wv[i] = buf_load(rs_w, idx < 16 * K ? ((unsigned)(m0 * K) + (unsigned)idx) * 4u : kOutside);
    }
    const rsrc_t rs_bias = make_rsrc(d.ptr[3], (unsigned)M * 4u);
    float bias[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) bias[j] = buf_load(rs_bias, (unsigned)(m0 + 4 * kq + j) * 4u);

    // phase 0: the patch.  Origin: input row 4 py0 - 5, column 4 px0 - 5.
    const rsrc_t rs_in = make_rsrc(d.ptr[0], (unsigned)C * (unsigned)(H * W) * 4u);
    const int iy0 = 4 * py0 - 5, ix0 = 4 * px0 - 5;
    {
        // every load of the thread's share on its way before the first value is stored
        constexpr int SHARE = (T::PATCH + kThreads - 1) / kThreads;
        float sh[T::CMAX];
#pragma unroll
        for (int c = 0; c < T::CMAX; ++c) sh[c] = (in_shift && c < C) ? in_shift[c] : 0.0f;
        float v[SHARE];
        int cc[SHARE];
        bool inside[SHARE];
#pragma unroll
        for (int i = 0; i < SHARE; ++i) {
            const int idx = (int)threadIdx.x + kThreads * i;
            const int c = idx / (T::PR * T::PC), rem = idx - c * (T::PR * T::PC);     // constants: shifts and a multiply
            const int iy = iy0 + (rem >> 6), ix = ix0 + (rem & 63);
            inside[i] = c < C && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
            cc[i] = c;
            v[i] = buf_load(rs_in, inside[i] ? (unsigned)(c * H * W + iy * W + ix) * 4u : kOutside);
        }
#pragma unroll
        for (int i = 0; i < SHARE; ++i) {
            const int idx = (int)threadIdx.x + kThreads * i;
            const float s = cc[i] == 0 ? sh[0] : cc[i] == 1 ? sh[1] : sh[2];
            if (idx < T::PATCH) patch[idx] = inside[i] ? v[i] + s : 0.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < WSHARE; ++i) {
        const int idx = (int)threadIdx.x + kThreads * i;
        if (idx < T::WFLOATS) WL[idx] = wv[i];
    }
    __syncthreads();

    // phase 1.  The weights of this lane's channel row: step s = filter row s / 2 (of channel s / 14),
    // tap kx = 4 (s % 2) + kq; kx = 7 does not exist (weight 0).
    const int act = a[REEF_CONV_ACT], act2 = a[REEF_CONV_ACT2];
    float ra[T::STEPS];
#pragma unroll
    for (int s = 0; s < T::STEPS; ++s) {
        const int c = s / 14, ky = (s % 14) / 2, kx0 = 4 * (s & 1);
        const bool real = c < C && kx0 + kq < 7;
        const float w = WL[i16 * K + min(c, C - 1) * 49 + ky * 7 + min(kx0 + kq, 6)];
        ra[s] = real ? w : 0.0f;
    }
    for (int g = wave; g < T::NG; g += 4) {
        const int r = g >> 1, gc = g & 1;
        const int j = min(16 * gc + i16, 28);          // columns past the 29 a tile needs: computed, never read
        const float* base = patch + (2 * r) * T::PC + 2 * j + kq;
        f32x4 acc0 = f32x4{0.0f, 0.0f, 0.0f, 0.0f}, acc1 = acc0;
        // a channel at a time: its fourteen patch values into registers, then fourteen MFMAs (a channel
        // the image does not have: weights 0 against a patch of zeros)
#pragma unroll
        for (int c = 0; c < T::CMAX; ++c) {
            float b[14];
#pragma unroll
            for (int i = 0; i < 14; ++i) b[i] = base[(c * T::PR + i / 2) * T::PC + 4 * (i & 1)];
            __builtin_amdgcn_sched_barrier(0);      // all fourteen reads issued before the first MFMA waits for one
#pragma unroll
            for (int i = 0; i < 14; ++i) {
                // the tap that does not exist (kx = 7): 0 x 0, whatever the patch holds there
                const float bv = (i & 1) ? (kq == 3 ? 0.0f : b[i]) : b[i];
                if (i & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[14 * c + i], bv, acc1, 0, 0, 0);
                else acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[14 * c + i], bv, acc0, 0, 0, 0);
            }
        }
        const int cy = 2 * py0 - 1 + r, cx = 2 * px0 - 1 + 16 * gc + i16;
        const bool inside = (unsigned)cy < (unsigned)Hc && (unsigned)cx < (unsigned)Wc;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const float v = act_apply((acc0[jj] + acc1[jj]) + bias[jj], act);
            E[(4 * kq + jj) * T::ESTRIDE + r * 32 + 16 * gc + i16] = inside ? v : -FLT_MAX;
        }
    }
    __syncthreads();

    // phase 2
    const int row = threadIdx.x >> 4, col = threadIdx.x & 15;
    const unsigned ch = (unsigned)(m0 + row);
    const rsrc_t rs_o = make_rsrc(d.ptr[2], (unsigned)M * (unsigned)(Ho * Wo) * 4u);
    const float sh2 = (pool_shift && ch < (unsigned)M) ? pool_shift[ch] : 0.0f;
    const float* Ec = E + row * T::ESTRIDE + 2 * col;
#pragma unroll
    for (int g = 0; g < T::G; ++g) {
        float m = -FLT_MAX;
#pragma unroll
        for (int ky = 0; ky < 3; ++ky)
#pragma unroll
            for (int kx = 0; kx < 3; ++kx) m = fmaxf(m, Ec[(2 * g + ky) * 32 + kx]);
        const bool ok = col < kRowSeg && px0 + col < Wo && py0 + g < Ho && ch < (unsigned)M;
        buf_store(rs_o, ok ? (ch * (unsigned)(Ho * Wo) + (unsigned)((py0 + g) * Wo + px0 + col)) * 4u : kOutside,
                  act_apply(m + sh2, act2));
    }
    return true;
}

// ---- reef_gemm ----------------------------------------------------------------
// TRANS_B: B stored [N][K] (dense layers, Q.K^T) -- both operands take 128-bit row
// loads, so K, lda, ldb and the batch strides must be multiples of 4 floats.
// !TRANS_B: B stored [K][N] (P.V) -- element-wise B loads, 128-bit A loads.
// LN_A (symbols reef_gemm_ntl_<tile>, REEF_GEMM_F_LN): C = act(alpha LayerNorm(A) W^T + bias) (+ R),
// LayerNorm(A)[m][k] = (A[m][k] - mean[m]) rstd[m] gamma[k] + beta[k].  A transformer layer
// normalises and then multiplies; as two launches the normalised matrix makes a round trip
// through memory behind a launch that only reads and writes 128 rows.  Normalising the rows on
// the way into the tiles needs their statistics BEFORE the K loop -- a pass over the rows that
// every column tile of a row block repeats (measured: 2.4 us of a 17 us kernel, plus 1.3 us
// for gamma and beta riding along with every load).  The product is linear in the row, so the
// normalisation moves behind the K loop instead:
//     sum_k LN(A)[m][k] W[n][k] = rstd[m] (sum_k A[m][k] Wg[n][k] - mean[m] c1[n]) + c2[n]
// with Wg[n][k] = gamma[k] W[n][k], c1[n] = sum_k Wg[n][k], c2[n] = sum_k beta[k] W[n][k], three
// tensors the model generator derives from the parameters once.  The K loop is the plain
// product A Wg^T; the A loader adds every value it moves to per-row sums around a pivot (the
// workgroup sees each of its rows completely), the threads of a row merge them after the loop,
// and the epilogue applies mean, rstd, c1 and c2.  The normalised rows themselves (the operand
// of the next residual, REEF_GEMM_F_LN_OUT) are written by the workgroups of a row block, a
// share each, from the statistics and a second look at their share of A.
// A and A' are [M][K] with leading dimension lda and no offset; no batch.
// ptr: A, Wg, C, bias (optional), residual (optional), c1, c2, gamma, beta, A' (optional).
template <class T, bool TRANS_B, bool LN_A, class Poll>
__device__ __forceinline__ bool gemm_body(const ReefOpDesc& d, int task, char* smem_raw,
                                          const Poll& poll) {
    const int* a = d.attr;
    const int M = a[REEF_GEMM_M], N = a[REEF_GEMM_N], K = a[REEF_GEMM_K];
    const int n_tiles = a[REEF_GEMM_N_TILES];
    const int tiles = a[REEF_GEMM_M_TILES] * n_tiles;
    const int b = div_small(task, tiles);
    const int rem = task - b * tiles;
    const int mt = div_small(rem, n_tiles), nt = rem - mt * n_tiles;
    const int m0 = mt * T::BM, n0 = nt * T::BN;
    const int lda = a[REEF_GEMM_LDA], ldb = a[REEF_GEMM_LDB], ldc = a[REEF_GEMM_LDC];
    const float* A = (const float*)d.ptr[0] + a[REEF_GEMM_OFF_A] + (size_t)b * a[REEF_GEMM_STRIDE_A];
    const float* B = (const float*)d.ptr[1] + a[REEF_GEMM_OFF_B] + (size_t)b * a[REEF_GEMM_STRIDE_B];
    float* C = (float*)d.ptr[2] + a[REEF_GEMM_OFF_C] + (size_t)b * a[REEF_GEMM_STRIDE_C];
    const int nk = (K + T::BK - 1) / T::BK;
    float* smem = (float*)smem_raw;
    f32x16 acc[T::TM][T::TN];

    bool ok;
    ALoader<T, true, LN_A> la;
    la.init(A, ((unsigned)(M - 1) * (unsigned)lda + (unsigned)K) * 4u, lda, m0, M, 0, K);
    static_assert(!LN_A || TRANS_B, "the LayerNorm form exists for K-contiguous B");
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
    const WaveGeom<T> wg;
    const int wm0 = wg.wm0, wn0 = wg.wn0;
    const int fl = a[REEF_GEMM_FLAGS];
    const float* bias = (fl & REEF_GEMM_F_BIAS) ? (const float*)d.ptr[3] : nullptr;
    // the residual: laid out as C is (same leading dimension, offset and batch stride)
    const float* R = (fl & REEF_GEMM_F_RES)
                         ? (const float*)d.ptr[bias ? 4 : 3] + a[REEF_GEMM_OFF_C] + (size_t)b * a[REEF_GEMM_STRIDE_C]
                         : nullptr;
    const int lnp = 3 + (bias ? 1 : 0) + (R ? 1 : 0);      // LN_A: first of c1, c2, gamma, beta, A'
    float e_c1[T::TN], e_c2[T::TN];
    // LN_A with REEF_GEMM_F_LN_OUT: the normalised rows go to memory as well, a share per column
    // tile -- the BM * K / 4 float4s of the row block in n_tiles contiguous runs (one workgroup
    // writing it all would be the launch's straggler).  What a thread needs for the first float4
    // of its share (the only one for rows of up to 256 n_tiles / BM float4s) is loaded here, ahead
    // of the K loop, so that after the loop only arithmetic and a store are left.
    float* Aout = nullptr;
    int o_share = 0, o_end = 0, o_row4 = 1, o_r = 0;
    unsigned o_off = kOutside, o_koff = kOutside;
    f32x4 o_v, o_g, o_b;
    rsrc_t rs_oa, rs_og, rs_ob;
    if (LN_A) {
        la.init_ln();
        if (fl & REEF_GEMM_F_LN_OUT) Aout = (float*)d.ptr[lnp + 4];
        const unsigned bytes = ((unsigned)(M - 1) * (unsigned)lda + (unsigned)K) * 4u;
        rs_oa = make_rsrc(A, Aout ? bytes : 0u);
        rs_og = make_rsrc(d.ptr[lnp + 2], Aout ? (unsigned)K * 4u : 0u);
        rs_ob = make_rsrc(d.ptr[lnp + 3], Aout ? (unsigned)K * 4u : 0u);
        o_row4 = K / 4;
        const int total = T::BM * o_row4;
        o_share = (total + n_tiles - 1) / n_tiles;
        o_end = (nt + 1) * o_share < total ? (nt + 1) * o_share : total;
        const int id = nt * o_share + (int)threadIdx.x;
        if (Aout && id < o_end) {
            o_r = div_small(id, o_row4);
            if (m0 + o_r < M) {
                o_koff = (unsigned)(id - o_r * o_row4) * 16u;
                o_off = (unsigned)(m0 + o_r) * (unsigned)lda * 4u + o_koff;
            }
        }
        o_v = buf_load4(rs_oa, o_off);
        o_g = buf_load4(rs_og, o_koff);
        o_b = buf_load4(rs_ob, o_koff);
        // c1 and c2 of this thread's output columns, on their way before the K loop
        const float* c1 = (const float*)d.ptr[lnp];
        const float* c2 = (const float*)d.ptr[lnp + 1];
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            const int n = n0 + wn0 + tn * 32 + l32;
            e_c1[tn] = n < N ? c1[n] : 0.0f;
            e_c2[tn] = n < N ? c2[n] : 0.0f;
        }
    }
    if (TRANS_B) {
        // B is [N][K]: stage it exactly like A (rows = n).
        typedef Tile<T::WGN, T::WGM, T::TN, T::TM, T::DEPTH, T::KW> TB;  // BM of TB == BN of T
        ALoader<TB, true> lb;
        lb.init(B, ((unsigned)(N - 1) * (unsigned)ldb + (unsigned)K) * 4u, ldb, n0, N, 0, K);
        ok = k_loop<T, true>(la, lb, nk, smem, acc, poll);
    } else {
        BknLoader<T> lb;
        lb.init(B, ((unsigned)(K - 1) * (unsigned)ldb + (unsigned)N) * 4u, ldb, n0, N, 0, K);
        ok = k_loop<T, false>(la, lb, nk, smem, acc, poll);
    }
    if (!ok) return false;
    float* stats = smem + (T::LDS_BYTES / 4);      // LN_A: mean, rstd per row, behind the staging buffers
    if (LN_A) {
        // a row's sums: the TPR threads that loaded its float4s are neighbouring lanes
        typedef ALoader<T, true, LN_A> LA;
        const float eps = __int_as_float(a[REEF_GEMM_LN_EPS_BITS]);
#pragma unroll
        for (int i = 0; i < LA::NV; ++i) {
            float t1 = la.s1[LN_A ? i : 0], t2 = la.s2[LN_A ? i : 0];
#pragma unroll
            for (int o = 1; o < LA::TPR; o <<= 1) {
                t1 += __shfl_xor(t1, o, 64);
                t2 += __shfl_xor(t2, o, 64);
            }
            if (threadIdx.x % LA::TPR == 0) {
                const int r = threadIdx.x / LA::TPR + LA::RPP * i;
                const float m1 = t1 / (float)K;                        // mean of a - pivot
                const float var = fmaxf(t2 / (float)K - m1 * m1, 0.0f);
                stats[2 * r] = la.pivot[LN_A ? i : 0] + m1;
                stats[2 * r + 1] = 1.0f / sqrtf(var + eps);
            }
        }
        __syncthreads();
        if (Aout) {
            const rsrc_t rs_o = make_rsrc(Aout, ((unsigned)(M - 1) * (unsigned)lda + (unsigned)K) * 4u);
            {   // the float4 whose operands have been waiting since before the K loop
                const float mu = stats[2 * o_r], rs = stats[2 * o_r + 1];
                f32x4 y;
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = (o_v[e] - mu) * rs * o_g[e] + o_b[e];
                buf_store4(rs_o, o_off, y);      // no share, or a row outside M: an offset outside the buffer
            }
            for (int id = nt * o_share + (int)threadIdx.x + kThreads; id < o_end; id += kThreads) {
                const int r = div_small(id, o_row4), k4 = (id - r * o_row4) * 4;
                if (m0 + r < M) {
                    const unsigned off = ((unsigned)(m0 + r) * (unsigned)lda + (unsigned)k4) * 4u;
                    const f32x4 v = buf_load4(rs_oa, off);
                    const f32x4 gm = buf_load4(rs_og, (unsigned)k4 * 4u), bt = buf_load4(rs_ob, (unsigned)k4 * 4u);
                    const float mu = stats[2 * r], rs = stats[2 * r + 1];
                    f32x4 y;
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] = (v[e] - mu) * rs * gm[e] + bt[e];
                    buf_store4(rs_o, off, y);
                }
            }
        }
    }
    float res[T::TM][T::TN][T::RPW];
    const int r0 = finish_tile<T>(acc, res, smem);

    const float alpha = __int_as_float(a[REEF_GEMM_ALPHA_BITS]);
    const int act = a[REEF_GEMM_ACT];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            const int n = n0 + wn0 + tn * 32 + l32;
            const float bv = (bias && n < N) ? bias[n] : 0.0f;
#pragma unroll
            for (int rr = 0; rr < T::RPW; ++rr) {
                const int r = r0 + rr;
                const int ml = wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);     // row inside the tile
                const int m = m0 + ml;
                if (m < M && n < N) {
                    float v = res[tm][tn][rr];
                    if (LN_A) v = stats[2 * ml + 1] * (v - stats[2 * ml] * e_c1[tn]) + e_c2[tn];
                    v = v * alpha + bv;
                    if (act == REEF_ACT_RELU) v = fmaxf(v, 0.0f);
                    else if (act == REEF_ACT_GELU) v = gelu_erf(v);
                    if (R) v += R[(size_t)m * ldc + n];
                    C[(size_t)m * ldc + n] = v;
                }
            }
        }
    return true;
}

// ---- reef_gemm_ntd: C = act(alpha A B^T + bias) with both operands straight from memory -----
// The direct scheme of reef_conv2d_d1 applied to a GEMM whose operands are both K-contiguous
// (dense layers, Q K^T): a lane of the A side (row = lane % 16 of a 16-row group, k slot =
// lane / 16) and a lane of the B side (column = lane % 16 of a 16-column group) each load the
// eight consecutive k values of their slot with two 128-bit loads; MFMA j multiplies value j of
// every slot.  The four wavefronts split K (a step is 128 k values), the partial tiles meet in
// LDS, thread t writes element (t / 16, t % 16) of every 16 x 16 sub-tile.  K % 8 == 0, lda, ldb
// and the batch strides multiples of 4.  No split of K across workgroups.
template <int TM, int TN, class Poll>
__device__ __forceinline__ bool gemm_nt_direct_body(const ReefOpDesc& d, int task, char* smem_raw,
                                                    const Poll& poll) {
    typedef TileD16<TN, TM> TD;
    constexpr int LOADS = 2 * (TM + TN);
    constexpr int NS = 3;      // steps of loads in flight (6: BERT-base +1.8 %, 4: +1.7 %, 2: +0.7 %, same process)
    float* smem = (float*)smem_raw;
    int* sflag = (int*)(smem + 4 * TD::SUBS * TD::PART);
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, i16 = lane & 15, kq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int M = a[REEF_GEMM_M], N = a[REEF_GEMM_N], K = a[REEF_GEMM_K];
    const int n_tiles = a[REEF_GEMM_N_TILES];
    const int tiles = a[REEF_GEMM_M_TILES] * n_tiles;
    // K split across workgroups (batch 1): the split_k workgroups of a tile are neighbours in the task order
    const int split_k = a[REEF_GEMM_SPLIT_K] > 1 ? a[REEF_GEMM_SPLIT_K] : 1;
    const int tile_task = split_k > 1 ? div_small(task, split_k) : task;
    const int split = task - tile_task * split_k;
    const int b = div_small(tile_task, tiles);
    const int rem = tile_task - b * tiles;
    const int mt = div_small(rem, n_tiles), nt = rem - mt * n_tiles;
    const int m0 = mt * TD::BM, n0 = nt * TD::BN;
    const unsigned lda = (unsigned)a[REEF_GEMM_LDA], ldb = (unsigned)a[REEF_GEMM_LDB],
                   ldc = (unsigned)a[REEF_GEMM_LDC];
    const rsrc_t rs_a = make_rsrc((const float*)d.ptr[0] + a[REEF_GEMM_OFF_A] + (size_t)b * a[REEF_GEMM_STRIDE_A],
                                  ((unsigned)(M - 1) * lda + (unsigned)K) * 4u);
    const rsrc_t rs_b = make_rsrc((const float*)d.ptr[1] + a[REEF_GEMM_OFF_B] + (size_t)b * a[REEF_GEMM_STRIDE_B],
                                  ((unsigned)(N - 1) * ldb + (unsigned)K) * 4u);
    const rsrc_t rs_c = make_rsrc((const float*)d.ptr[2] + a[REEF_GEMM_OFF_C] + (size_t)b * a[REEF_GEMM_STRIDE_C],
                                  ((unsigned)(M - 1) * ldc + (unsigned)N) * 4u);
    const bool has_bias = a[REEF_GEMM_FLAGS] & REEF_GEMM_F_BIAS, has_res = a[REEF_GEMM_FLAGS] & REEF_GEMM_F_RES;
    const rsrc_t rs_bias = make_rsrc(d.ptr[has_bias ? 3 : 2], (unsigned)N * 4u);
    // the residual is laid out as C is; without one an empty buffer, whose loads give 0
    const rsrc_t rs_res = make_rsrc((const float*)d.ptr[has_res ? (has_bias ? 4 : 3) : 2] + a[REEF_GEMM_OFF_C] +
                                        (size_t)b * a[REEF_GEMM_STRIDE_C],
                                    has_res ? ((unsigned)(M - 1) * ldc + (unsigned)N) * 4u : 0u);

    // the outputs of this thread and their bias, ahead of the K loop
    const int orow = threadIdx.x >> 4, ocol = threadIdx.x & 15;
    unsigned ooff[TM][TN];
    float e_bias[TN], e_res[TM][TN];
#pragma unroll
    for (int g = 0; g < TN; ++g) {
        const unsigned n = (unsigned)(n0 + 16 * g + ocol);
        e_bias[g] = has_bias ? buf_load(rs_bias, n * 4u) : 0.0f;
#pragma unroll
        for (int h = 0; h < TM; ++h) {
            const unsigned m = (unsigned)(m0 + 16 * h + orow);
            ooff[h][g] = n < (unsigned)N ? (m * ldc + n) * 4u : kOutside;
            e_res[h][g] = buf_load(rs_res, ooff[h][g]);
        }
    }

    const int k_lo = split_k > 1 ? split * a[REEF_GEMM_K_CHUNK] : 0;        // this workgroup's part of K
    const int k_hi = split_k > 1 ? min(K, k_lo + a[REEF_GEMM_K_CHUNK]) : K;
    const int lane_k = k_lo + (wave * 4 + kq) * 8;   // first k of this lane's slot
    const int nsteps = (k_hi - k_lo + 127) / 128;
    const int lane_steps = lane_k < k_hi ? (k_hi - lane_k + 127) / 128 : 0;
    unsigned va[TM], vb[TN];
#pragma unroll
    for (int h = 0; h < TM; ++h) va[h] = ((unsigned)(m0 + 16 * h + i16) * lda + (unsigned)lane_k) * 4u;
#pragma unroll
    for (int g = 0; g < TN; ++g) vb[g] = ((unsigned)(n0 + 16 * g + i16) * ldb + (unsigned)lane_k) * 4u;

    float ra[NS][TM][8], rb[NS][TN][8];
    auto load8 = [&](float (&dst)[8], rsrc_t rs, unsigned off, unsigned soff) {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const f32x4 v = __builtin_bit_cast(
                f32x4, __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(off + 16u * q), (int)soff, 0));
            dst[4 * q] = v[0]; dst[4 * q + 1] = v[1]; dst[4 * q + 2] = v[2]; dst[4 * q + 3] = v[3];
        }
    };
    auto load_step = [&](int s, int step) {
        const unsigned outm = step < lane_steps ? 0u : kOutside;
        const unsigned so = (unsigned)step * 512u;   // 128 k values, uniform
#pragma unroll
        for (int h = 0; h < TM; ++h) load8(ra[s][h], rs_a, va[h] | outm, so);
#pragma unroll
        for (int g = 0; g < TN; ++g) load8(rb[s][g], rs_b, vb[g] | outm, so);
    };
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        load_step(s, s);
        asm volatile("" ::: "memory");
    }
    if (Poll::enabled) {
        // The flag check every best-effort workgroup makes before it does anything
        // (script/best_effort_kernel.py:22-29) is made here, with the first loads of the K loop
        // already on their way: its trip to memory hides behind theirs instead of standing in
        // front of them.  A workgroup that finds the flag raised has only read.
        if (threadIdx.x == 0) *sflag = poll.load();
        __syncthreads();
        if (*sflag) return false;
    }
    f32x4 acc[TM][TN][2];
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            acc[h][g][0] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            acc[h][g][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    auto mma_stage = [&](int s) {
#pragma unroll
        for (int q = 0; q < 8; ++q)
#pragma unroll
            for (int h = 0; h < TM; ++h)
#pragma unroll
                for (int g = 0; g < TN; ++g)
                    acc[h][g][q & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[s][h][q], rb[s][g][q],
                                                                            acc[h][g][q & 1], 0, 0, 0);
    };
    int pf = 0, it = 0;
    bool left = false;
    // (groups whose refills all exist, then the last whole group with the refills the remaining steps
    // need and no others, as in the convolution)
    for (; it + 2 * NS <= nsteps; it += NS) {
        if (Poll::enabled) {
            if (pf) {
                *sflag = 1;
                left = true;
                break;
            }
            pf = poll.load();
        }
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            mma_stage(s);
            load_step(s, it + s + NS);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (!left && it + NS <= nsteps) {
        if (Poll::enabled && pf) {
            *sflag = 1;
            left = true;
        } else {
            if (Poll::enabled) pf = poll.load();
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                mma_stage(s);
                if (it + s + NS < nsteps) load_step(s, it + s + NS);
                __builtin_amdgcn_sched_barrier(0);
            }
            it += NS;
        }
    }
    if (!left) {
#pragma unroll
        for (int s = 0; s < NS - 1; ++s)
            if (it + s < nsteps) mma_stage(s);
    }

    float* part = smem + wave * (TD::SUBS * TD::PART);
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                part[(h * TN + g) * TD::PART + (5 * kq + j) * 16 + i16] = acc[h][g][0][j] + acc[h][g][1][j];
    __syncthreads();
    if (Poll::enabled && *sflag) return false;
    const float* mine = smem + threadIdx.x + (threadIdx.x >> 6) * 16;
    constexpr int WSTRIDE = TD::SUBS * TD::PART;
    const float alpha = __int_as_float(a[REEF_GEMM_ALPHA_BITS]);
    const int act = a[REEF_GEMM_ACT];
    auto finish = [&](float sum, int h, int g) {
        float v = sum * alpha + e_bias[g];
        if (act == REEF_ACT_RELU) v = fmaxf(v, 0.0f);
        else if (act == REEF_ACT_GELU) v = gelu_erf(v);
        buf_store(rs_c, ooff[h][g], v + e_res[h][g]);
    };
    float v[TM][TN];
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            const float* e = mine + (h * TN + g) * TD::PART;
            v[h][g] = ((e[0] + e[WSTRIDE]) + e[2 * WSTRIDE]) + e[3 * WSTRIDE];
        }
    if (split_k == 1) {
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g) finish(v[h][g], h, g);
        return true;
    }

    // The split_k partial tiles of an output tile meet inside the launch, as those of the direct
    // convolutions do: a split of two through one exchange per element where every launch on the
    // buffers runs to completion, otherwise partial tiles to the workspace, a count per tile,
    // and the last arrival sums them in split order.  The sums and their order are the same.
    // ptr: .., workspace (split_k [+1] regions of M x N), arrival counters.
    const int aux = 3 + (has_bias ? 1 : 0) + (has_res ? 1 : 0);
    const size_t MN = (size_t)M * N;
    float* ws = (float*)d.ptr[aux];
    unsigned widx[TM][TN];         // element m * N + n of a dense M x N region, ~0u outside the matrix
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g) {
            const unsigned m = (unsigned)(m0 + 16 * h + orow), n = (unsigned)(n0 + 16 * g + ocol);
            widx[h][g] = (m < (unsigned)M && n < (unsigned)N) ? m * (unsigned)N + n : ~0u;
        }
    if (split_k == 2 && (a[REEF_GEMM_FLAGS] & REEF_GEMM_F_PAIR_FOLD) && poll.pair_fold_ok()) {
        // a value is parked with its sign bit flipped, so a parked value is never the empty slot's 0
        unsigned* slots = (unsigned*)(ws + 2 * MN);
        unsigned got[TM][TN];
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g) {
                got[h][g] = 0;
                if (widx[h][g] != ~0u) {
                    unsigned parked = __float_as_uint(v[h][g]) ^ 0x80000000u;
                    parked = parked ? parked : 0x80000000u;
                    got[h][g] = __hip_atomic_exchange(&slots[widx[h][g]], parked, __ATOMIC_RELAXED,
                                                      __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#pragma unroll
        for (int h = 0; h < TM; ++h)
#pragma unroll
            for (int g = 0; g < TN; ++g)
                if (got[h][g] != 0) {   // second to arrive: the other half is here
                    const float other = __uint_as_float(got[h][g] ^ 0x80000000u);
                    finish(split == 0 ? v[h][g] + other : other + v[h][g], h, g);   // split order
                    __hip_atomic_store(&slots[widx[h][g]], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
        return true;
    }
    int* counters = (int*)d.ptr[aux + 1] + a[REEF_GEMM_SYNC_OFF];
    int* s_last = sflag + 1;
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g)
            if (widx[h][g] != ~0u) store_agent(ws + (size_t)split * MN + widx[h][g], v[h][g]);
    partial_stores_done();   // every store of this workgroup is acknowledged before it counts in
    __syncthreads();
    if (threadIdx.x == 0) {
        const int old = __hip_atomic_fetch_add(&counters[rem], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *s_last = (old == split_k - 1);
    }
    __syncthreads();
    if (!*s_last) return true;
#pragma unroll
    for (int h = 0; h < TM; ++h)
#pragma unroll
        for (int g = 0; g < TN; ++g)
            if (widx[h][g] != ~0u) {
                const float* src = ws + widx[h][g];
                float sum = 0.0f;
                for (int s0 = 0; s0 < split_k; s0 += 4) {
                    float p[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) p[j] = load_agent(src + (size_t)min(s0 + j, split_k - 1) * MN);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (s0 + j < split_k) sum = (s0 + j == 0) ? p[j] : sum + p[j];
                }
                finish(sum, h, g);
            }
    if (threadIdx.x == 0)  // ready for the next run
        __hip_atomic_store(&counters[rem], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

}  // namespace reef_dev
