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

template <int WGM_, int WGN_, int TM_, int TN_>
struct Tile {
    static constexpr int WGM = WGM_, WGN = WGN_, TM = TM_, TN = TN_;
    static constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32, BK = 32;
    static constexpr int LDA = BK + 4;
    static constexpr int A_FLOATS = BM * LDA;
    static constexpr int BK_FLOATS = BK * BN;   // B tile, k-major
    static constexpr int BN_FLOATS = BN * LDA;  // B tile, n-major (trans_b GEMM)
    static constexpr int B_FLOATS = BN_FLOATS > BK_FLOATS ? BN_FLOATS : BK_FLOATS;
    static constexpr int LDS_BYTES = 2 * (A_FLOATS + B_FLOATS) * 4 + 16;
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
};

typedef Tile<2, 2, 2, 2> Tile128x128;
typedef Tile<2, 2, 2, 1> Tile128x64;
typedef Tile<2, 2, 1, 1> Tile64x64;
typedef Tile<4, 1, 1, 1> Tile128x32;
typedef Tile<1, 4, 1, 1> Tile32x128;
typedef Tile<2, 2, 1, 2> Tile64x128;

// ---- A tile: rows of a K-contiguous matrix -------------------------------
template <class T>
struct ALoader {
    static constexpr int NV = T::BM / 32;  // float4 per thread per tile
    const float* base[NV];                 // row pointer + kq*4, or null when the row is outside M
    int k;                                 // k of this thread's first float4 in the next tile
    int k_end;
    bool vec;
    f32x4 reg[NV];

    __device__ __forceinline__ void init(const float* a, int lda, int m0, int M, int k_begin,
                                         int k_end_, bool vec_) {
        const int tid = threadIdx.x;
        k_end = k_end_;
        vec = vec_;
        const int kq = tid & 7;
        k = k_begin + kq * 4;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            int row = (tid >> 3) + 32 * i;
            base[i] = (m0 + row < M) ? a + (size_t)(m0 + row) * lda : nullptr;
        }
    }
    __device__ __forceinline__ void load() {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (base[i]) {
                const float* p = base[i] + k;
                if (vec) {
                    if (k < k_end) v = *(const f32x4*)p;
                } else {
                    if (k + 0 < k_end) v.x = p[0];
                    if (k + 1 < k_end) v.y = p[1];
                    if (k + 2 < k_end) v.z = p[2];
                    if (k + 3 < k_end) v.w = p[3];
                }
            }
            reg[i] = v;
        }
        k += 32;
    }
    __device__ __forceinline__ void store(float* As) const {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            int row = (tid >> 3) + 32 * i;
            *(f32x4*)(As + row * T::LDA + (tid & 7) * 4) = reg[i];
        }
    }
};

// ---- B tile for convolution: im2col gather, one n per thread --------------
template <class T>
struct Im2colLoader {
    static constexpr int RS = kThreads / T::BN;  // k rows covered per pass
    static constexpr int NR = 32 / RS;           // rows per thread per tile
    const float* in;
    int H, W, HW, kh, kw;
    int soff, iy0, ix0;
    bool nvalid;
    int k, k_end, c, ky, kx;
    int dkx, dky, dc;
    float reg[NR];

    __device__ __forceinline__ void init(const float* in_, const int* a, int n0, int N, int k_begin,
                                         int k_end_) {
        const int tid = threadIdx.x;
        in = in_;
        H = a[REEF_CONV_H];
        W = a[REEF_CONV_W];
        HW = H * W;
        kh = a[REEF_CONV_KH];
        kw = a[REEF_CONV_KW];
        const int Wo = a[REEF_CONV_WO];
        const int n = n0 + (tid & (T::BN - 1));
        nvalid = n < N;
        const int y = n / Wo, x = n - y * Wo;
        iy0 = y * a[REEF_CONV_SH] - a[REEF_CONV_PH];
        ix0 = x * a[REEF_CONV_SW] - a[REEF_CONV_PW];
        soff = iy0 * W + ix0;
        k_end = k_end_;
        k = k_begin + tid / T::BN;
        const int khw = kh * kw;
        c = k / khw;
        const int r = k - c * khw;
        ky = r / kw;
        kx = r - ky * kw;
        dkx = RS % kw;
        const int t = RS / kw;
        dky = t % kh;
        dc = t / kh;
    }
    __device__ __forceinline__ void load() {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            const bool ok = nvalid && k < k_end && (unsigned)(iy0 + ky) < (unsigned)H &&
                            (unsigned)(ix0 + kx) < (unsigned)W;
            const int off = c * HW + ky * W + kx + soff;
            reg[i] = ok ? in[off] : 0.0f;
            k += RS;
            kx += dkx;
            if (kx >= kw) { kx -= kw; ++ky; }
            ky += dky;
            if (ky >= kh) { ky -= kh; ++c; }
            c += dc;
        }
    }
    __device__ __forceinline__ void store(float* Bs) const {
        const int tid = threadIdx.x;
        const int nl = tid & (T::BN - 1), kr0 = tid / T::BN;
#pragma unroll
        for (int i = 0; i < NR; ++i) Bs[(kr0 + RS * i) * T::BN + nl] = reg[i];
    }
};

// ---- B tile for GEMM with B stored [K][N] (n contiguous) -------------------
template <class T>
struct BknLoader {
    static constexpr int RS = kThreads / T::BN;
    static constexpr int NR = 32 / RS;
    const float* col;  // B + n, or null
    int ldb, k, k_end;
    float reg[NR];
    __device__ __forceinline__ void init(const float* b, int ldb_, int n0, int N, int k_begin,
                                         int k_end_) {
        const int tid = threadIdx.x;
        const int n = n0 + (tid & (T::BN - 1));
        col = n < N ? b + n : nullptr;
        ldb = ldb_;
        k = k_begin + tid / T::BN;
        k_end = k_end_;
    }
    __device__ __forceinline__ void load() {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
            reg[i] = (col && k < k_end) ? col[(size_t)k * ldb] : 0.0f;
            k += RS;
        }
    }
    __device__ __forceinline__ void store(float* Bs) const {
        const int tid = threadIdx.x;
        const int nl = tid & (T::BN - 1), kr0 = tid / T::BN;
#pragma unroll
        for (int i = 0; i < NR; ++i) Bs[(kr0 + RS * i) * T::BN + nl] = reg[i];
    }
};

// ---- the MFMA inner product over one staged K step -------------------------
template <class T, bool B_NMAJOR>
__device__ __forceinline__ void mma_step(const float* As, const float* Bs, f32x16 (&acc)[T::TM][T::TN],
                                         int wm0, int wn0) {
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f32x4 af[T::TM];
        f32x4 bf[T::TN];
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
            af[tm] = *(const f32x4*)(As + (wm0 + tm * 32 + l32) * T::LDA + 8 * j + 4 * h);
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            if (B_NMAJOR) {
                bf[tn] = *(const f32x4*)(Bs + (wn0 + tn * 32 + l32) * T::LDA + 8 * j + 4 * h);
            } else {
                const float* bp = Bs + (8 * j + 4 * h) * T::BN + wn0 + tn * 32 + l32;
                bf[tn].x = bp[0];
                bf[tn].y = bp[T::BN];
                bf[tn].z = bp[2 * T::BN];
                bf[tn].w = bp[3 * T::BN];
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < T::TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[tm][t], bf[tn][t],
                                                                       acc[tm][tn], 0, 0, 0);
    }
}

// Double-buffered K loop shared by conv and GEMM.  Returns false when the
// preemption flag was seen (the whole workgroup leaves together: the value
// read by thread 0 is published through LDS before the step's barrier).
template <class T, bool B_NMAJOR, class LA, class LB, class Poll>
__device__ __forceinline__ bool k_loop(LA& la, LB& lb, int nk, float* smem, f32x16 (&acc)[T::TM][T::TN],
                                       const Poll& poll) {
    float* As = smem;
    float* Bs = smem + 2 * T::A_FLOATS;
    int* sflag = (int*)(smem + 2 * (T::A_FLOATS + T::B_FLOATS));
    const int wave = threadIdx.x >> 6;
    const int wm0 = (wave / T::WGN) * (T::TM * 32), wn0 = (wave % T::WGN) * (T::TN * 32);
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.0f;

    if (Poll::enabled && threadIdx.x == 0) *sflag = 0;
    la.load();
    lb.load();
    la.store(As);
    lb.store(Bs);
    __syncthreads();
    for (int it = 0; it < nk; ++it) {
        const int cur = it & 1;
        const bool more = it + 1 < nk;
        int pf = 0;
        if (more) {
            la.load();
            lb.load();
        }
        if (Poll::enabled && threadIdx.x == 0) pf = poll.load();
        mma_step<T, B_NMAJOR>(As + cur * T::A_FLOATS, Bs + cur * T::B_FLOATS, acc, wm0, wn0);
        if (more) {
            la.store(As + (cur ^ 1) * T::A_FLOATS);
            lb.store(Bs + (cur ^ 1) * T::B_FLOATS);
        }
        if (Poll::enabled && threadIdx.x == 0 && pf) *sflag = 1;
        __syncthreads();
        if (Poll::enabled && *sflag) return false;
    }
    return true;
}

// ---- reef_conv2d ------------------------------------------------------------
template <class T, class Poll>
__device__ __forceinline__ bool conv2d_body(const ReefOpDesc& d_in, int task, char* smem_raw,
                                            const Poll& poll) {
  int M, N, split_k, split, rem, m0, n0;
  float* smem = (float*)smem_raw;
  f32x16 acc[T::TM][T::TN];
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
    split = task / tiles;
    rem = task - split * tiles;
    const int mt = rem / n_tiles, nt = rem - mt * n_tiles;
    m0 = mt * T::BM;
    n0 = nt * T::BN;
    const int k_begin = split * k_chunk;
    const int k_end = min(K, k_begin + k_chunk);
    const int nk = (k_end - k_begin + 31) >> 5;

    ALoader<T> la;
    Im2colLoader<T> lb;
    la.init((const float*)d.ptr[1], K, m0, M, k_begin, k_end, (K & 3) == 0);
    lb.init((const float*)d.ptr[0], a, n0, N, k_begin, k_end);

    if (!k_loop<T, false>(la, lb, nk, smem, acc, poll)) return false;
  }

    // Everything the epilogue needs is re-read from the argument block here, so the
    // K loop does not carry the epilogue's pointers in scalar registers.
    const ReefOpDesc* dp = &d_in;
    asm volatile("" : "+s"(dp));
    const ReefOpDesc& d = *dp;
    const int* a = d.attr;
    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5, wave = threadIdx.x >> 6;
    const int wm0 = (wave / T::WGN) * (T::TM * 32), wn0 = (wave % T::WGN) * (T::TN * 32);
    float* dst = (float*)d.ptr[2];
    const int flags = a[REEF_CONV_FLAGS];
    const size_t MN = (size_t)M * N;

    if (split_k > 1 && !(flags & REEF_F_FUSED_REDUCE)) {
        // plain split-K: partial tile to the workspace, reef_splitk_reduce folds
        float* ws = dst + (size_t)split * MN;
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn) {
                const int n = n0 + wn0 + tn * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < M && n < N) ws[(size_t)m * N + n] = acc[tm][tn][r];
                }
            }
        return true;
    }

    Epilogue ep;
    ep.unpack(d, 3, flags, a[REEF_CONV_ACT], a[REEF_CONV_ACT2]);
    if (split_k > 1) {
        // fused split-K: store the partial, count in, the last arrival folds all
        // partials in ascending split order (fixed order => same bits whoever is last)
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
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < M && n < N) part[(size_t)m * N + n] = acc[tm][tn][r];
                }
            }
        __threadfence();  // release the partial tile device-wide before counting in
        __syncthreads();
        if (threadIdx.x == 0) {
            const int old = atomicAdd(&counters[rem], 1);
            *s_last = (old == split_k - 1);
        }
        __syncthreads();
        if (!*s_last) return true;
        __threadfence();  // acquire the other splits' partial tiles
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn) {
                const int n = n0 + wn0 + tn * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                    if (m < M && n < N) {
                        const size_t idx = (size_t)m * N + n;
                        float v = ws[idx];
                        for (int s = 1; s < split_k; ++s) v += ws[(size_t)s * MN + idx];
                        ep.store(dst, v, m, idx);
                    }
                }
            }
        if (threadIdx.x == 0) counters[rem] = 0;  // ready for the next run
        return true;
    }

#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            const int n = n0 + wn0 + tn * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < M && n < N) ep.store(dst, acc[tm][tn][r], m, (size_t)m * N + n);
            }
        }
    return true;
}

// ---- reef_gemm ----------------------------------------------------------------
template <class T, class Poll>
__device__ __forceinline__ bool gemm_body(const ReefOpDesc& d, int task, char* smem_raw,
                                          const Poll& poll) {
    const int* a = d.attr;
    const int M = a[REEF_GEMM_M], N = a[REEF_GEMM_N], K = a[REEF_GEMM_K];
    const int n_tiles = a[REEF_GEMM_N_TILES];
    const int tiles = a[REEF_GEMM_M_TILES] * n_tiles;
    const int b = task / tiles;
    const int rem = task - b * tiles;
    const int mt = rem / n_tiles, nt = rem - mt * n_tiles;
    const int m0 = mt * T::BM, n0 = nt * T::BN;
    const int lda = a[REEF_GEMM_LDA], ldb = a[REEF_GEMM_LDB], ldc = a[REEF_GEMM_LDC];
    const float* A = (const float*)d.ptr[0] + (size_t)b * a[REEF_GEMM_STRIDE_A];
    const float* B = (const float*)d.ptr[1] + (size_t)b * a[REEF_GEMM_STRIDE_B];
    float* C = (float*)d.ptr[2] + (size_t)b * a[REEF_GEMM_STRIDE_C];
    const int nk = (K + 31) >> 5;
    float* smem = (float*)smem_raw;
    f32x16 acc[T::TM][T::TN];

    ALoader<T> la;
    la.init(A, lda, m0, M, 0, K, ((K | lda) & 3) == 0);
    bool ok;
    if (a[REEF_GEMM_TRANS_B]) {
        // B is [N][K]: stage it exactly like A (rows = n).
        typedef Tile<T::WGN, T::WGM, T::TN, T::TM> TB;  // BM of TB == BN of T
        ALoader<TB> lb;
        lb.init(B, ldb, n0, N, 0, K, ((K | ldb) & 3) == 0);
        ok = k_loop<T, true>(la, lb, nk, smem, acc, poll);
    } else {
        BknLoader<T> lb;
        lb.init(B, ldb, n0, N, 0, K);
        ok = k_loop<T, false>(la, lb, nk, smem, acc, poll);
    }
    if (!ok) return false;

    const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5, wave = threadIdx.x >> 6;
    const int wm0 = (wave / T::WGN) * (T::TM * 32), wn0 = (wave % T::WGN) * (T::TN * 32);
    const float* bias = (a[REEF_GEMM_FLAGS] & 1) ? (const float*)d.ptr[3] : nullptr;
    const float alpha = __int_as_float(a[REEF_GEMM_ALPHA_BITS]);
    const int act = a[REEF_GEMM_ACT];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            const int n = n0 + wn0 + tn * 32 + l32;
            const float bv = (bias && n < N) ? bias[n] : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < M && n < N) {
                    float v = acc[tm][tn][r] * alpha + bv;
                    if (act == REEF_ACT_RELU) v = fmaxf(v, 0.0f);
                    else if (act == REEF_ACT_GELU) v = gelu_erf(v);
                    C[(size_t)m * ldc + n] = v;
                }
            }
        }
    return true;
}

}  // namespace reef_dev
