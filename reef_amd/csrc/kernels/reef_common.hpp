// Shared device helpers for the gfx950 REEF kernels: preemption polling
// policies, wavefront reductions, optional-operand unpacking.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "reef_kernels.h"

namespace reef_dev {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;
constexpr int kThreads = REEF_WG_THREADS;

// ---- preemption polling -------------------------------------------------
// The reference's best-effort wrapper reads *preempted once at block start
// (script/best_effort_kernel.py:22-29) and relies on a patched driver to kill
// running wavefronts (src/reef/server/scheduler.cpp:331-333).  Stock ROCm has
// no such call, so long-running bodies re-read the flag inside their main loop
// and the whole workgroup leaves together.  The flag lives in memory the host
// can write while kernels run; it is read with a system-scope relaxed atomic so
// the load is not served from a stale cache line.
struct NoPoll {
    static constexpr bool enabled = false;
    // true: every launch of this kernel on this model's buffers runs to completion (a real-time
    // model: plain launches and the real-time side of a padded launch).  What a folded split of
    // two may leave between its two workgroups in the pair slots relies on it (REEF_F_PAIR_FOLD).
    bool completes = false;
    __device__ __forceinline__ int load() const { return 0; }
    __device__ __forceinline__ bool pair_fold_ok() const { return completes; }
};
struct FlagPoll {
    static constexpr bool enabled = true;
    const int* flag;
    __device__ __forceinline__ bool pair_fold_ok() const { return false; }
    __device__ __forceinline__ int load() const {
        return __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
};

// Device-coherent accesses for data one workgroup hands to another inside a kernel
// (split-K partial tiles).  The scope travels on the instruction, so no L2-wide
// write-back or invalidate is needed -- a __threadfence() per workgroup costs two
// orders of magnitude more here.
__device__ __forceinline__ void store_agent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Waits until every vector-memory operation this lane has issued, device-scope stores included,
// has been acknowledged; keeps the compiler from moving memory operations across it.
__device__ __forceinline__ void partial_stores_done() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
}

// ---- buffer addressing ------------------------------------------------------------
// Tile loads and output stores go through buffer instructions: the tensor is described by a
// resource (base, size in bytes) held in scalar registers, the lane supplies a 32-bit byte
// offset, and the hardware checks the offset against the size -- a load outside the tensor
// returns 0 and a store outside it is dropped.  Everything a tile loader or an epilogue would
// otherwise do per element with compares, selects and exec masks (row >= M, k >= k_end,
// padding taps, the ragged last tile) becomes: pick kOutside as the offset.  Tensors are
// smaller than 1 GiB, so kOutside is outside every one of them, and so is the sum of a valid
// offset and kOutside or of two kOutside (offsets are built as row part + column part).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr unsigned kOutside = 0x40000000u;

// a / b for 0 <= a < 2^22 and 0 < b < 2^22 (task, tile and pixel numbers): the quotient of the
// float reciprocal is off by at most one, which the remainder tells.  Six instructions instead
// of the forty of a 32-bit integer division, several of which stand between a kernel's start
// and its first load.
__device__ __forceinline__ int div_small(int a, int b) {
    int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
    const int r = a - q * b;
    q += (r >= b) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return q;
}

// The same for an element index that may be larger (tensors of more than 4 M elements take the
// exact division).
__device__ __forceinline__ int div_index(size_t i, int b) {
    return i < (size_t)(1u << 22) ? div_small((int)i, b) : (int)(i / (size_t)b);
}


__device__ __forceinline__ rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load(rsrc_t r, unsigned byte_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}
__device__ __forceinline__ f32x4 buf_load4(rsrc_t r, unsigned byte_off) {
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
}
__device__ __forceinline__ void buf_store(rsrc_t r, unsigned byte_off, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, (int)byte_off, 0, 0);
}
__device__ __forceinline__ void buf_store4(rsrc_t r, unsigned byte_off, f32x4 v) {
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, (int)byte_off, 0, 0);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__device__ __forceinline__ float act_apply(float v, int act) {
    if (act == REEF_ACT_RELU) return fmaxf(v, 0.0f);
    if (act == REEF_ACT_RELU6) return fminf(fmaxf(v, 0.0f), 6.0f);
    return v;
}

__device__ __forceinline__ float gelu_erf(float x) {
    return x * (0.5f + 0.5f * erff(x * 0.70710678f));
}

// Optional operands of the conv / reduce epilogue follow the fixed pointers in
// flag-bit order: bias, residual, scale, shift.
struct Epilogue {
    const float* bias;
    const float* residual;
    const float* scale;
    const float* shift;
    float* out2;
    const float* shift2;
    int act, act2;
    int next;  // first pointer slot after the optional operands
    __device__ __forceinline__ void unpack(const ReefOpDesc& d, int first, int flags, int act_,
                                           int act2_ = 0) {
        int p = first;
        bias = (flags & REEF_F_BIAS) ? (const float*)d.ptr[p++] : nullptr;
        residual = (flags & REEF_F_RESIDUAL) ? (const float*)d.ptr[p++] : nullptr;
        if (flags & REEF_F_AFFINE) {
            scale = (const float*)d.ptr[p];
            shift = (const float*)d.ptr[p + 1];
            p += 2;
        } else {
            scale = shift = nullptr;
        }
        if (flags & REEF_F_DUAL) {
            out2 = (float*)d.ptr[p];
            shift2 = (const float*)d.ptr[p + 1];
            p += 2;
        } else {
            out2 = nullptr;
            shift2 = nullptr;
        }
        act = act_;
        act2 = act2_;
        next = p;
    }
    // v = acc; v += residual; v += bias; v = fma(v, scale, shift); act
    __device__ __forceinline__ float apply(float v, int ch, size_t idx) const {
        if (residual) v = v + residual[idx];
        if (bias) v = v + bias[ch];
        if (scale) v = fmaf(v, scale[ch], shift[ch]);
        return act_apply(v, act);
    }
    // out[idx] = apply(...); out2[idx] = act2(out[idx] + shift2[ch])
    __device__ __forceinline__ void store(float* out, float v, int ch, size_t idx) const {
        const float o = apply(v, ch, idx);
        out[idx] = o;
        if (out2) out2[idx] = act_apply(o + shift2[ch], act2);
    }
    // The same with residual[idx], bias[ch] and shift2[ch] already in registers (loaded at
    // kernel start, so their trip to memory overlaps the main loop instead of following it).
    __device__ __forceinline__ void store_pre(float* out, float v, int ch, size_t idx, float resv,
                                              float biasv, float sh2v) const {
        if (residual) v = v + resv;
        if (bias) v = v + biasv;
        if (scale) v = fmaf(v, scale[ch], shift[ch]);
        const float o = act_apply(v, act);
        out[idx] = o;
        if (out2) out2[idx] = act_apply(o + sh2v, act2);
    }
};

}  // namespace reef_dev
