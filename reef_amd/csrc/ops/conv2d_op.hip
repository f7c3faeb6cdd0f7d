// One fused convolution on plain device pointers: the call a generated kernel of the
// reference's fused_nn_conv2d_* family serves (resource/resnet152/resnet152.cu:376: in, W, out,
// bias), without a model directory around it.  Picks one of this build's gfx950 kernels, splits
// K across workgroups when the layer alone cannot fill the device, and folds the split inside
// the launch (partial tiles + arrival counters, summed in ascending split order).
//
// Two entry points (include/reef_c.h):
//   reef_ops_conv2d          takes the partial-tile workspace and the counters from hipMalloc
//                            for the duration of the call;
//   reef_ops_conv2d_noalloc  takes them from a fixed array in device memory that belongs to
//                            this library -- no allocation of any kind, for callers that
//                            cannot allocate (stream capture, serving loops).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

#include "reef_c.h"
#include "reef_hal.h"
#include "reef_kernels.h"

namespace {

// ---- scratch of the allocation-free entry point -------------------------------------------
// [0, kCounterBytes): one arrival counter per output tile; [kCounterBytes, ..): partial tiles.
constexpr size_t kCounterBytes = 64 * 1024;
// The plan below puts at most 256 workgroups on a split layer and a workgroup's tile has at
// most 64 x 64 outputs, so no layer needs more than 256 x 4096 partial sums = 4 MiB; the
// size check in the entry point guards that bound.
constexpr size_t kWorkspaceBytes = 4u * 1024 * 1024;
constexpr size_t kScratchBytes = kCounterBytes + kWorkspaceBytes;
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kScratchBytes];

// Fills n 32-bit words (a captured stream must not hold a memset node: a small kernel instead).
__global__ void fill_words(uint32_t* p, uint32_t value, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

constexpr int kMaxDevices = 16;
struct DeviceState {
    bool ready = false;
    hipModule_t module = nullptr;
    hipFunction_t rows_g2 = nullptr, d1 = nullptr, d3 = nullptr, d7 = nullptr, d9 = nullptr, general = nullptr,
                  unaligned = nullptr;
    unsigned char* scratch_ptr = nullptr;   // device address of `scratch` on this GPU
};
DeviceState g_dev[kMaxDevices];
std::mutex g_mtx;
std::string g_co_path;

int fail(const std::string& m) {
    reef_hal_set_error(m.c_str());
    return 1;   // Status::Fail
}
int hip_fail(hipError_t e, const char* what) { return fail(std::string(what) + ": " + hipGetErrorString(e)); }

// Loads the kernels and finds this GPU's copy of the scratch array.  Once per device, with
// that device current.
int ensure_device(DeviceState** out, bool may_set_up = true) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail("reef_ops: device index out of range");
    std::lock_guard<std::mutex> lock(g_mtx);
    DeviceState& d = g_dev[dev];
    if (!d.ready) {
        if (!may_set_up) return fail("reef_ops_conv2d_noalloc: reef_ops_init has not run with this device current");
        if (g_co_path.empty()) return fail("reef_ops_init has not been called");
        e = hipModuleLoad(&d.module, g_co_path.c_str());
        if (e != hipSuccess) return hip_fail(e, ("hipModuleLoad " + g_co_path).c_str());
        struct { hipFunction_t* fn; const char* name; } syms[] = {
            {&d.rows_g2, "reef_conv2d_r9_g2"}, {&d.d1, "reef_conv2d_d1_16x32k4"},
            {&d.d3, "reef_conv2d_d3_16x32k4"}, {&d.d7, "reef_conv2d_d7_16x32k4"},
            {&d.d9, "reef_conv2d_d9_16x32k4"}, {&d.general, "reef_conv2d_64x64"},
            {&d.unaligned, "reef_conv2d_u_64x64"}};
        for (auto& s : syms) {
            e = hipModuleGetFunction(s.fn, d.module, s.name);
            if (e != hipSuccess) return hip_fail(e, (std::string("hipModuleGetFunction ") + s.name).c_str());
        }
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        d.scratch_ptr = (unsigned char*)p;
        d.ready = true;
    }
    *out = &d;
    return 0;
}

struct Plan {
    hipFunction_t fn;
    ReefOpDesc desc;
    uint32_t tasks;
    int split_k, tiles;
    size_t ws_floats;
    int ws_slot, sync_slot;   // pointer slots of workspace and counters (split_k > 1)
};

int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Kernel, tile and split of one layer.  The split puts about one workgroup on every CU.
int make_plan(const DeviceState& dv, const reef_conv2d_desc* c, const float* in, const float* w,
              const float* bias, const float* residual, float* out, Plan* p) {
    if (!c || !in || !w || !out) return fail("reef_ops_conv2d: null argument");
    if (c->cin <= 0 || c->cout <= 0 || c->h <= 0 || c->w <= 0 || c->kh <= 0 || c->kw <= 0 || c->stride_h <= 0 ||
        c->stride_w <= 0 || c->pad_h < 0 || c->pad_w < 0)
        return fail("reef_ops_conv2d: bad shape");
    const int Ho = (c->h + 2 * c->pad_h - c->kh) / c->stride_h + 1;
    const int Wo = (c->w + 2 * c->pad_w - c->kw) / c->stride_w + 1;
    if (Ho <= 0 || Wo <= 0) return fail("reef_ops_conv2d: empty output");
    if (c->act != REEF_ACT_NONE && c->act != REEF_ACT_RELU && c->act != REEF_ACT_RELU6)
        return fail("reef_ops_conv2d: unknown activation");
    const int M = c->cout, N = Ho * Wo, taps = c->kh * c->kw;
    const long long K = (long long)c->cin * taps;
    if ((long long)M * N >= (1ll << 28) || K * M >= (1ll << 28) || (long long)c->cin * c->h * c->w >= (1ll << 28))
        return fail("reef_ops_conv2d: tensor of 1 GiB or more");
    // the kernels decode pixel, tile and task numbers with a float reciprocal that is exact below 2^22
    if (N >= (1 << 22) || (long long)c->h * c->w >= (1 << 22))
        return fail("reef_ops_conv2d: image of 4 Mi pixels or more");
    int mode, tile, bm, bk, n_tiles;
    const bool rows = c->kh == 3 && c->kw == 3 && c->stride_h == 1 && c->stride_w == 1 && c->pad_h == 1 && c->pad_w == 1;
    if (rows) {
        mode = REEF_CONV_MODE_ROWS; tile = REEF_TILE_R9G2; bm = 16; bk = 144;
        n_tiles = ceil_div(Ho, 2) * ceil_div(Wo, 14);
        p->fn = dv.rows_g2;
    } else if ((taps == 1 && c->cin % 8 == 0) || taps == 3 || taps == 7 || taps == 9) {
        mode = REEF_CONV_MODE_DIRECT; tile = REEF_TILE_16x32k4; bm = 16; bk = taps == 1 ? 128 : 16 * taps;
        n_tiles = ceil_div(N, 32);
        p->fn = taps == 1 ? dv.d1 : taps == 3 ? dv.d3 : taps == 7 ? dv.d7 : dv.d9;
    } else {
        mode = K % 4 == 0 ? REEF_CONV_MODE_GENERAL : REEF_CONV_MODE_UNALIGNED;
        tile = REEF_TILE_64x64; bm = 64; bk = 32;
        n_tiles = ceil_div(N, 64);
        p->fn = K % 4 == 0 ? dv.general : dv.unaligned;
    }
    const int m_tiles = ceil_div(M, bm);
    const int tiles = m_tiles * n_tiles;
    const int max_split = ceil_div((int)K, bk);
    int split = 256 / tiles;
    if (split < 1) split = 1;
    if (split > max_split) split = max_split;
    if (split > 16) split = 16;
    int k_chunk = ceil_div(ceil_div((int)K, split), bk) * bk;
    split = ceil_div((int)K, k_chunk);
    int flags = (bias ? REEF_F_BIAS : 0) | (residual ? REEF_F_RESIDUAL : 0) | (split > 1 ? REEF_F_FUSED_REDUCE : 0);

    std::memset(&p->desc, 0, sizeof(p->desc));
    int32_t* a = p->desc.attr;
    a[REEF_CONV_CIN] = c->cin; a[REEF_CONV_H] = c->h; a[REEF_CONV_W] = c->w; a[REEF_CONV_COUT] = c->cout;
    a[REEF_CONV_HO] = Ho; a[REEF_CONV_WO] = Wo; a[REEF_CONV_KH] = c->kh; a[REEF_CONV_KW] = c->kw;
    a[REEF_CONV_SH] = c->stride_h; a[REEF_CONV_SW] = c->stride_w; a[REEF_CONV_PH] = c->pad_h; a[REEF_CONV_PW] = c->pad_w;
    a[REEF_CONV_FLAGS] = flags; a[REEF_CONV_ACT] = c->act; a[REEF_CONV_TILE] = tile;
    a[REEF_CONV_SPLIT_K] = split; a[REEF_CONV_K_CHUNK] = k_chunk; a[REEF_CONV_M_TILES] = m_tiles;
    a[REEF_CONV_N_TILES] = n_tiles; a[REEF_CONV_ACT2] = 0; a[REEF_CONV_SYNC_OFF] = 0; a[REEF_CONV_MODE] = mode;
    a[REEF_CONV_DST_OFF] = 0;
    int s = 0;
    p->desc.ptr[s++] = const_cast<float*>(in);
    p->desc.ptr[s++] = const_cast<float*>(w);
    p->desc.ptr[s++] = out;
    if (bias) p->desc.ptr[s++] = const_cast<float*>(bias);
    if (residual) p->desc.ptr[s++] = const_cast<float*>(residual);
    p->ws_slot = s;
    p->sync_slot = s + 1;
    p->split_k = split;
    p->tiles = tiles;
    p->tasks = (uint32_t)(split * tiles);
    p->ws_floats = split > 1 ? (size_t)split * M * N : 0;
    return 0;
}

int launch(const Plan& p, hipStream_t stream) {
    size_t sz = sizeof(p.desc);
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<ReefOpDesc*>(&p.desc),
                     HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
    hipError_t e = hipModuleLaunchKernel(p.fn, p.tasks, 1, 1, REEF_WG_THREADS, 1, 1, 0, stream, nullptr, extra);
    return e == hipSuccess ? 0 : hip_fail(e, "hipModuleLaunchKernel");
}

}  // namespace

extern "C" {

int reef_ops_init(const char* kernels_co_path) {
    if (!kernels_co_path) return fail("reef_ops_init: null path");
    {
        std::lock_guard<std::mutex> lock(g_mtx);
        g_co_path = kernels_co_path;
    }
    hipError_t e = hipInit(0);
    if (e != hipSuccess) return hip_fail(e, "hipInit");
    DeviceState* d = nullptr;
    return ensure_device(&d);
}

size_t reef_ops_scratch_bytes(void) { return kWorkspaceBytes; }

int reef_ops_conv2d(const reef_conv2d_desc* c, const float* in, const float* w, const float* bias,
                    const float* residual, float* out, void* stream) {
    DeviceState* d = nullptr;
    if (int rc = ensure_device(&d)) return rc;
    Plan p;
    if (int rc = make_plan(*d, c, in, w, bias, residual, out, &p)) return rc;
    hipStream_t s = (hipStream_t)stream;
    void* ws = nullptr;
    void* cnt = nullptr;
    if (p.split_k > 1) {
        hipError_t e = hipMalloc(&ws, p.ws_floats * 4);
        if (e != hipSuccess) return hip_fail(e, "hipMalloc(workspace)");
        e = hipMalloc(&cnt, (size_t)p.tiles * 4);
        if (e != hipSuccess) {
            (void)hipFree(ws);
            return hip_fail(e, "hipMalloc(counters)");
        }
        hipLaunchKernelGGL(fill_words, dim3((p.tiles + 255) / 256), dim3(256), 0, s, (uint32_t*)cnt, 0u, (size_t)p.tiles);
        e = hipGetLastError();
        if (e != hipSuccess) {
            // the convolution would count on whatever the fresh allocation holds
            (void)hipFree(ws);
            (void)hipFree(cnt);
            return hip_fail(e, "fill_words(counters)");
        }
        p.desc.ptr[p.ws_slot] = ws;
        p.desc.ptr[p.sync_slot] = cnt;
    }
    int rc = launch(p, s);
    if (p.split_k > 1) {
        // the buffers live until the kernel is done with them
        hipError_t e = hipStreamSynchronize(s);
        const hipError_t f1 = hipFree(ws), f2 = hipFree(cnt);
        if (rc == 0 && e != hipSuccess) rc = hip_fail(e, "hipStreamSynchronize");
        if (rc == 0 && (f1 != hipSuccess || f2 != hipSuccess)) rc = hip_fail(f1 != hipSuccess ? f1 : f2, "hipFree");
    }
    return rc;
}

int reef_ops_conv2d_noalloc(const reef_conv2d_desc* c, const float* in, const float* w, const float* bias,
                            const float* residual, float* out, void* stream) {
    DeviceState* d = nullptr;
    if (int rc = ensure_device(&d, false)) return rc;   // set-up (module load, scratch address) is reef_ops_init's
    Plan p;
    if (int rc = make_plan(*d, c, in, w, bias, residual, out, &p)) return rc;
    hipStream_t s = (hipStream_t)stream;
    if (p.split_k > 1) {
        if (p.ws_floats * 4 > kWorkspaceBytes || (size_t)p.tiles * 4 > kCounterBytes) {
            char msg[200];
            std::snprintf(msg, sizeof(msg),
                          "reef_ops_conv2d_noalloc: the layer needs %zu bytes of partial tiles and %d counters; "
                          "the fixed scratch holds %zu bytes and %zu counters",
                          p.ws_floats * 4, p.tiles, kWorkspaceBytes, kCounterBytes / 4);
            return fail(msg);
        }
        uint32_t* cnt = (uint32_t*)d->scratch_ptr;
        float* ws = (float*)(d->scratch_ptr + kCounterBytes);
        // the array keeps what the last call left: the counters of this launch start at zero
        hipLaunchKernelGGL(fill_words, dim3((p.tiles + 255) / 256), dim3(256), 0, s, cnt, 0u, (size_t)p.tiles);
        // a fill that was not launched would leave the last call's counts in place: wrong sums, no error
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return hip_fail(e, "fill_words(counters)");
        p.desc.ptr[p.ws_slot] = ws;
        p.desc.ptr[p.sync_slot] = cnt;
    }
    return launch(p, s);
}

}  // extern "C"
