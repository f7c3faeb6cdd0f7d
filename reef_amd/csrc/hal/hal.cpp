// Backend-independent part of the C-ABI layer: the forwarding functions, the
// thread-local error string and the gfx950 occupancy model.
#include <algorithm>
#include <cstring>
#include <string>

#include "reef_hal.h"

namespace {
thread_local std::string g_err;
const reef_hal_backend* g_backend = nullptr;

inline const reef_hal_backend* be() { return g_backend ? g_backend : reef_hal_hip_backend(); }
}  // namespace

extern "C" {

const char* reef_hal_last_error(void) { return g_err.c_str(); }
void reef_hal_set_error(const char* msg) { g_err = msg ? msg : ""; }
void reef_hal_set_backend(const reef_hal_backend* b) { g_backend = b; }

int reef_hal_init(int device) { return be()->init(device); }
int reef_hal_device_info(reef_device_info* out) { return be()->device_info(out); }
int reef_hal_module_load(const char* path, reef_module_t* out) { return be()->module_load(path, out); }
int reef_hal_module_unload(reef_module_t mod) { return be()->module_unload(mod); }
int reef_hal_module_get_function(reef_module_t mod, const char* name, reef_function_t* out) {
    return be()->module_get_function(mod, name, out);
}
int reef_hal_function_resource(reef_function_t fn, reef_kernel_resource* out) {
    out->agprs = 0;   // a backend that knows nothing of accumulation registers leaves it
    return be()->function_resource(fn, out);
}
int reef_hal_module_kernel_entry(reef_module_t mod, const char* name, uint64_t* address) {
    if (!be()->module_kernel_entry) { if (address) *address = 0; return 0; }   // a backend without device code
    return be()->module_kernel_entry(mod, name, address);
}
int reef_hal_malloc(size_t bytes, int kind, reef_devptr_t* out) { return be()->malloc_(bytes, kind, out); }
int reef_hal_free(reef_devptr_t ptr, int kind) { return be()->free_(ptr, kind); }
int reef_hal_memset(reef_devptr_t ptr, int byte, size_t bytes) { return be()->memset_(ptr, byte, bytes); }
int reef_hal_memcpy_h2d(reef_devptr_t dst, const void* src, size_t bytes) {
    return be()->memcpy_h2d(dst, src, bytes);
}
int reef_hal_memcpy_d2h(void* dst, reef_devptr_t src, size_t bytes) {
    return be()->memcpy_d2h(dst, src, bytes);
}
int reef_hal_memset_async(reef_devptr_t ptr, int byte, size_t bytes, reef_stream_t s) {
    return be()->memset_async(ptr, byte, bytes, s);
}
int reef_hal_memcpy_h2d_async(reef_devptr_t dst, const void* src, size_t bytes, reef_stream_t s) {
    return be()->memcpy_h2d_async(dst, src, bytes, s);
}
int reef_hal_memcpy_d2h_async(void* dst, reef_devptr_t src, size_t bytes, reef_stream_t s) {
    return be()->memcpy_d2h_async(dst, src, bytes, s);
}
int reef_hal_stream_create(int launch_window, reef_stream_t* out) {
    return be()->stream_create(launch_window, out);
}
int reef_hal_stream_destroy(reef_stream_t s) { return be()->stream_destroy(s); }
int reef_hal_stream_sync(reef_stream_t s) { return be()->stream_sync(s); }
int reef_hal_stream_query(reef_stream_t s, int* idle) { return be()->stream_query(s, idle); }
int reef_hal_stream_drained(reef_stream_t s, int* drained) {
    if (be()->stream_drained) return be()->stream_drained(s, drained);
    return be()->stream_query(s, drained);
}
int reef_hal_device_sync(void) { return be()->device_sync(); }
int reef_hal_stream_pump(reef_stream_t s) { return be()->stream_pump(s); }
int reef_hal_launch(reef_function_t fn, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t dyn_lds, reef_stream_t s, const void* kernarg, size_t kernarg_bytes) {
    return be()->launch(fn, grid, block, dyn_lds, s, kernarg, kernarg_bytes);
}
int reef_hal_write_value32(reef_stream_t s, reef_devptr_t ptr, int32_t value) {
    return be()->write_value32(s, ptr, value);
}
int reef_hal_host_write32(reef_devptr_t ptr, int32_t value) { return be()->host_write32(ptr, value); }
int reef_hal_host_fill32(reef_devptr_t ptr, int32_t value, size_t n_words) {
    if (be()->host_fill32) return be()->host_fill32(ptr, value, n_words);
    for (size_t i = 0; i < n_words; i++)   // a backend without a call of its own: word by word
        if (int rc = be()->host_write32((char*)ptr + 4 * i, value)) return rc;
    return 0;
}
int reef_hal_stream_wait_device(reef_stream_t s) { return be()->stream_wait_device(s); }
int reef_hal_graph_begin(reef_stream_t s) { return be()->graph_begin(s); }
int reef_hal_graph_end(reef_stream_t s, reef_graph_t* out) { return be()->graph_end(s, out); }
int reef_hal_graph_launch(reef_graph_t g, reef_stream_t s) { return be()->graph_launch(g, s); }
int reef_hal_graph_destroy(reef_graph_t g) { return be()->graph_destroy(g); }
int reef_hal_stream_set_completion(reef_stream_t s, int mode) {
    return be()->stream_set_completion ? be()->stream_set_completion(s, mode) : 0;
}
int reef_hal_stream_progress(reef_stream_t s, uint32_t* submitted, uint32_t* done) {
    if (!be()->stream_progress) { reef_hal_set_error("stream_progress: not in this backend"); return 1; }
    return be()->stream_progress(s, submitted, done);
}
int reef_hal_stream_exit_ticks(reef_stream_t s, uint32_t seq, uint64_t* ticks) {
    if (!be()->stream_exit_ticks) { if (ticks) *ticks = 0; return 0; }
    return be()->stream_exit_ticks(s, seq, ticks);
}
int reef_hal_clock_sync(int64_t* host_ns, uint64_t* device_ticks, int64_t* err_ns, int* ticks_per_us) {
    if (!be()->clock_sync) { reef_hal_set_error("clock_sync: not in this backend"); return 1; }
    return be()->clock_sync(host_ns, device_ticks, err_ns, ticks_per_us);
}
int reef_hal_stream_clear_queue(reef_stream_t s, uint64_t* n_dropped) {
    return be()->stream_clear_queue(s, n_dropped);
}
int reef_hal_reset_cus(void) { return be()->reset_cus(); }
int reef_hal_event_create(reef_event_t* out) { return be()->event_create(out); }
int reef_hal_event_destroy(reef_event_t e) { return be()->event_destroy(e); }
int reef_hal_event_record(reef_event_t e, reef_stream_t s) { return be()->event_record(e, s); }
int reef_hal_event_sync(reef_event_t e) { return be()->event_sync(e); }
int reef_hal_event_elapsed_us(reef_event_t a, reef_event_t b, float* us) {
    return be()->event_elapsed_us(a, b, us);
}

// Workgroups of `block_threads` threads that fit on one CU.
//
// The reference's formula is for gfx906 (hip_impl.cpp:55-74): 256 VGPRs per
// lane and 10 waves per SIMD, 800 SGPRs, 64 KiB LDS (and it divides the LDS by
// the block size instead of by the LDS need, :66).  gfx950 has a unified
// 512-entry VGPR+AGPR file allocated in granules of 8, at most 8 waves per
// SIMD, 160 KiB LDS per CU allocated in granules of 1280 bytes; SGPRs no
// longer limit occupancy below 8 waves (102 per wave, 800 per SIMD).
int reef_hal_occupancy(const reef_kernel_resource* res, int block_threads, int dyn_lds,
                       int* blocks_per_cu) {
    reef_device_info di;
    if (reef_hal_device_info(&di) != 0) return 1;
    if (!res || block_threads <= 0 || !blocks_per_cu) {
        reef_hal_set_error("reef_hal_occupancy: bad argument");
        return 1;
    }
    const int gran = di.vgpr_granule > 0 ? di.vgpr_granule : 8;
    int vg = std::max(res->vgprs, 1);
    vg = (vg + gran - 1) / gran * gran;
    int waves_simd = std::min(di.vgprs_per_simd / vg, di.max_waves_per_simd);
    if (res->sgprs > 0) {
        const int sg = (res->sgprs + 15) / 16 * 16;
        waves_simd = std::min(waves_simd, std::max(800 / sg, 0));
    }
    const int waves_per_wg = (block_threads + 63) / 64;
    int blocks = waves_simd * di.simds_per_cu / waves_per_wg;
    const int lds = res->shared_memory + dyn_lds;
    if (lds > 0) {
        const int lg = di.lds_granule > 0 ? di.lds_granule : 1;
        const int need = (lds + lg - 1) / lg * lg;
        blocks = std::min(blocks, di.lds_bytes_per_cu / need);
    }
    blocks = std::min(blocks, di.max_wg_per_cu);
    if (di.max_threads_per_cu > 0)
        blocks = std::min(blocks, di.max_threads_per_cu / (waves_per_wg * 64));
    *blocks_per_cu = std::max(blocks, 0);
    return 0;
}

}  // extern "C"
