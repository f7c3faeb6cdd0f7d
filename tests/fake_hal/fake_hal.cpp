// A recording, host-memory backend for the C-ABI layer (include/reef_hal.h).
// TEST INFRASTRUCTURE: lets the executors and the scheduler run on a machine
// without a GPU.  "Device memory" is host memory; a launch is recorded and put
// in flight on its stream; kernels "complete" in FIFO order when the stream is
// queried (one per query, as if time passed), synchronised, or stepped by the
// test.  On completion an optional callback runs the kernel's effect (the tests
// plug the CPU oracle in there), so outputs are real.
//
// Launch-window semantics match the HIP backend: at most `window` kernels of a
// windowed stream are in flight, the rest wait in a host-side queue that
// stream_clear_queue drops.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "reef_hal.h"

struct reef_module_s { std::string path; };
struct reef_function_s { std::string name; std::string module_path; };

namespace {

struct Op {
    int kind;  // 0 kernel, 1 write32, 2 memcpy
    reef_function_s* fn;
    uint32_t grid[3], block[3], lds;
    std::vector<char> kernarg;
    int32_t* wptr; int32_t wval;
    void* dst; const void* src; size_t bytes;
};

}  // namespace

struct reef_stream_s {
    int id;
    int window;
    std::deque<Op> inflight, held;
};
struct reef_event_s { int dummy; };
struct reef_graph_s { std::vector<Op> ops; };

namespace {

typedef void (*kernel_cb_t)(const char* symbol, const char* module_path, const void* kernarg,
                            size_t kernarg_bytes, const uint32_t* grid, const uint32_t* block,
                            uint32_t lds, int stream_id);

std::recursive_mutex g_mtx;
reef_device_info g_info;
bool g_info_set = false;
kernel_cb_t g_cb = nullptr;
std::map<std::string, reef_kernel_resource> g_res;
std::vector<std::string> g_missing;
std::vector<reef_stream_s*> g_streams;
reef_stream_s g_null_stream{0, 0, {}, {}};
int g_next_stream = 1;
std::map<reef_stream_s*, std::vector<Op>> g_recording;
long g_graph_launches = 0;
long g_launches = 0, g_completed = 0, g_dropped = 0;
struct LogEntry { std::string symbol; int stream; uint32_t grid, block, lds; };
std::vector<LogEntry> g_log;
int g_auto_progress = 1;  // kernels completed per stream_query

reef_stream_s* S(reef_stream_t s) { return s ? s : &g_null_stream; }

void complete(reef_stream_s* st, Op& op) {
    if (op.kind == 0) {
        ++g_completed;
        if (g_cb) g_cb(op.fn->name.c_str(), op.fn->module_path.c_str(), op.kernarg.data(), op.kernarg.size(),
                       op.grid, op.block, op.lds, st->id);
    } else if (op.kind == 1) {
        *op.wptr = op.wval;
    } else {
        std::memcpy(op.dst, op.src, op.bytes);
    }
}
int n_kernels_inflight(reef_stream_s* st) {
    int n = 0;
    for (auto& o : st->inflight) n += o.kind == 0;
    return n;
}
void pump(reef_stream_s* st) {
    while (!st->held.empty() && (st->window <= 0 || n_kernels_inflight(st) < st->window)) {
        st->inflight.push_back(std::move(st->held.front()));
        st->held.pop_front();
    }
}
void progress(reef_stream_s* st, int n) {
    while (n-- > 0 && !st->inflight.empty()) {
        Op op = std::move(st->inflight.front());
        st->inflight.pop_front();
        complete(st, op);
        pump(st);
    }
    // non-kernel ops at the head run at once
    while (!st->inflight.empty() && st->inflight.front().kind != 0) {
        Op op = std::move(st->inflight.front());
        st->inflight.pop_front();
        complete(st, op);
    }
}
void enqueue(reef_stream_s* st, Op&& op) {
    if (!st->held.empty() || (st->window > 0 && op.kind == 0 && n_kernels_inflight(st) >= st->window)) {
        st->held.push_back(std::move(op));
    } else if (op.kind != 0 && st->inflight.empty()) {
        complete(st, op);
    } else {
        st->inflight.push_back(std::move(op));
    }
}
void drain(reef_stream_s* st) {
    for (;;) {
        pump(st);
        if (st->inflight.empty()) break;
        progress(st, 1);
    }
}

int f_init(int) { return 0; }
int f_device_info(reef_device_info* out) {
    if (!g_info_set) {
        std::memset(&g_info, 0, sizeof(g_info));
        g_info.num_cus = 256; g_info.num_xcds = 8; g_info.simds_per_cu = 4;
        g_info.max_waves_per_simd = 8; g_info.vgprs_per_simd = 512; g_info.vgpr_granule = 8;
        g_info.lds_bytes_per_cu = 160 * 1024; g_info.lds_granule = 1280; g_info.max_wg_per_cu = 32; g_info.max_threads_per_cu = 2048;
        g_info.clock_khz = 2400000; std::strcpy(g_info.arch, "fake");
        g_info_set = true;
    }
    *out = g_info;
    return 0;
}
int f_module_load(const char* path, reef_module_t* out) {
    FILE* fp = std::fopen(path, "rb");
    if (!fp) { reef_hal_set_error((std::string("fake: cannot open ") + path).c_str()); return 1; }
    std::fclose(fp);
    *out = new reef_module_s{path};
    return 0;
}
int f_module_unload(reef_module_t m) { delete m; return 0; }
int f_get_function(reef_module_t m, const char* name, reef_function_t* out) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    for (auto& miss : g_missing)
        if (miss == name) { reef_hal_set_error((std::string("fake: no symbol ") + name).c_str()); return 1; }
    *out = new reef_function_s{name, m->path};
    return 0;
}
int f_function_resource(reef_function_t f, reef_kernel_resource* out) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    auto it = g_res.find(f->name);
    if (it != g_res.end()) *out = it->second;
    else *out = reef_kernel_resource{0, 32, 16, 0};
    return 0;
}
std::map<char*, size_t> g_allocs;
int f_malloc(size_t bytes, int, reef_devptr_t* out) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    if (!bytes) bytes = 4;
    *out = std::calloc(1, bytes);
    if (!*out) return 1;
    g_allocs[(char*)*out] = bytes;
    return 0;
}
int f_free(reef_devptr_t p, int) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    g_allocs.erase((char*)p);
    std::free(p);
    return 0;
}
int f_memset(reef_devptr_t p, int b, size_t n) { std::memset(p, b, n); return 0; }
int f_h2d(reef_devptr_t d, const void* s, size_t n) { std::memcpy(d, s, n); return 0; }
int f_d2h(void* d, reef_devptr_t s, size_t n) { std::memcpy(d, s, n); return 0; }
int f_copy_async(void* d, const void* s, size_t n, reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    Op op{}; op.kind = 2; op.dst = d; op.src = s; op.bytes = n;
    enqueue(S(st), std::move(op));
    return 0;
}
int f_h2d_async(reef_devptr_t d, const void* s, size_t n, reef_stream_t st) { return f_copy_async(d, s, n, st); }
int f_d2h_async(void* d, reef_devptr_t s, size_t n, reef_stream_t st) { return f_copy_async(d, s, n, st); }
int f_stream_create(int window, reef_stream_t* out) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    reef_stream_s* st = new reef_stream_s{g_next_stream++, window, {}, {}};
    g_streams.push_back(st);
    *out = st;
    return 0;
}
int f_stream_destroy(reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    if (!st) return 0;
    drain(st);
    for (auto& p : g_streams) if (p == st) p = nullptr;
    delete st;
    return 0;
}
int f_stream_sync(reef_stream_t st) { std::lock_guard<std::recursive_mutex> lock(g_mtx); drain(S(st)); return 0; }
int f_stream_query(reef_stream_t st, int* idle) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    reef_stream_s* s = S(st);
    pump(s);
    progress(s, g_auto_progress);
    *idle = s->inflight.empty() && s->held.empty();
    return 0;
}
int f_device_sync() {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    drain(&g_null_stream);
    for (auto* s : g_streams) if (s) drain(s);
    return 0;
}
int f_stream_pump(reef_stream_t st) { std::lock_guard<std::recursive_mutex> lock(g_mtx); pump(S(st)); return 0; }
int f_launch(reef_function_t f, const uint32_t* g, const uint32_t* b, uint32_t lds, reef_stream_t st,
             const void* kernarg, size_t bytes) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    Op op{};
    op.kind = 0; op.fn = f; op.lds = lds;
    std::memcpy(op.grid, g, sizeof(op.grid));
    std::memcpy(op.block, b, sizeof(op.block));
    op.kernarg.assign((const char*)kernarg, (const char*)kernarg + bytes);
    auto rec = g_recording.find(S(st));
    if (rec != g_recording.end()) {
        rec->second.push_back(std::move(op));
        return 0;
    }
    ++g_launches;
    g_log.push_back(LogEntry{f->name, S(st)->id, g[0] * g[1] * g[2], b[0] * b[1] * b[2], lds});
    enqueue(S(st), std::move(op));
    return 0;
}
int f_write_value32(reef_stream_t st, reef_devptr_t p, int32_t v) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    Op op{}; op.kind = 1; op.wptr = (int32_t*)p; op.wval = v;
    enqueue(S(st), std::move(op));
    return 0;
}
int f_clear_queue(reef_stream_t st, uint64_t* n) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    reef_stream_s* s = S(st);
    uint64_t d = 0;
    for (auto& o : s->held) d += o.kind == 0;
    s->held.clear();
    g_dropped += (long)d;
    if (n) *n = d;
    return 0;
}
int f_reset_cus() { return 0; }
int f_memset_async(reef_devptr_t p, int b, size_t n, reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    drain(S(st));   // keeps stream order without a fill op type
    std::memset(p, b, n);
    return 0;
}
int f_host_write32(reef_devptr_t p, int32_t v) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    *(int32_t*)p = v;
    return 0;
}
// everything already "on the device" completes; held launches stay held
int f_stream_wait_device(reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    reef_stream_s* s = S(st);
    while (!s->inflight.empty()) {
        Op op = std::move(s->inflight.front());
        s->inflight.pop_front();
        complete(s, op);
    }
    return 0;
}
// graphs: launches on a recording stream are kept aside and replayed as ordinary launches
int f_graph_begin(reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    reef_stream_s* s = S(st);
    if (s->window > 0 || g_recording.count(s)) return 1;
    g_recording[s] = {};
    return 0;
}
int f_graph_end(reef_stream_t st, reef_graph_t* out) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    auto it = g_recording.find(S(st));
    if (it == g_recording.end()) return 1;
    *out = new reef_graph_s{std::move(it->second)};
    g_recording.erase(it);
    return 0;
}
int f_graph_launch(reef_graph_t g, reef_stream_t st) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    if (!g || S(st)->window > 0) return 1;
    ++g_graph_launches;
    for (const Op& o : g->ops) {
        Op op = o;
        ++g_launches;
        g_log.push_back(LogEntry{op.fn->name, S(st)->id, op.grid[0] * op.grid[1] * op.grid[2],
                                 op.block[0] * op.block[1] * op.block[2], op.lds});
        enqueue(S(st), std::move(op));
    }
    return 0;
}
int f_graph_destroy(reef_graph_t g) { delete g; return 0; }
int f_event_create(reef_event_t* out) { *out = new reef_event_s{0}; return 0; }
int f_event_destroy(reef_event_t e) { delete e; return 0; }
int f_event_record(reef_event_t, reef_stream_t) { return 0; }
int f_event_sync(reef_event_t) { return f_device_sync(); }
int f_event_elapsed(reef_event_t, reef_event_t, float* us) { *us = 1.0f; return 0; }

const reef_hal_backend kFake = {
    f_init, f_device_info, f_module_load, f_module_unload, f_get_function, f_function_resource,
    f_malloc, f_free, f_memset, f_h2d, f_d2h, f_h2d_async, f_d2h_async, f_stream_create,
    f_stream_destroy, f_stream_sync, f_stream_query, f_device_sync, f_stream_pump, f_launch,
    f_write_value32, f_clear_queue, f_reset_cus, f_event_create, f_event_destroy, f_event_record,
    f_event_sync, f_event_elapsed, f_memset_async, f_host_write32, f_stream_wait_device,
    f_graph_begin, f_graph_end, f_graph_launch, f_graph_destroy,
};

}  // namespace

extern "C" {
const reef_hal_backend* fake_hal_backend(void) { return &kFake; }
void fake_hal_set_callback(kernel_cb_t cb) { std::lock_guard<std::recursive_mutex> lock(g_mtx); g_cb = cb; }
void fake_hal_set_device(const reef_device_info* info) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    g_info = *info;
    g_info_set = true;
}
void fake_hal_set_kernel_resource(const char* name, int lds, int vgprs, int sgprs, int stack) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    g_res[name] = reef_kernel_resource{lds, vgprs, sgprs, stack};
}
void fake_hal_set_missing(const char* name) { std::lock_guard<std::recursive_mutex> lock(g_mtx); g_missing.push_back(name); }
void fake_hal_set_auto_progress(int n) { g_auto_progress = n; }
void fake_hal_reset(void) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    g_launches = g_completed = g_dropped = 0;
    g_graph_launches = 0;
    g_recording.clear();
    g_log.clear();
    g_res.clear();
    g_missing.clear();
    g_info_set = false;
    g_auto_progress = 1;
}
// Bytes from `p` to the end of the allocation that holds it (0 when unknown).
size_t fake_hal_extent(const void* p) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    auto it = g_allocs.upper_bound((char*)p);
    if (it == g_allocs.begin()) return 0;
    --it;
    const char* end = it->first + it->second;
    return (const char*)p < end ? (size_t)(end - (const char*)p) : 0;
}
long fake_hal_launches(void) { return g_launches; }
long fake_hal_completed(void) { return g_completed; }
long fake_hal_dropped(void) { return g_dropped; }
long fake_hal_graph_launches(void) { return g_graph_launches; }
long fake_hal_log_size(void) { std::lock_guard<std::recursive_mutex> lock(g_mtx); return (long)g_log.size(); }
int fake_hal_log_entry(long i, char* symbol, size_t cap, int* stream, uint32_t* grid, uint32_t* block,
                       uint32_t* lds) {
    std::lock_guard<std::recursive_mutex> lock(g_mtx);
    if (i < 0 || i >= (long)g_log.size()) return 1;
    std::strncpy(symbol, g_log[i].symbol.c_str(), cap - 1);
    symbol[cap - 1] = 0;
    *stream = g_log[i].stream; *grid = g_log[i].grid; *block = g_log[i].block; *lds = g_log[i].lds;
    return 0;
}
}
