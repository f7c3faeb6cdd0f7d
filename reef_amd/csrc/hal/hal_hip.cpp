// HIP backend of the C-ABI layer (stock ROCm, no patched runtime).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "hal/code_object.h"
#include "reef_hal.h"

// hal_device.hip
int reef_hal_hip_fill(hipStream_t stream, void* p, int byte, size_t n);
int reef_hal_hip_clock_probe(hipStream_t stream, int64_t* host_ns, uint64_t* device_ticks, int64_t* err_ns,
                             int* ticks_per_us);

struct reef_module_s {
    hipModule_t mod;
    std::map<std::string, reef::hal::KernelMeta> meta;
    std::vector<reef_function_s*> fns;
};
struct reef_function_s {
    hipFunction_t fn;
    reef::hal::KernelMeta meta;
    bool has_meta;
    std::string name;
};

namespace {

// One launch a windowed stream keeps on the host.  The argument block is stored
// inline and the queue is a ring that never shrinks, so that dropping the whole
// queue (the first step of a preemption) costs no allocator calls.
constexpr size_t kMaxHeldKernarg = 512;
struct Held {
    hipFunction_t fn;
    uint32_t grid[3], block[3], lds, bytes;
    alignas(16) char kernarg[kMaxHeldKernarg];
};
struct HeldRing {
    std::vector<Held> slots;
    size_t head = 0, count = 0;
    bool empty() const { return count == 0; }
    size_t size() const { return count; }
    Held& front() { return slots[head]; }
    void pop_front() { head = (head + 1) % slots.size(); --count; }
    void clear() { head = 0; count = 0; }
    Held& push_back() {
        if (count == slots.size()) {
            std::vector<Held> bigger(slots.empty() ? 1024 : slots.size() * 2);
            for (size_t i = 0; i < count; i++) bigger[i] = slots[(head + i) % slots.size()];
            slots.swap(bigger);
            head = 0;
        }
        Held& h = slots[(head + count) % slots.size()];
        ++count;
        return h;
    }
};

}  // namespace

// A stream with an optional launch window.  `done` is a pinned host word the
// device writes after every kernel of a windowed stream; submitted - *done is
// the number of kernels still on the device.
//
// A windowed stream is served by a feeder thread that moves held launches to the
// device as the window frees up.  The caller of reef_hal_launch (the scheduler
// thread) then only copies the launch into the ring; the runtime call per kernel
// (3 us of host time) is paid by the feeder, so several best-effort streams are fed in
// parallel instead of one after the other from the scheduler's loop.  Feeders are a
// small pool (Feeder below): the first streams get a thread each, further streams
// share them, so the host cores this costs do not grow with the number of queues.
// `mtx` guards the ring and `submitted` and is only held for copies; `submit_mtx` is
// held around the runtime calls on the HIP stream.  A launch counts as in flight from the moment the feeder takes it out
// of the ring, so "ring dropped + at most `window` kernels not known complete" -- what
// the rollback after a preemption relies on -- holds at every instant.
constexpr int kExitRing = 8;   // launches whose exit clock is kept

namespace {
struct Feeder;
}

struct reef_stream_s {
    hipStream_t s;
    int window;
    int completion = REEF_COMPLETE_STREAM_WRITE;
    volatile uint64_t* exit_ticks = nullptr;   // pinned, kExitRing slots (slot = seq % kExitRing)
    uint32_t* exit_count = nullptr;            // device counter of workgroups that have left
    uint32_t submitted;
    volatile uint32_t* done;
    HeldRing held;
    std::mutex mtx;
    std::mutex submit_mtx;
    Feeder* feeder = nullptr;            // the pool thread that serves this stream
    std::atomic<int> feeder_error{0};
    std::atomic<size_t> held_count{0};   // mirror of held.size(), readable without mtx
    std::atomic<uint32_t> enqueued{0};   // highest seq whose runtime calls have returned
    bool has_feeder = false;
};

struct reef_graph_s {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

namespace {

int fail(hipError_t e, const char* what) {
    std::string m = std::string(what) + ": " + hipGetErrorString(e);
    reef_hal_set_error(m.c_str());
    return 1;
}
#define HIPCHK(call)                          \
    do {                                      \
        hipError_t _e = (call);               \
        if (_e != hipSuccess) return fail(_e, #call); \
    } while (0)

int g_device = 0;
bool g_host_visible = false;       // device memory can be stored to from the host (large BAR)
hipStream_t g_flag_stream = nullptr;  // fallback path of host_write32

// Streams draw their hardware queue from a per-process pool (GPU_MAX_HW_QUEUES entries, 4 unless
// the environment says otherwise): the first streams each open a new queue, later ones join the
// queue with the fewest users.  Left alone, the pool fills up with whichever streams happen to
// come first, and two best-effort streams can end up on one hardware queue, where their kernels
// run strictly one after the other (measured with 4 DenseNet-201 clients: 408 inferences/s and a
// 30 us preemption drain that way, 688 inferences/s and 19 us when no two of them share).  So
// the pool is opened here, once, by idle streams that are kept for the life of the process: every
// stream created afterwards joins the least used queue, which spreads up to a pool's worth of
// best-effort streams over different queues.  REEF_HAL_HOLD_QUEUES=0 turns this off.
std::vector<hipStream_t> g_queue_holders;
int hold_hardware_queues() {
    if (!g_queue_holders.empty()) return 0;
    if (const char* v = std::getenv("REEF_HAL_HOLD_QUEUES"))
        if (std::atoi(v) == 0) return 0;
    int pool = 4;
    if (const char* v = std::getenv("GPU_MAX_HW_QUEUES"))
        if (std::atoi(v) > 0) pool = std::atoi(v);
    if (pool > 32) pool = 32;
    for (int i = 0; i < pool; ++i) {
        hipStream_t s;
        HIPCHK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        HIPCHK(hipStreamSynchronize(s));
        g_queue_holders.push_back(s);
    }
    return 0;
}

int h_init(int device) {
    HIPCHK(hipInit(0));
    int n = 0;
    HIPCHK(hipGetDeviceCount(&n));
    if (device < 0 || device >= n) {
        reef_hal_set_error("reef_hal_init: no such device");
        return 1;
    }
    g_device = device;
    HIPCHK(hipSetDevice(device));
    int large_bar = 0;
    if (hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, device) == hipSuccess)
        g_host_visible = large_bar != 0;
    return hold_hardware_queues();
}

int h_device_info(reef_device_info* out) {
    if (!out) return 1;
    std::memset(out, 0, sizeof(*out));
    hipDeviceProp_t p;
    HIPCHK(hipGetDeviceProperties(&p, g_device));
    out->num_cus = p.multiProcessorCount;
    out->num_xcds = 8;
    if (out->num_cus % out->num_xcds != 0) out->num_xcds = 1;
    out->simds_per_cu = 4;
    out->max_waves_per_simd = 8;
    out->vgprs_per_simd = 512;
    out->vgpr_granule = 8;
    out->lds_bytes_per_cu = 160 * 1024;
    out->lds_granule = 1280;
    out->max_wg_per_cu = 32;
    out->max_threads_per_cu = 2048;
    out->clock_khz = p.clockRate;
    std::strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
    if (char* c = std::strchr(out->arch, ':')) *c = 0;
    return 0;
}

int h_module_load(const char* path, reef_module_t* out) {
    reef_module_s* m = new reef_module_s;
    hipError_t e = hipModuleLoad(&m->mod, path);
    if (e != hipSuccess) {
        delete m;
        return fail(e, (std::string("hipModuleLoad ") + path).c_str());
    }
    std::string err;
    if (!reef::hal::read_code_object_metadata(path, &m->meta, &err)) m->meta.clear();
    *out = m;
    return 0;
}

int h_module_unload(reef_module_t m) {
    if (!m) return 0;
    hipError_t e = hipModuleUnload(m->mod);
    for (auto* f : m->fns) delete f;
    delete m;
    return e == hipSuccess ? 0 : fail(e, "hipModuleUnload");
}

int h_module_get_function(reef_module_t m, const char* name, reef_function_t* out) {
    hipFunction_t fn;
    hipError_t e = hipModuleGetFunction(&fn, m->mod, name);
    if (e != hipSuccess) return fail(e, (std::string("hipModuleGetFunction ") + name).c_str());
    reef_function_s* f = new reef_function_s;
    f->fn = fn;
    f->name = name;
    auto it = m->meta.find(name);
    f->has_meta = it != m->meta.end();
    if (f->has_meta) f->meta = it->second;
    m->fns.push_back(f);
    *out = f;
    return 0;
}

int h_function_resource(reef_function_t f, reef_kernel_resource* out) {
    if (!f->has_meta) {
        reef_hal_set_error(("no metadata for kernel " + f->name).c_str());
        return 1;
    }
    out->shared_memory = f->meta.lds;
    // On gfx90a and later .vgpr_count is already the unified total (arch VGPRs
    // rounded to 4, plus AGPRs).
    out->vgprs = f->meta.vgprs;
    out->sgprs = f->meta.sgprs;
    out->stack_size = f->meta.scratch;
    out->agprs = f->meta.agprs;
    return 0;
}

int h_module_kernel_entry(reef_module_t m, const char* name, uint64_t* address) {
    if (!m || !name || !address) { reef_hal_set_error("reef_hal_module_kernel_entry: null argument"); return 1; }
    hipDeviceptr_t var = nullptr;
    size_t bytes = 0;
    const std::string sym = std::string(name) + "_entry";
    hipError_t e = hipModuleGetGlobal(&var, &bytes, m->mod, sym.c_str());
    if (e != hipSuccess) return fail(e, ("hipModuleGetGlobal " + sym).c_str());
    if (bytes != sizeof(uint64_t)) { reef_hal_set_error((sym + ": not an 8-byte variable").c_str()); return 1; }
    HIPCHK(hipMemcpy(address, var, sizeof(uint64_t), hipMemcpyDeviceToHost));
    return 0;
}

int h_malloc(size_t bytes, int kind, reef_devptr_t* out) {
    if (bytes == 0) bytes = 4;
    switch (kind) {
        case REEF_MEM_DEVICE: HIPCHK(hipMalloc(out, bytes)); break;
        case REEF_MEM_DEVICE_FINEGRAINED:
            HIPCHK(hipExtMallocWithFlags(out, bytes, hipDeviceMallocFinegrained));
            break;
        case REEF_MEM_HOST_PINNED: HIPCHK(hipHostMalloc(out, bytes, hipHostMallocDefault)); break;
        default: reef_hal_set_error("reef_hal_malloc: bad kind"); return 1;
    }
    return 0;
}
int h_free(reef_devptr_t p, int kind) {
    if (kind == REEF_MEM_HOST_PINNED) HIPCHK(hipHostFree(p));
    else HIPCHK(hipFree(p));
    return 0;
}
int h_memset(reef_devptr_t p, int byte, size_t n) { HIPCHK(hipMemset(p, byte, n)); return 0; }
int h_h2d(reef_devptr_t d, const void* s, size_t n) { HIPCHK(hipMemcpy(d, s, n, hipMemcpyHostToDevice)); return 0; }
int h_d2h(void* d, reef_devptr_t s, size_t n) { HIPCHK(hipMemcpy(d, s, n, hipMemcpyDeviceToHost)); return 0; }
int h_h2d_async(reef_devptr_t d, const void* s, size_t n, reef_stream_t st) {
    HIPCHK(hipMemcpyAsync(d, s, n, hipMemcpyHostToDevice, st ? st->s : nullptr));
    return 0;
}
int h_d2h_async(void* d, reef_devptr_t s, size_t n, reef_stream_t st) {
    HIPCHK(hipMemcpyAsync(d, s, n, hipMemcpyDeviceToHost, st ? st->s : nullptr));
    return 0;
}

int submit(reef_stream_t st, hipFunction_t fn, const uint32_t* g, const uint32_t* b, uint32_t lds,
           const void* kernarg, size_t bytes, uint32_t seq);
inline uint32_t in_flight(reef_stream_t st) { return st->submitted - *st->done; }

// Moves held launches to the device while the window has room.  Caller holds st->mtx.
int pump_locked(reef_stream_t st) {
    while (!st->held.empty() && (int)in_flight(st) < st->window) {
        Held& h = st->held.front();
        int rc = submit(st, h.fn, h.grid, h.block, h.lds, h.kernarg, h.bytes, ++st->submitted);
        st->held.pop_front();
        st->held_count.store(st->held.size(), std::memory_order_release);
        if (rc) return rc;
    }
    return 0;
}

// One thread of the feeder pool and the windowed streams it serves.
//
// While a best-effort model runs, its stream's window is full most of the time and its kernels
// take a few microseconds -- far below what a sleep costs -- so a feeder polls the completion
// words of its streams: one busy host core per feeder while any of its streams has launches
// held.  With a thread per stream that was one core per best-effort queue (32 at the
// reference's queue limit).  The pool has kMaxFeeders threads (REEF_HAL_FEEDERS, default 4: the
// number of hardware queues a process gets, i.e. of best-effort streams that can really run
// side by side); stream k is served by feeder k mod n.  Streams that share a feeder also share
// the device, so each needs its window refilled proportionally less often.
//
// A feeder looks at the ring sizes and the windows through lock-free mirrors and only takes a
// stream's locks when there is a launch to move: a thread that re-takes a mutex in a tight loop
// starves whoever else wants it (here the scheduler thread in the middle of a preemption) for
// milliseconds.
struct Feeder {
    std::thread th;
    std::mutex mtx;                        // guards `streams`; the condition variable's mutex
    std::condition_variable cv;            // a launch was held on one of the streams, or the list changed
    std::vector<reef_stream_s*> streams;
    std::atomic<uint32_t> version{0};      // bumped whenever `streams` changes
    std::atomic<uint32_t> seen{0};         // the version the thread is working with
};
constexpr int kMaxFeeders = 16;
Feeder* g_feeders[kMaxFeeders] = {};
int g_n_feeders = 0;                       // pool size, fixed when the first windowed stream is made
unsigned g_next_feeder = 0;
std::mutex g_feeders_mtx;

// Moves one held launch of `st` to the device if its window has room.  Returns true when it did.
bool feed_one(reef_stream_s* st, Held& h) {
    // `submitted` only changes in the stream's feeder thread
    if ((int)in_flight(st) >= st->window) return false;
    std::lock_guard<std::mutex> sub(st->submit_mtx);
    uint32_t seq = 0;
    {
        std::lock_guard<std::mutex> lock(st->mtx);
        if (st->held.empty()) return false;   // dropped in the meantime
        h = st->held.front();
        st->held.pop_front();
        st->held_count.store(st->held.size(), std::memory_order_release);
        seq = ++st->submitted;   // in flight from now on
    }
    if (submit(st, h.fn, h.grid, h.block, h.lds, h.kernarg, h.bytes, seq) != 0) st->feeder_error.store(1);
    return true;
}

void feeder_main(Feeder* f) {
    hipSetDevice(g_device);
    std::vector<reef_stream_s*> mine;
    uint32_t ver = ~0u;
    int idle_spins = 0, full_spins = 0;
    Held h;
    for (;;) {   // pool threads live as long as the process
        const uint32_t v = f->version.load(std::memory_order_acquire);
        if (v != ver) {
            std::lock_guard<std::mutex> lock(f->mtx);
            mine = f->streams;
            ver = f->version.load(std::memory_order_acquire);
            f->seen.store(ver, std::memory_order_release);   // a stream taken off the list is not touched again
        }
        bool any_held = false, fed = false;
        for (reef_stream_s* st : mine) {
            if (st->held_count.load(std::memory_order_acquire) == 0) continue;
            any_held = true;
            fed = feed_one(st, h) || fed;
        }
        if (fed) {
            idle_spins = full_spins = 0;
            continue;
        }
        if (!any_held) {
            // nothing to feed: after a while sleep until a launch is held (bounded, so that a
            // missed wake-up costs little)
            full_spins = 0;
            if (++idle_spins > 2000) {
                std::unique_lock<std::mutex> lock(f->mtx);
                if (f->version.load(std::memory_order_acquire) == ver)
                    f->cv.wait_for(lock, std::chrono::microseconds(mine.empty() ? 20000 : 200));
                idle_spins = 0;
            } else {
                __builtin_ia32_pause();
            }
            continue;
        }
        // every stream with held launches has a full window: the steady state while best-effort
        // models run.  Behind kernels that run for long the core is given away.
        idle_spins = 0;
        if (++full_spins > 20000) std::this_thread::yield();
        else __builtin_ia32_pause();
    }
}

// The feeder a new windowed stream is served by; starts the pool on first use.
Feeder* attach_feeder(reef_stream_s* st) {
    std::lock_guard<std::mutex> pool(g_feeders_mtx);
    if (g_n_feeders == 0) {
        int n = 4;
        if (const char* v = std::getenv("REEF_HAL_FEEDERS")) n = std::atoi(v);
        g_n_feeders = std::max(1, std::min(n, kMaxFeeders));
    }
    Feeder*& f = g_feeders[g_next_feeder++ % (unsigned)g_n_feeders];
    if (!f) {
        f = new Feeder;                    // never deleted: its thread runs until the process ends
        f->th = std::thread(feeder_main, f);
        f->th.detach();
    }
    {
        std::lock_guard<std::mutex> lock(f->mtx);
        f->streams.push_back(st);
        f->version.fetch_add(1, std::memory_order_release);
    }
    f->cv.notify_all();
    return f;
}

// Takes a stream off its feeder's list and waits until the thread has let go of it.
void detach_feeder(reef_stream_s* st) {
    Feeder* f = st->feeder;
    uint32_t want;
    {
        std::lock_guard<std::mutex> lock(f->mtx);
        for (size_t i = 0; i < f->streams.size(); ++i)
            if (f->streams[i] == st) {
                f->streams.erase(f->streams.begin() + (long)i);
                break;
            }
        want = f->version.fetch_add(1, std::memory_order_release) + 1;
    }
    f->cv.notify_all();
    while ((int32_t)(f->seen.load(std::memory_order_acquire) - want) < 0) std::this_thread::sleep_for(std::chrono::microseconds(50));
    st->feeder = nullptr;
}

bool g_use_feeder = true;

int h_stream_create(int window, reef_stream_t* out) {
    reef_stream_s* st = new reef_stream_s;
    st->window = window;
    st->submitted = 0;
    st->done = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&st->s, hipStreamNonBlocking);
    if (e != hipSuccess) { delete st; return fail(e, "hipStreamCreateWithFlags"); }
    if (window > 0) {
        void* p = nullptr;
        // one pinned block: the completion word, and from byte 64 on the exit clocks of the
        // last launches (8-byte slots)
        e = hipHostMalloc(&p, 64 + 8 * kExitRing, hipHostMallocDefault);
        if (e != hipSuccess) { hipStreamDestroy(st->s); delete st; return fail(e, "hipHostMalloc"); }
        std::memset(p, 0, 64 + 8 * kExitRing);
        st->done = (volatile uint32_t*)p;
        st->exit_ticks = (volatile uint64_t*)((char*)p + 64);
        void* cnt = nullptr;
        e = hipMalloc(&cnt, 64);
        if (e == hipSuccess) e = hipMemset(cnt, 0, 64);
        if (e != hipSuccess) { hipStreamDestroy(st->s); hipHostFree(p); delete st; return fail(e, "hipMalloc"); }
        st->exit_count = (uint32_t*)cnt;
        if (const char* v = std::getenv("REEF_HAL_FEEDER")) g_use_feeder = std::atoi(v) != 0;
        if (g_use_feeder) {
            st->has_feeder = true;
            st->feeder = attach_feeder(st);
        }
    }
    *out = st;
    return 0;
}
int h_stream_destroy(reef_stream_t st) {
    if (!st) return 0;
    if (st->has_feeder) detach_feeder(st);
    hipStreamSynchronize(st->s);
    hipStreamDestroy(st->s);
    if (st->done) hipHostFree((void*)st->done);
    if (st->exit_count) hipFree(st->exit_count);
    delete st;
    return 0;
}

// `seq` != 0: the launch belongs to a windowed stream and is its seq-th; the device writes
// seq to the stream's completion word when the kernel has finished.
int submit(reef_stream_t st, hipFunction_t fn, const uint32_t* g, const uint32_t* b, uint32_t lds,
           const void* kernarg, size_t bytes, uint32_t seq) {
    size_t sz = bytes;
    alignas(16) char patched[kMaxHeldKernarg];
    const bool in_kernel = seq != 0 && st->completion == REEF_COMPLETE_IN_KERNEL;
    if (in_kernel) {
        // the kernel signals by itself: its argument block starts with the completion record
        if (bytes < sizeof(reef_hal_completion) || bytes > sizeof(patched)) {
            reef_hal_set_error("reef_hal_launch: argument block cannot hold a completion record");
            return 1;
        }
        std::memcpy(patched, kernarg, bytes);
        reef_hal_completion c;
        c.done_word = (uint32_t*)st->done;
        c.exit_ticks = (uint64_t*)&st->exit_ticks[seq % kExitRing];
        c.exit_count = st->exit_count;
        c.seq = seq;
        c.reserved = 0;
        std::memcpy(patched, &c, sizeof(c));
        kernarg = patched;
    }
    void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(kernarg),
                     HIP_LAUNCH_PARAM_BUFFER_SIZE, &sz, HIP_LAUNCH_PARAM_END};
    HIPCHK(hipModuleLaunchKernel(fn, g[0], g[1], g[2], b[0], b[1], b[2], lds, st ? st->s : nullptr,
                                 nullptr, extra));
    if (seq != 0) {
        if (!in_kernel) HIPCHK(hipStreamWriteValue32(st->s, (void*)st->done, seq, 0));
        st->enqueued.store(seq, std::memory_order_release);
    }
    return 0;
}

int h_stream_pump(reef_stream_t st) {
    if (!st || st->window <= 0) return 0;
    if (st->has_feeder) return st->feeder_error.load() ? 1 : 0;   // the feeder does it
    std::lock_guard<std::mutex> lock(st->mtx);
    return pump_locked(st);
}

int h_launch(reef_function_t f, const uint32_t* g, const uint32_t* b, uint32_t lds, reef_stream_t st,
             const void* kernarg, size_t bytes) {
    if (st && st->window > 0) {
        if (bytes > kMaxHeldKernarg) {
            reef_hal_set_error("reef_hal_launch: argument block too large for a windowed stream");
            return 1;
        }
        std::unique_lock<std::mutex> lock(st->mtx);
        if (!st->has_feeder) {
            if (int rc = pump_locked(st)) return rc;
            if (st->held.empty() && (int)in_flight(st) < st->window)
                return submit(st, f->fn, g, b, lds, kernarg, bytes, ++st->submitted);
        }
        const bool was_empty = st->held.empty();
        Held& h = st->held.push_back();
        h.fn = f->fn;
        std::memcpy(h.grid, g, sizeof(h.grid));
        std::memcpy(h.block, b, sizeof(h.block));
        h.lds = lds;
        h.bytes = (uint32_t)bytes;
        std::memcpy(h.kernarg, kernarg, bytes);
        st->held_count.store(st->held.size(), std::memory_order_release);
        lock.unlock();
        if (st->has_feeder && was_empty) st->feeder->cv.notify_one();
        return st->feeder_error.load() ? 1 : 0;
    }
    return submit(st, f->fn, g, b, lds, kernarg, bytes, 0);
}

// Waits until the ring of a windowed stream is empty (everything handed to the device).
int drain_ring(reef_stream_t st) {
    for (;;) {
        {
            std::lock_guard<std::mutex> lock(st->mtx);
            if (!st->has_feeder) {
                if (int rc = pump_locked(st)) return rc;
            }
            if (st->held.empty()) return st->feeder_error.load() ? 1 : 0;
        }
        __builtin_ia32_pause();
    }
}
int h_stream_sync(reef_stream_t st) {
    if (st && st->window > 0) {
        if (int rc = drain_ring(st)) return rc;
        std::lock_guard<std::mutex> sub(st->submit_mtx);   // a launch the feeder has in hand is enqueued
    }
    HIPCHK(hipStreamSynchronize(st ? st->s : nullptr));
    return 0;
}
int h_stream_query(reef_stream_t st, int* idle) {
    if (st && st->window > 0) {
        std::lock_guard<std::mutex> lock(st->mtx);
        if (!st->has_feeder) {
            if (int rc = pump_locked(st)) return rc;
        }
        if (!st->held.empty()) { *idle = 0; return 0; }
        // everything is on the device: the completion word says whether it is done
        *idle = in_flight(st) == 0 ? 1 : 0;
        if (*idle && st->completion == REEF_COMPLETE_IN_KERNEL) {
            // the last workgroup signals just before the kernel retires: "idle" is only reported
            // once the runtime agrees, so that whoever reads the results next sees them all
            hipError_t e = hipStreamQuery(st->s);
            if (e == hipErrorNotReady) *idle = 0;
            else if (e != hipSuccess) return fail(e, "hipStreamQuery");
        }
        return st->feeder_error.load() ? 1 : 0;
    }
    hipError_t e = hipStreamQuery(st ? st->s : nullptr);
    if (e == hipSuccess) *idle = 1;
    else if (e == hipErrorNotReady) *idle = 0;
    else return fail(e, "hipStreamQuery");
    return 0;
}
int h_device_sync() { HIPCHK(hipDeviceSynchronize()); return 0; }

int h_write_value32(reef_stream_t st, reef_devptr_t p, int32_t v) {
    HIPCHK(hipStreamWriteValue32(st ? st->s : nullptr, p, (uint32_t)v, 0));
    return 0;
}
int h_host_write32(reef_devptr_t p, int32_t v) {
    if (g_host_visible) {
        __atomic_store_n((volatile int32_t*)p, v, __ATOMIC_RELEASE);
        __atomic_thread_fence(__ATOMIC_SEQ_CST);  // push the write-combined store out now
        return 0;
    }
    if (!g_flag_stream) HIPCHK(hipStreamCreateWithFlags(&g_flag_stream, hipStreamNonBlocking));
    HIPCHK(hipStreamWriteValue32(g_flag_stream, p, (uint32_t)v, 0));
    HIPCHK(hipStreamSynchronize(g_flag_stream));
    return 0;
}
int h_host_fill32(reef_devptr_t p, int32_t v, size_t n_words) {
    if (!g_host_visible) return 2;
    volatile int32_t* w = (volatile int32_t*)p;
    for (size_t i = 0; i < n_words; i++) w[i] = v;
    __atomic_thread_fence(__ATOMIC_SEQ_CST);   // push the write-combined stores out now
    return 0;
}
int h_stream_wait_device(reef_stream_t st) {
    if (st && st->window > 0) {
        // What the device has been given by now.  A launch the feeder has taken out of the ring
        // but whose runtime call has not returned yet is not waited for (the runtime blocks a
        // launching thread for milliseconds now and then): it reaches the device later, reads the
        // raised flag and leaves at once.
        const uint32_t target = st->has_feeder ? st->enqueued.load(std::memory_order_acquire)
                                               : st->submitted;
        // bounded spin on the pinned completion word, then let the runtime sleep
        for (long spins = 0; (int32_t)(*st->done - target) < 0; ++spins) {
            if (spins > 20000000L) break;
            __builtin_ia32_pause();
        }
        if ((int32_t)(*st->done - target) >= 0) return 0;
    }
    HIPCHK(hipStreamSynchronize(st ? st->s : nullptr));
    return 0;
}
int h_stream_set_completion(reef_stream_t st, int mode) {
    if (!st || st->window <= 0) return 0;
    if (const char* v = std::getenv("REEF_HAL_COMPLETION"))   // "stream": keep the stream write
        if (std::strcmp(v, "stream") == 0) mode = REEF_COMPLETE_STREAM_WRITE;
    std::lock_guard<std::mutex> lock(st->mtx);
    if (st->submitted != 0) {
        reef_hal_set_error("reef_hal_stream_set_completion: the stream has launches already");
        return 1;
    }
    st->completion = mode;
    return 0;
}
int h_stream_progress(reef_stream_t st, uint32_t* submitted, uint32_t* done) {
    if (!st || st->window <= 0) {
        reef_hal_set_error("reef_hal_stream_progress: needs a stream with a launch window");
        return 1;
    }
    std::lock_guard<std::mutex> lock(st->mtx);
    if (submitted) *submitted = st->submitted;
    if (done) *done = *st->done;
    return 0;
}
int h_stream_drained(reef_stream_t st, int* drained) {
    if (!st || st->window <= 0) return h_stream_query(st, drained);
    std::lock_guard<std::mutex> lock(st->mtx);
    *drained = st->held.empty() && in_flight(st) == 0 ? 1 : 0;
    return st->feeder_error.load() ? 1 : 0;
}
int h_stream_exit_ticks(reef_stream_t st, uint32_t seq, uint64_t* ticks) {
    if (!ticks) return 1;
    *ticks = 0;
    if (!st || st->window <= 0 || st->completion != REEF_COMPLETE_IN_KERNEL || seq == 0) return 0;
    const uint32_t done = *st->done;
    if ((int32_t)(done - seq) < 0 || done - seq >= (uint32_t)kExitRing) return 0;   // not yet, or overwritten
    *ticks = st->exit_ticks[seq % kExitRing];
    return 0;
}
int h_clock_sync(int64_t* host_ns, uint64_t* device_ticks, int64_t* err_ns, int* ticks_per_us) {
    if (!g_flag_stream) HIPCHK(hipStreamCreateWithFlags(&g_flag_stream, hipStreamNonBlocking));
    return reef_hal_hip_clock_probe(g_flag_stream, host_ns, device_ticks, err_ns, ticks_per_us);
}
int h_graph_begin(reef_stream_t st) {
    if (!st || st->window > 0) {
        reef_hal_set_error("reef_hal_graph_begin: needs a stream without a launch window");
        return 1;
    }
    HIPCHK(hipStreamBeginCapture(st->s, hipStreamCaptureModeThreadLocal));
    return 0;
}
int h_graph_end(reef_stream_t st, reef_graph_t* out) {
    if (!st || !out) return 1;
    hipGraph_t g = nullptr;
    HIPCHK(hipStreamEndCapture(st->s, &g));
    hipGraphExec_t ge = nullptr;
    hipError_t e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        hipGraphDestroy(g);
        return fail(e, "hipGraphInstantiate");
    }
    *out = new reef_graph_s{g, ge};
    return 0;
}
int h_graph_launch(reef_graph_t g, reef_stream_t st) {
    if (!g || (st && st->window > 0)) {
        reef_hal_set_error("reef_hal_graph_launch: bad graph or windowed stream");
        return 1;
    }
    HIPCHK(hipGraphLaunch(g->exec, st ? st->s : nullptr));
    return 0;
}
int h_graph_destroy(reef_graph_t g) {
    if (!g) return 0;
    hipGraphExecDestroy(g->exec);
    hipGraphDestroy(g->graph);
    delete g;
    return 0;
}
int h_clear_queue(reef_stream_t st, uint64_t* n) {
    uint64_t d = 0;
    if (st) {
        // a launch the feeder has already taken out of the ring counts as in flight, not as dropped
        std::lock_guard<std::mutex> lock(st->mtx);
        d = st->held.size();
        st->held.clear();
        st->held_count.store(0, std::memory_order_release);
    }
    if (n) *n = d;
    return 0;
}
int h_reset_cus() { return 0; }

// Word-sized fills go out as a small kernel of this library (see fill_words), anything else
// through the runtime.
int fill_async(reef_devptr_t p, int byte, size_t n, hipStream_t s) {
    if (n % 4 == 0 && ((uintptr_t)p) % 4 == 0 && n <= (size_t)1 << 30) return reef_hal_hip_fill(s, p, byte, n);
    HIPCHK(hipMemsetAsync(p, byte, n, s));
    return 0;
}

int h_memset_async(reef_devptr_t p, int byte, size_t n, reef_stream_t st) {
    // a windowed stream may hold launches on the host: the fill must not overtake them
    if (st && st->window > 0) {
        if (int rc = drain_ring(st)) return rc;
        std::lock_guard<std::mutex> sub(st->submit_mtx);   // behind a launch the feeder has in hand
        return fill_async(p, byte, n, st->s);
    }
    return fill_async(p, byte, n, st ? st->s : nullptr);
}

int h_event_create(reef_event_t* out) {
    hipEvent_t e;
    HIPCHK(hipEventCreate(&e));
    *out = (reef_event_t)e;
    return 0;
}
int h_event_destroy(reef_event_t e) { HIPCHK(hipEventDestroy((hipEvent_t)e)); return 0; }
int h_event_record(reef_event_t e, reef_stream_t st) {
    HIPCHK(hipEventRecord((hipEvent_t)e, st ? st->s : nullptr));
    return 0;
}
int h_event_sync(reef_event_t e) { HIPCHK(hipEventSynchronize((hipEvent_t)e)); return 0; }
int h_event_elapsed_us(reef_event_t a, reef_event_t b, float* us) {
    float ms = 0.f;
    HIPCHK(hipEventElapsedTime(&ms, (hipEvent_t)a, (hipEvent_t)b));
    *us = ms * 1000.0f;
    return 0;
}

const reef_hal_backend kHip = {
    h_init, h_device_info, h_module_load, h_module_unload, h_module_get_function,
    h_function_resource, h_malloc, h_free, h_memset, h_h2d, h_d2h, h_h2d_async, h_d2h_async,
    h_stream_create, h_stream_destroy, h_stream_sync, h_stream_query, h_device_sync, h_stream_pump,
    h_launch, h_write_value32, h_clear_queue, h_reset_cus,
    h_event_create, h_event_destroy, h_event_record, h_event_sync, h_event_elapsed_us,
    h_memset_async, h_host_write32, h_stream_wait_device,
    h_graph_begin, h_graph_end, h_graph_launch, h_graph_destroy,
    h_stream_set_completion, h_stream_progress, h_stream_exit_ticks, h_clock_sync,
    h_module_kernel_entry, h_host_fill32, h_stream_drained,
};

}  // namespace

extern "C" const reef_hal_backend* reef_hal_hip_backend(void) { return &kHip; }
