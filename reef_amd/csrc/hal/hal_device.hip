// Device code that belongs to the C-ABI layer itself (not to a model's code objects):
// the clock probe behind reef_hal_clock_sync.  Compiled by hipcc for gfx950 and linked
// into libreef_amd.so.
#include <hip/hip_runtime.h>

#include <chrono>
#include <mutex>
#include <cstdint>

#include "reef_hal.h"

namespace {

// Answers a word the host writes with the device wall clock.  `mailbox` is pinned host
// memory: [0] request (host -> device), [1] reply flag (device -> host), [2..3] clock.
// The wait is bounded: after `spin_limit` polls the kernel leaves with reply flag 2.
__global__ void clock_probe(volatile uint32_t* mailbox, uint32_t round, uint32_t spin_limit) {
    uint32_t seen = 0;
    for (uint32_t i = 0; i < spin_limit; ++i) {
        seen = __hip_atomic_load((uint32_t*)&mailbox[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        if (seen == round) break;
        __builtin_amdgcn_s_sleep(1);
    }
    const uint64_t now = wall_clock64();
    __hip_atomic_store((uint64_t*)&mailbox[2], now, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __hip_atomic_store((uint32_t*)&mailbox[1], seen == round ? round : 0xFFFFFFFFu, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
}

// Fills n 32-bit words.  What reef_hal_memset_async launches instead of a runtime fill: the
// runtime's own fill costs about 20 us on a stream that has kernels ahead of it (it is not an
// ordinary dispatch of that stream), this one what any small kernel costs; it can also be
// recorded into a graph, where a memset node cannot be relied on.
__global__ void fill_words(uint32_t* p, uint32_t value, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

int64_t now_ns() {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(
               std::chrono::steady_clock::now().time_since_epoch()).count();
}

// the mailbox of the clock exchange and its round number: one exchange at a time per process
std::mutex g_probe_mtx;
volatile uint32_t* g_mailbox = nullptr;
uint32_t g_round = 0;

}  // namespace

// byte pattern -> n bytes at p (both multiples of 4), as a kernel on `stream`
int reef_hal_hip_fill(hipStream_t stream, void* p, int byte, size_t n) {
    const uint32_t b = (uint32_t)(byte & 0xFF);
    const uint32_t word = b | (b << 8) | (b << 16) | (b << 24);
    const size_t words = n / 4;
    if (words == 0) return 0;
    hipLaunchKernelGGL(fill_words, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, (uint32_t*)p, word, words);
    if (hipGetLastError() != hipSuccess) {
        reef_hal_set_error("reef_hal_memset_async: fill kernel launch failed");
        return 1;
    }
    return 0;
}

// One correlated (host steady clock, device wall clock) pair: best of `tries` exchanges.
int reef_hal_hip_clock_probe(hipStream_t stream, int64_t* host_ns, uint64_t* device_ticks, int64_t* err_ns,
                             int* ticks_per_us) {
    std::lock_guard<std::mutex> probe_lock(g_probe_mtx);
    if (!g_mailbox) {
        void* p = nullptr;
        if (hipHostMalloc(&p, 64, hipHostMallocDefault) != hipSuccess) {
            reef_hal_set_error("clock probe: hipHostMalloc failed");
            return 1;
        }
        g_mailbox = (volatile uint32_t*)p;
        for (int i = 0; i < 16; ++i) g_mailbox[i] = 0;
    }
    int khz = 0;
    if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, 0) != hipSuccess || khz <= 0) {
        reef_hal_set_error("clock probe: no wall clock rate");
        return 1;
    }
    if (ticks_per_us) *ticks_per_us = khz / 1000;
    int64_t best_window = -1, best_host = 0;
    uint64_t best_ticks = 0;
    for (int t = 0; t < 8; ++t) {
        const uint32_t round = ++g_round ? g_round : ++g_round;
        g_mailbox[1] = 0;
        // about 20 ms of polling at most, then the kernel gives up by itself
        hipLaunchKernelGGL(clock_probe, dim3(1), dim3(1), 0, stream, g_mailbox, round, 2000000u);
        if (hipGetLastError() != hipSuccess) {
            reef_hal_set_error("clock probe: launch failed");
            return 1;
        }
        // let the kernel start polling before the request is written
        for (int i = 0; i < 2000; ++i) __builtin_ia32_pause();
        const int64_t h0 = now_ns();
        __atomic_store_n((volatile uint32_t*)&g_mailbox[0], round, __ATOMIC_RELEASE);
        int64_t h1 = h0;
        uint32_t reply = 0;
        while ((reply = __atomic_load_n((volatile uint32_t*)&g_mailbox[1], __ATOMIC_ACQUIRE)) == 0) {
            h1 = now_ns();
            if (h1 - h0 > 200000000) break;   // 0.2 s: the kernel has long given up
        }
        h1 = now_ns();
        if (hipStreamSynchronize(stream) != hipSuccess) {
            reef_hal_set_error("clock probe: synchronize failed");
            return 1;
        }
        if (reply != round) continue;   // the kernel started after the request or timed out
        const uint64_t ticks = *(volatile uint64_t*)&g_mailbox[2];
        if (best_window < 0 || h1 - h0 < best_window) {
            best_window = h1 - h0;
            best_host = h0 + (h1 - h0) / 2;
            best_ticks = ticks;
        }
    }
    if (best_window < 0) {
        reef_hal_set_error("clock probe: no exchange completed");
        return 1;
    }
    if (host_ns) *host_ns = best_host;
    if (device_ticks) *device_ticks = best_ticks;
    if (err_ns) *err_ns = best_window / 2;
    return 0;
}
