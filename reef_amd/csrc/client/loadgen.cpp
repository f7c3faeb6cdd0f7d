#include "client/loadgen.h"

#include <atomic>
#include <chrono>
#include <cmath>
#include <thread>

namespace reef {
namespace client {

namespace {
// SplitMix64: the generator every seeded quantity of this build uses.
struct SplitMix64 {
    uint64_t s;
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)((next() >> 11) + 1) * (1.0 / 9007199254740993.0); }  // (0,1)
};

int64_t ns_between(server::REEFScheduler::TimePoint a, server::REEFScheduler::TimePoint b) {
    return std::chrono::duration_cast<std::chrono::nanoseconds>(b - a).count();
}
}  // namespace

Status run_load(server::REEFScheduler& sched, const LoadConfig& cfg, LoadResult& out) {
    using Sched = server::REEFScheduler;
    typedef std::chrono::steady_clock Steady;
    const size_t n_be = cfg.be_models.size();
    out = LoadResult();
    out.be_completed.assign(n_be, 0);
    out.be_preempted.assign(n_be, 0);
    out.be_padded.assign(n_be, 0);

    std::atomic<bool> stop{false};
    std::atomic<bool> recording{false};
    std::atomic<int> failures{0};
    std::vector<std::thread> be_threads;
    for (size_t c = 0; c < n_be; c++) {
        be_threads.emplace_back([&, c] {
            while (!stop.load(std::memory_order_acquire)) {
                Sched::TaskID tid;
                if (sched.new_task(cfg.be_models[c], tid) != Status::Succ) { failures++; return; }
                if (sched.wait_task(tid) != Status::Succ) { failures++; return; }
                if (!recording.load(std::memory_order_acquire)) continue;
                std::shared_ptr<Sched::Task> t;
                if (sched.get_task(tid, t) != Status::Succ) { failures++; return; }
                out.be_completed[c]++;
                if (t->is_preempted()) out.be_preempted[c]++;
                if (t->is_padded()) out.be_padded[c]++;
            }
        });
    }

    const int total = cfg.warmup + cfg.requests;
    std::vector<Sched::TaskID> tids((size_t)total);
    Steady::time_point rec_start = Steady::now(), rec_end = rec_start;
    if (total == 0) {
        recording.store(true, std::memory_order_release);
        rec_start = Steady::now();
        std::this_thread::sleep_for(std::chrono::milliseconds(cfg.be_only_ms));
        rec_end = Steady::now();
        recording.store(false, std::memory_order_release);
    } else {
        SplitMix64 rng{cfg.seed};
        Steady::time_point next = Steady::now();
        for (int i = 0; i < total; i++) {
            if (i == cfg.warmup) {
                recording.store(true, std::memory_order_release);
                rec_start = Steady::now();
            }
            if (cfg.mean_interval_us > 0) {
                const double gap_us = -std::log(rng.uniform()) * cfg.mean_interval_us;
                next += std::chrono::nanoseconds((int64_t)(gap_us * 1e3));
                // sleep most of the gap, spin the rest: the submit instant should not carry
                // the wake-up jitter of the sleep
                const auto coarse = next - std::chrono::microseconds(200);
                if (Steady::now() < coarse) std::this_thread::sleep_until(coarse);
                while (Steady::now() < next) {}
                if (sched.new_task(cfg.rt_model, tids[i]) != Status::Succ) { failures++; break; }
            } else {
                if (sched.new_task(cfg.rt_model, tids[i]) != Status::Succ) { failures++; break; }
                if (sched.wait_task(tids[i]) != Status::Succ) { failures++; break; }
            }
        }
        if (failures.load() == 0)
            for (int i = 0; i < total; i++)
                if (sched.wait_task(tids[i]) != Status::Succ) failures++;
        rec_end = Steady::now();
        recording.store(false, std::memory_order_release);
    }
    stop.store(true, std::memory_order_release);
    for (auto& t : be_threads) t.join();
    if (failures.load()) return Status::Fail;

    out.recorded_span_s = std::chrono::duration<double>(rec_end - rec_start).count();
    for (int i = cfg.warmup; i < total; i++) {
        std::shared_ptr<Sched::Task> t;
        RETURN_STATUS(sched.get_task(tids[i], t));
        const auto ts = t->get_timestamp();
        out.rt_latency_ns.push_back(ns_between(ts[0], ts[2]));
        out.rt_queue_ns.push_back(ns_between(ts[0], ts[1]));
        out.rt_exec_ns.push_back(ns_between(ts[1], ts[2]));
    }
    return Status::Succ;
}

}  // namespace client
}  // namespace reef
