// In-process load generator: the request patterns of the reference's example
// clients (src/example/rpc_client.cpp, rpc_client_cont.cpp:20-36 -- one thread
// per client, submit / wait in a loop) without the RPC hop, driving a
// REEFScheduler directly.
//   * one real-time client, open loop: arrival times are drawn up front from an
//     exponential distribution (Poisson process) and each request is submitted at
//     its arrival time whether or not the previous one has returned;
//   * N best-effort clients, closed loop: each submits its model again as soon as
//     the previous inference returns, until the real-time client is done.
#pragma once
#include <cstdint>
#include <vector>

#include "server/scheduler.h"

namespace reef {
namespace client {

struct LoadConfig {
    uint32_t rt_model = 0;
    std::vector<uint32_t> be_models;  // one closed-loop client per entry
    double mean_interval_us = 20000;  // real-time inter-arrival mean; <= 0: back-to-back closed loop
    uint64_t seed = 0x5EEF;
    int warmup = 0;    // real-time requests issued before the recorded ones
    int requests = 0;  // recorded real-time requests (0: best-effort only for `be_only_ms`)
    int be_only_ms = 0;
};

struct LoadResult {
    std::vector<int64_t> rt_latency_ns;  // end - submit per recorded request
    std::vector<int64_t> rt_queue_ns;    // start - submit
    std::vector<int64_t> rt_exec_ns;     // end - start
    std::vector<uint64_t> be_completed;  // inferences finished inside the recorded span, per client
    std::vector<uint64_t> be_preempted;  // of those, how many were preempted at least once
    std::vector<uint64_t> be_padded;     // ... ran at least one kernel inside a real-time launch
    double recorded_span_s = 0;
};

Status run_load(server::REEFScheduler& sched, const LoadConfig& cfg, LoadResult& out);

}  // namespace client
}  // namespace reef
