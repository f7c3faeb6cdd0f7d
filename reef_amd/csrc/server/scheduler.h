// REEFScheduler: one real-time queue, up to 32 best-effort queues, one
// scheduler thread.  Real-time tasks run first; their arrival preempts
// best-effort work (reset-based: flag + host-queue drop + rollback) and, in REEF
// mode, each real-time kernel is padded with best-effort workgroups that fit on
// the CUs it leaves free (dynamic kernel padding).
//
// Same public interface and scheduling policy as the reference
// (src/reef/server/scheduler.h:15-190, scheduler.cpp).  What differs on
// MI355X / stock ROCm:
//   * "clear the host queue" and "reset the CUs" go through the C-ABI layer's
//     launch-window streams and the device flag that every best-effort
//     workgroup polls (include/reef_hal.h) -- no patched runtime;
//   * real-time kernels never read the preemption flag, so the flag is not
//     cleared on the real-time stream before a real-time task
//     (scheduler.cpp:458 does that because it launches the best-effort flavour);
//   * the CU geometry is 256 virtual CUs in 8 XCD groups and the partition is
//     rounded to whole slots per XCD (TransExecutor::cu_partition_for);
//   * the scheduler thread sleeps on a condition variable when no task is
//     pending instead of spinning (scheduler.cpp:237-243 spins).
#pragma once
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "executor/hybrid_executor.h"
#include "util/common.h"

namespace reef {
namespace server {

class REEFScheduler {
    struct Model;

public:
    typedef uint32_t ModelID;
    typedef uint32_t QueueID;
    typedef uint32_t TaskID;
    typedef std::chrono::system_clock::time_point TimePoint;

    enum ScheduleMode {
        NoPreempt,    // no preemption
        MultiStream,  // multiple GPU streams
        WaitPreempt,  // wait-based preemption
        REEF,         // reset-based preemption + dynamic kernel padding
        Reset         // reset-based preemption without DKP
    };
    enum TaskQueueType { RealTimeQueue, BestEffortQueue };
    enum TaskState { Init, Waiting, Executing, Finish };

    struct Task {
        friend class REEFScheduler;

    private:
        std::shared_ptr<Model> model;
        QueueID qid;
        TaskID id;
        std::atomic<int> state;
        int launch_offset;  // last kernel handed to the stream
        int kernel_offset;  // first kernel not known to be complete
        int block_offset;   // progress inside kernel_offset under DKP
        std::mutex mtx;
        std::condition_variable cv;
        TimePoint submit, start, end;
        bool preempted;
        bool padding;
        bool padding_to_finish;
        bool sync_dirty;    // an interrupted run may have left split-K arrival counters non-zero
        bool sync_touched;  // padding ran part of a kernel: counters hold live partial counts

    public:
        bool is_preempted() const { return preempted; }
        bool is_padded() const { return padding; }
        bool is_padded_to_complete() const { return padding_to_finish; }
        std::vector<TimePoint> get_timestamp() const { return {submit, start, end}; }
        TaskState get_state() const { return (TaskState)state.load(); }
    };

    // One DKP decision (exposed so the arithmetic can be checked on the host).
    struct PadDecision {
        bool merge = false;
        int rt_occupancy = 0;
        int be_occupancy = 0;
        int final_occupancy = 0;
        int cu_partition = 0;
        int be_block_num = 0;
        int merged_block_size = 0;
        executor::GPUConfig::KernelResource resource{};
    };
    // Pure function of the two kernels' records (scheduler.cpp:533-602).
    static PadDecision decide_padding(const executor::TransExecutor::KernelArg& rt,
                                      const executor::TransExecutor::KernelArg& be,
                                      int be_block_offset,
                                      const executor::GPUConfig::KernelResource& proxy,
                                      int num_cus, int num_xcds, int slack_percent = 100);
    // Rollback after a reset (scheduler.cpp:320-323).
    static int rollback_kernel_offset(int launch_offset, int dropped, int window, int kernel_offset);

public:
    explicit REEFScheduler(ScheduleMode _mode = ScheduleMode::REEF);
    ~REEFScheduler();

    Status load_model(const std::string& model_dir, const std::string& model_name, ModelID& mid);
    Status load_model(const std::string& rt_co_path, const std::string& be_co_path,
                      const std::string& json_path, const std::string& profile_path,
                      const std::string& param_path, ModelID& mid);
    Status create_queue(const TaskQueueType& qtp, QueueID& qid);
    Status bind_model_queue(const QueueID& qid, const ModelID& mid);
    Status get_data_size(ModelID mid, const std::string& name, size_t& size);
    Status set_input(ModelID mid, const void* data, size_t len, const std::string& name = "data");
    Status get_output(ModelID mid, void* data, size_t len, const std::string& name = "output");
    // ExecutorBase::get_data of a loaded model (executor_base.cpp:153-162): any storage by index.
    Status get_data(ModelID mid, int idx, void* data, size_t len);
    Status new_task(const ModelID& mid, TaskID& tid);
    Status wait_task(TaskID tid);
    Status get_task(TaskID tid, std::shared_ptr<Task>& t);
    ScheduleMode sche_mode() const { return mode; }
    void set_wait_sync(bool value) { wait_sync = value; }
    // The window is a property of the best-effort streams, which are created with it; it can
    // only change while no best-effort queue exists (afterwards the rollback after a
    // preemption would assume a window the streams do not have).  Returns Fail then.
    Status set_be_stream_cap(int value) {
        if (be_queue_cnt.load() != 0 || value < 1) return Status::Fail;
        be_stream_device_queue_cap = value;
        return Status::Succ;
    }
    uint64_t num_pending_tasks() const { return pending_tasks.load(); }
    // Share of a real-time kernel's profiled latency that padded best-effort workgroups may
    // take (100 = the reference's rule, be.latency <= rt.latency, scheduler.cpp:565-572).
    // The merged launch ends when its slowest workgroup ends, and on this device kernels run
    // for microseconds, so a best-effort workgroup predicted to take exactly as long as the
    // real-time kernel usually ends after it; a smaller share keeps that out of the
    // real-time latency at the price of fewer padded kernels.  Default 50 (REEF_DKP_SLACK in
    // the environment overrides): measured on MI355X with ResNet-152 real-time, 100 costs the
    // real-time task 7 % (DenseNet-201 best-effort) for 2-4 % best-effort throughput, 50
    // costs it under 1 %.
    void set_dkp_slack_percent(int value) { dkp_slack_percent = value; }
    Status run();
    Status shutdown();
    int64_t avg_preempt_latency() const;     // microseconds
    int64_t avg_kernel_sel_latency() const;  // nanoseconds per real-time kernel
    uint64_t preempt_times() const { return preempt_count; }
    int64_t max_preempt_latency() const { return preempt_latency_max; }
    uint64_t padded_kernels() const { return padded_kernel_count; }
    // Merged launches so far by the op of their best-effort side (index = REEF_OP_*).
    void padded_kernels_by_op(uint64_t out[REEF_OP_COUNT]) const {
        for (int i = 0; i < REEF_OP_COUNT; i++) out[i] = padded_by_op[i];
    }
    // Copies the last `cap` preemption latencies (microseconds); returns how many.
    size_t preempt_latency_samples(int64_t* out, size_t cap) const;
    // The same preemptions timed by the device: nanoseconds from the flag store (host clock)
    // to the moment the last best-effort workgroup that was on the device left it (device wall
    // clock written by that workgroup, mapped to the host clock through reef_hal_clock_sync).
    // A launch that a stream's feeder thread was handing to the runtime while the flag was
    // raised is counted too: its sample is completed when it has left the device.  Only
    // preemptions that found best-effort kernels on the device have a sample.
    size_t preempt_device_samples(int64_t* out_ns, size_t cap) const;
    // 1 where the sample waited for a launch that reached the device after the flag was raised
    size_t preempt_device_late(uint8_t* out, size_t cap) const;
    // Half the length of the host-device clock exchange the mapping rests on (nanoseconds), -1: no mapping.
    int64_t clock_sync_error_ns() const { return clk_valid ? clk_err_ns : -1; }
    // Average nanoseconds per reset-based preemption spent in: raising the flag, dropping the
    // host queues + rollback, waiting for the device to drain (0 unless wait_sync).
    void preempt_phase_avg_ns(int64_t out[3]) const;

private:
    ScheduleMode mode;
    static constexpr size_t model_pool_capacity = 1024;
    static constexpr size_t max_num_be_queues = 32;
    static constexpr QueueID rt_queue_id = 32;

    std::atomic<uint32_t> model_pool_size;
    struct Model {
        executor::HybridExecutor executor;
        QueueID qid;
    };
    std::vector<std::shared_ptr<Model>> model_pool;

    std::atomic<uint32_t> task_idx_pool;
    std::unordered_map<TaskID, std::shared_ptr<Task>> task_pool;
    std::mutex task_pool_mtx;

    struct TaskQueue {
        std::mutex mtx;
        std::deque<std::shared_ptr<Task>> tasks;
        std::atomic<size_t> count{0};
        executor::GPUStream_t stream = nullptr;
        bool empty() const { return count.load(std::memory_order_acquire) == 0; }
        void push(std::shared_ptr<Task> t);
        std::shared_ptr<Task> front();
        void pop();
    };
    std::mutex be_queues_mtx;
    std::vector<std::shared_ptr<TaskQueue>> be_queues;
    std::atomic<uint32_t> be_queue_cnt;
    std::shared_ptr<TaskQueue> rt_queue;

    std::mutex task_cnt_mtx;
    std::condition_variable task_cnt_cv;
    std::atomic<uint64_t> pending_tasks;  // submitted and not yet finished
    bool wait_sync;

    std::unique_ptr<std::thread> scheduler;
    executor::GPUStream_t preempt_stream;
    executor::GPUDevicePtr_t preempt_flag;
    bool preempted;
    int be_stream_device_queue_cap;
    int dkp_slack_percent;
    std::atomic<bool> _shutdown;

    uint64_t preempt_count;
    uint64_t preempt_latency_sum;
    int64_t preempt_latency_max;
    std::vector<int64_t> preempt_samples;
    uint64_t preempt_phase_ns[3];
    // device-side timing of preemptions
    struct LateSample { size_t slot; uint32_t queue; uint32_t seq; int64_t t0_ns; uint64_t ticks; };   // ticks 0: not there yet
    std::vector<int64_t> preempt_device_ns;   // -1: open until the real-time task that caused it is done
    std::vector<uint8_t> preempt_device_late_flag;   // same index: a late launch was part of it
    std::vector<LateSample> late_samples;
    bool clk_valid = false;
    int64_t clk_host_ns = 0, clk_err_ns = 0, clk_synced_at_ns = 0;
    uint64_t clk_dev_ticks = 0;
    int clk_ticks_per_us = 100;
    void sync_clock();
    int64_t device_ticks_to_host_ns(uint64_t ticks) const;
    void resolve_late_samples();
    mutable std::mutex stats_mtx;
    uint64_t kernel_sel_count;
    uint64_t kernel_sel_latency_sum;
    uint64_t padded_kernel_count;
    uint64_t padded_by_op[REEF_OP_COUNT] = {};
    bool gpu_ready;

private:
    Status ensure_gpu();
    Status create_task_queue(std::shared_ptr<TaskQueue>& ret, bool rt);
    void loop_body();
    void execute_be_task(std::shared_ptr<Task>& task, std::shared_ptr<TaskQueue>& tqueue);
    void execute_rt_task(std::shared_ptr<Task>& task);
    void preempt_be_tasks();
    void reset_preempt_flag_async();
    void preempt_reset();
    void preempt_wait();
    void dynamic_kernel_padding(std::shared_ptr<Task>& rt_task);
    void finish_task(const std::shared_ptr<Task>& task, TimePoint end);
};

}  // namespace server
}  // namespace reef
