#include "server/scheduler.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace reef {
namespace server {

using executor::GPUConfig;
using executor::HybridExecutor;
using executor::TransExecutor;
typedef std::chrono::system_clock Clock;

// ---------------------------------------------------------------- task queues
void REEFScheduler::TaskQueue::push(std::shared_ptr<Task> t) {
    std::lock_guard<std::mutex> lock(mtx);
    tasks.push_back(std::move(t));
    count.store(tasks.size(), std::memory_order_release);
}
std::shared_ptr<REEFScheduler::Task> REEFScheduler::TaskQueue::front() {
    std::lock_guard<std::mutex> lock(mtx);
    return tasks.empty() ? nullptr : tasks.front();
}
void REEFScheduler::TaskQueue::pop() {
    std::lock_guard<std::mutex> lock(mtx);
    if (!tasks.empty()) tasks.pop_front();
    count.store(tasks.size(), std::memory_order_release);
}

// ---------------------------------------------------------------- life cycle
REEFScheduler::REEFScheduler(ScheduleMode _mode)
    : mode(_mode),
      model_pool_size(0),
      model_pool(model_pool_capacity),
      task_idx_pool(0),
      be_queues(max_num_be_queues),
      be_queue_cnt(0),
      pending_tasks(0),
      wait_sync(false),
      preempt_stream(nullptr),
      preempt_flag(nullptr),
      preempted(false),
      _shutdown(false),
      preempt_count(0),
      preempt_latency_sum(0),
      preempt_latency_max(0),
      kernel_sel_count(0),
      kernel_sel_latency_sum(0),
      padded_kernel_count(0),
      gpu_ready(false) {
    preempt_phase_ns[0] = preempt_phase_ns[1] = preempt_phase_ns[2] = 0;
    // Window of kernels a best-effort stream keeps on the device
    // (scheduler.cpp:29-33: 2, or 1024 when preemption waits for completion).
    be_stream_device_queue_cap = (mode == WaitPreempt) ? 1024 : 2;
    dkp_slack_percent = 50;
    if (const char* e = std::getenv("REEF_DKP_SLACK")) dkp_slack_percent = std::atoi(e);
}

REEFScheduler::~REEFScheduler() {
    if (scheduler) shutdown();
    // give the hardware queues back: a later scheduler in the same process would otherwise
    // share them with streams nobody uses
    for (auto& q : be_queues)
        if (q && q->stream) reef_hal_stream_destroy(q->stream);
    if (rt_queue && rt_queue->stream) reef_hal_stream_destroy(rt_queue->stream);
    if (preempt_stream) reef_hal_stream_destroy(preempt_stream);
    model_pool.clear();
    if (preempt_flag) reef_hal_free(preempt_flag, REEF_MEM_DEVICE_FINEGRAINED);
}

// Streams and the shared preemption flag (scheduler.cpp:24-28).
Status REEFScheduler::ensure_gpu() {
    if (gpu_ready) return Status::Succ;
    GPU_RETURN_STATUS(reef_hal_init(0));
    // only wait-based preemption orders anything on a stream of its own
    if (mode == WaitPreempt) GPU_RETURN_STATUS(reef_hal_stream_create(0, &preempt_stream));
    GPU_RETURN_STATUS(reef_hal_malloc(4, REEF_MEM_DEVICE_FINEGRAINED, &preempt_flag));
    GPU_RETURN_STATUS(reef_hal_memset(preempt_flag, 0, 4));
    sync_clock();
    gpu_ready = true;
    return Status::Succ;
}

Status REEFScheduler::create_task_queue(std::shared_ptr<TaskQueue>& ret, bool rt) {
    RETURN_STATUS(ensure_gpu());
    executor::GPUStream_t stream;
    if (rt) {
        REEF_LOG_INFO("create rt stream");
        GPU_RETURN_STATUS(reef_hal_stream_create(0, &stream));
    } else {
        REEF_LOG_INFO("create be stream");
        GPU_RETURN_STATUS(reef_hal_stream_create(be_stream_device_queue_cap, &stream));
        // best-effort kernels tell the stream themselves when they are done (ReefBeArgs)
        GPU_RETURN_STATUS(reef_hal_stream_set_completion(stream, REEF_COMPLETE_IN_KERNEL));
    }
    ret = std::make_shared<TaskQueue>();
    ret->stream = stream;
    return Status::Succ;
}

Status REEFScheduler::load_model(const std::string& model_dir, const std::string& model_name,
                                 ModelID& mid) {
    const std::string base = model_dir + "/" + model_name;
    return load_model(base + ".trans.co", base + ".be.co", base + ".json", base + ".profile.json",
                      "", mid);
}

Status REEFScheduler::load_model(const std::string& rt_co_path, const std::string& be_co_path,
                                 const std::string& json_path, const std::string& profile_path,
                                 const std::string& param_path, ModelID& mid) {
    RETURN_STATUS(ensure_gpu());
    std::shared_ptr<Model> model(new Model);
    RETURN_STATUS(model->executor.load_hybrid_model_from_file(
        json_path.c_str(), profile_path.c_str(), rt_co_path.c_str(), be_co_path.c_str()));
    model->qid = rt_queue_id;  // real-time queue by default
    if (!param_path.empty()) RETURN_STATUS(model->executor.load_param_from_file(param_path.c_str()));
    const uint32_t idx = model_pool_size.fetch_add(1);
    if (idx >= model_pool_capacity) {
        REEF_LOG_ERROR("model pool is full");
        model_pool_size.fetch_sub(1);
        return Status::Fail;
    }
    RETURN_STATUS(model->executor.set_preempt_flag(preempt_flag));
    model_pool[idx] = std::move(model);
    REEF_LOG_INFO("load model from %s, idx %u", json_path.c_str(), idx);
    mid = idx;
    return Status::Succ;
}

Status REEFScheduler::create_queue(const TaskQueueType& qtp, QueueID& qid) {
    if (qtp == TaskQueueType::RealTimeQueue) {
        qid = rt_queue_id;
        std::lock_guard<std::mutex> lock(be_queues_mtx);
        if (!rt_queue) RETURN_STATUS(create_task_queue(rt_queue, true));
        return Status::Succ;
    }
    std::shared_ptr<TaskQueue> q;
    RETURN_STATUS(create_task_queue(q, false));
    std::lock_guard<std::mutex> lock(be_queues_mtx);
    const uint32_t idx = be_queue_cnt.load();
    if (idx >= max_num_be_queues) RETURN_STATUS(Status::Full);
    be_queues[idx] = std::move(q);
    be_queue_cnt.store(idx + 1);
    qid = idx;
    return Status::Succ;
}

Status REEFScheduler::bind_model_queue(const QueueID& qid, const ModelID& mid) {
    if (model_pool_size.load() <= mid) RETURN_STATUS(Status::OutOfRange);
    if (be_queue_cnt.load() <= qid && qid != rt_queue_id) RETURN_STATUS(Status::OutOfRange);
    model_pool[mid]->qid = qid;
    return Status::Succ;
}

Status REEFScheduler::new_task(const ModelID& mid, TaskID& tid) {
    if (model_pool_size.load() <= mid) RETURN_STATUS(Status::OutOfRange);
    auto& model = model_pool[mid];
    if (model->qid == rt_queue_id && !rt_queue) RETURN_STATUS(Status::NotFound);
    std::shared_ptr<Task> task(new Task);
    task->model = model;
    task->id = task_idx_pool.fetch_add(1);
    task->qid = model->qid;
    task->block_offset = 0;
    task->kernel_offset = 0;
    task->launch_offset = 0;
    task->state.store(TaskState::Init);
    task->submit = Clock::now();
    task->preempted = false;
    task->padding = false;
    task->padding_to_finish = false;
    task->sync_dirty = false;
    task->sync_touched = false;
    tid = task->id;
    {
        std::lock_guard<std::mutex> lock(task_pool_mtx);
        task_pool.insert({tid, task});
    }
    if (model->qid == rt_queue_id) rt_queue->push(task);
    else be_queues[model->qid]->push(task);
    {
        std::lock_guard<std::mutex> lock(task_cnt_mtx);
        pending_tasks.fetch_add(1);
    }
    task_cnt_cv.notify_all();
    return Status::Succ;
}

Status REEFScheduler::get_task(TaskID tid, std::shared_ptr<Task>& t) {
    std::lock_guard<std::mutex> lock(task_pool_mtx);
    auto it = task_pool.find(tid);
    if (it == task_pool.end()) return Status::NotFound;
    t = it->second;
    return Status::Succ;
}

Status REEFScheduler::wait_task(TaskID tid) {
    std::shared_ptr<Task> task;
    RETURN_STATUS(get_task(tid, task));
    std::unique_lock<std::mutex> lock(task->mtx);
    task->cv.wait(lock, [&] { return task->state.load() == TaskState::Finish; });
    return Status::Succ;
}

Status REEFScheduler::get_data_size(ModelID mid, const std::string& name, size_t& size) {
    if (mid >= model_pool_size.load()) RETURN_STATUS(Status::OutOfRange);
    return model_pool[mid]->executor.get_data_size(name, size);
}
Status REEFScheduler::set_input(ModelID mid, const void* data, size_t len, const std::string& name) {
    if (mid >= model_pool_size.load()) RETURN_STATUS(Status::OutOfRange);
    return model_pool[mid]->executor.set_input(name, data, len);
}
// The name is accepted and ignored, as in the reference (scheduler.cpp:226-230).
Status REEFScheduler::get_output(ModelID mid, void* data, size_t len, const std::string&) {
    if (mid >= model_pool_size.load()) RETURN_STATUS(Status::OutOfRange);
    return model_pool[mid]->executor.get_output(data, len);
}

Status REEFScheduler::get_data(ModelID mid, int idx, void* data, size_t len) {
    if (mid >= model_pool_size.load()) RETURN_STATUS(Status::OutOfRange);
    return model_pool[mid]->executor.get_data(idx, data, len);
}

Status REEFScheduler::run() {
    if (scheduler) RETURN_STATUS(Status::Fail);
    {
        std::lock_guard<std::mutex> lock(be_queues_mtx);
        if (!rt_queue) RETURN_STATUS(create_task_queue(rt_queue, true));
    }
    _shutdown.store(false);
    scheduler.reset(new std::thread([this] {
        reef_hal_init(0);  // bind the device to this thread
        while (!_shutdown.load()) {
            if (pending_tasks.load() == 0) {
                std::unique_lock<std::mutex> lock(task_cnt_mtx);
                task_cnt_cv.wait_for(lock, std::chrono::milliseconds(2), [this] {
                    return pending_tasks.load() != 0 || _shutdown.load();
                });
                continue;
            }
            loop_body();
        }
    }));
    return Status::Succ;
}

Status REEFScheduler::shutdown() {
    if (!scheduler) return Status::Succ;
    _shutdown.store(true);
    task_cnt_cv.notify_all();
    scheduler->join();
    scheduler.reset();
    return Status::Succ;
}

// Finishing is idempotent: a task is reported (and counted out of pending_tasks) once,
// whichever path notices its completion first.
void REEFScheduler::finish_task(const std::shared_ptr<Task>& task, TimePoint end) {
    {
        std::lock_guard<std::mutex> lock(task->mtx);
        if (task->state.load() == TaskState::Finish) return;
        task->end = end;
        task->state.store(TaskState::Finish);
    }
    task->cv.notify_all();
    pending_tasks.fetch_sub(1);
}

// ---------------------------------------------------------------- scheduling loop
// Real-time tasks to exhaustion, then one pass over the best-effort queues,
// going back to real-time mode as soon as a real-time task shows up
// (scheduler.cpp:262-303).
void REEFScheduler::loop_body() {
    for (;;) {
        while (!rt_queue->empty()) {
            preempt_be_tasks();
            auto rt_task = rt_queue->front();
            rt_queue->pop();
            execute_rt_task(rt_task);
        }
        bool rt_arrived = false;
        const uint32_t n = be_queue_cnt.load();
        for (uint32_t i = 0; i < n && !rt_arrived; i++) {
            auto& q = be_queues[i];
            while (!q->empty()) {
                if (!rt_queue->empty()) { rt_arrived = true; break; }
                auto be_task = q->front();
                execute_be_task(be_task, q);
                // A finished task leaves its queue before anything else can look at the
                // queue head: a real-time arrival in this instant must not find it there
                // (the padding pass would run its kernels a second time).
                if (be_task->state.load() == TaskState::Finish) {
                    q->pop();
                    continue;
                }
                if (!rt_queue->empty()) { rt_arrived = true; break; }
                break;
            }
        }
        if (!rt_arrived) return;
    }
}

int REEFScheduler::rollback_kernel_offset(int launch_offset, int dropped, int window, int kernel_offset) {
    return std::max(launch_offset - dropped - window, kernel_offset);
}

// Reset-based preemption (scheduler.cpp:305-346): raise the flag, drop what the
// best-effort streams still hold on the host, roll every running task back to a
// kernel that is certainly complete, and (optionally) wait until the kernels
// that were already on the device have left.  The flag is stored from this
// thread straight into device memory: a stream write would queue behind whatever
// best-effort kernel shares the hardware queue with the preemption stream.
void REEFScheduler::preempt_reset() {
    typedef std::chrono::steady_clock Steady;
    const auto t0 = Steady::now();
    reef_hal_host_write32(preempt_flag, 1);
    const auto t1 = Steady::now();
    const uint32_t n = be_queue_cnt.load();
    // launches each stream has handed to the device by now (a launch its feeder thread is
    // passing to the runtime this instant included) and how many of them are still there
    uint32_t target[max_num_be_queues], busy[max_num_be_queues];
    for (uint32_t i = 0; i < n; i++) {
        uint64_t dropped = 0;
        reef_hal_stream_clear_queue(be_queues[i]->stream, &dropped);
        uint32_t sub = 0, done = 0;
        target[i] = busy[i] = 0;
        if (clk_valid && reef_hal_stream_progress(be_queues[i]->stream, &sub, &done) == 0) {
            target[i] = sub;
            busy[i] = sub - done;
        }
        auto task = be_queues[i]->front();
        if (task && task->state.load() == TaskState::Executing) {
            task->kernel_offset = rollback_kernel_offset(task->launch_offset, (int)dropped,
                                                         be_stream_device_queue_cap,
                                                         task->kernel_offset);
            task->block_offset = 0;
            task->state.store(TaskState::Waiting);
            task->preempted = true;
            task->sync_dirty = true;
        }
    }
    for (int i = 0; i < be_stream_device_queue_cap + 1; i++) reef_hal_reset_cus();
    const auto t2 = Steady::now();
    if (wait_sync) {
        for (uint32_t i = 0; i < n; i++) reef_hal_stream_wait_device(be_queues[i]->stream);
    }
    const auto t3 = Steady::now();
    auto ns = [](Steady::time_point a, Steady::time_point b) {
        return (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(b - a).count();
    };
    // the device's own account: when did the last workgroup of each stream's newest launch leave.
    // Only the raw device clock is kept here; it is mapped to the host clock once the real-time
    // task is done (resolve_late_samples), with a clock exchange that is at most one task old --
    // the two clocks drift by tens of microseconds per second.
    if (clk_valid && wait_sync) {
        const int64_t t0_ns = std::chrono::duration_cast<std::chrono::nanoseconds>(t1.time_since_epoch()).count();
        bool any = false, late = false;
        std::lock_guard<std::mutex> lock(stats_mtx);
        const size_t slot = preempt_device_ns.size();
        for (uint32_t i = 0; i < n; i++) {
            if (busy[i] == 0) continue;
            any = true;
            uint64_t ticks = 0;
            reef_hal_stream_exit_ticks(be_queues[i]->stream, target[i], &ticks);
            // ticks == 0: still inside the runtime call or on the device, read later
            late_samples.push_back(LateSample{slot, i, target[i], t0_ns, ticks});
            late = late || ticks == 0;
        }
        if (any) {
            preempt_device_ns.push_back(-1);   // open until the task is done
            preempt_device_late_flag.push_back(late ? 1 : 0);
        }
    }
    std::lock_guard<std::mutex> lock(stats_mtx);
    preempt_phase_ns[0] += ns(t0, t1);
    preempt_phase_ns[1] += ns(t1, t2);
    preempt_phase_ns[2] += ns(t2, t3);
}

// Host clock <-> device wall clock, one exchange (see reef_hal_clock_sync).
void REEFScheduler::sync_clock() {
    int64_t h = 0, err = 0;
    uint64_t d = 0;
    int tpu = 0;
    if (reef_hal_clock_sync(&h, &d, &err, &tpu) != 0 || tpu <= 0) return;   // a backend without a device clock
    std::lock_guard<std::mutex> lock(stats_mtx);
    clk_host_ns = h;
    clk_dev_ticks = d;
    clk_err_ns = err;
    clk_ticks_per_us = tpu;
    clk_synced_at_ns = h;
    clk_valid = true;
}

int64_t REEFScheduler::device_ticks_to_host_ns(uint64_t ticks) const {
    const int64_t dt = (int64_t)(ticks - clk_dev_ticks);
    return clk_host_ns + dt * 1000 / clk_ticks_per_us;
}

// Closes the samples of the preemptions since the last call: exit clocks that were not there yet
// (a launch that reached the device after the flag was raised has long left by the time a
// real-time task is done) are read now, and every exit clock is mapped to the host clock.
void REEFScheduler::resolve_late_samples() {
    std::lock_guard<std::mutex> lock(stats_mtx);
    for (const LateSample& l : late_samples) {
        if (l.slot >= preempt_device_ns.size()) continue;
        uint64_t ticks = l.ticks;
        if (ticks == 0 && l.queue < be_queue_cnt.load())
            reef_hal_stream_exit_ticks(be_queues[l.queue]->stream, l.seq, &ticks);
        if (ticks == 0) continue;   // overwritten in the meantime: the other streams' exits stand
        const int64_t v = std::max<int64_t>(device_ticks_to_host_ns(ticks) - l.t0_ns, 0);
        preempt_device_ns[l.slot] = std::max(preempt_device_ns[l.slot], v);
    }
    for (const LateSample& l : late_samples)
        if (l.slot < preempt_device_ns.size() && preempt_device_ns[l.slot] < 0) preempt_device_ns[l.slot] = 0;
    late_samples.clear();
}

size_t REEFScheduler::preempt_device_late(uint8_t* out, size_t cap) const {
    std::lock_guard<std::mutex> lock(stats_mtx);
    size_t k = 0;
    for (size_t i = 0; i < preempt_device_ns.size() && k < cap; i++)
        if (preempt_device_ns[i] >= 0) out[k++] = preempt_device_late_flag[i];
    return k;
}

size_t REEFScheduler::preempt_device_samples(int64_t* out_ns, size_t cap) const {
    std::lock_guard<std::mutex> lock(stats_mtx);
    size_t k = 0;
    for (size_t i = 0; i < preempt_device_ns.size() && k < cap; i++)
        if (preempt_device_ns[i] >= 0) out_ns[k++] = preempt_device_ns[i];
    return k;
}

void REEFScheduler::preempt_phase_avg_ns(int64_t out[3]) const {
    std::lock_guard<std::mutex> lock(stats_mtx);
    for (int i = 0; i < 3; i++) out[i] = preempt_count ? (int64_t)(preempt_phase_ns[i] / preempt_count) : 0;
}

// Wait-based preemption (scheduler.cpp:348-372): raise the flag, let the device
// drain, then find per running task the first kernel whose workgroups did not all
// finish (HybridExecutor::get_be_kernel_offset, hybrid_executor.cpp:141-151).
// The completion counters of the kernels a run is about to launch are zeroed on the
// task's own stream when the run (re)starts (execute_be_task), so a count read here
// belongs to this run only; a task that has not been launched yet is left alone.
void REEFScheduler::preempt_wait() {
    reef_hal_host_write32(preempt_flag, 1);
    const uint32_t n = be_queue_cnt.load();
    for (uint32_t i = 0; i < n; i++) {
        uint64_t dropped = 0;
        reef_hal_stream_clear_queue(be_queues[i]->stream, &dropped);
    }
    for (uint32_t i = 0; i < n; i++) reef_hal_stream_sync(be_queues[i]->stream);
    for (uint32_t i = 0; i < n; i++) {
        auto be_task = be_queues[i]->front();
        if (!be_task || be_task->state.load() != TaskState::Executing) continue;
        auto& exe = be_task->model->executor;
        exe.copy_be_kernel_offset(preempt_stream);
        reef_hal_stream_sync(preempt_stream);
        const int off = exe.get_be_kernel_offset(be_task->kernel_offset);
        be_task->kernel_offset = std::max(be_task->kernel_offset, off);
        be_task->block_offset = 0;
        be_task->preempted = true;
        be_task->sync_dirty = true;
    }
}

void REEFScheduler::preempt_be_tasks() {
    if (preempted) return;
    preempted = true;
    REEF_LOG_INFO("preempt");
    const auto t0 = std::chrono::steady_clock::now();
    switch (mode) {
        case ScheduleMode::NoPreempt: {
            const uint32_t n = be_queue_cnt.load();
            for (uint32_t i = 0; i < n; i++) reef_hal_stream_sync(be_queues[i]->stream);
            for (uint32_t i = 0; i < n; i++) {
                auto be_task = be_queues[i]->front();
                if (be_task && be_task->state.load() == TaskState::Executing)
                    be_task->kernel_offset = be_task->launch_offset + 1;
            }
            break;
        }
        case ScheduleMode::Reset:
        case ScheduleMode::REEF: preempt_reset(); break;
        case ScheduleMode::WaitPreempt: preempt_wait(); break;
        default: break;
    }
    const auto t1 = std::chrono::steady_clock::now();
    const int64_t us = std::chrono::duration_cast<std::chrono::nanoseconds>(t1 - t0).count() / 1000;
    {
        std::lock_guard<std::mutex> lock(stats_mtx);
        preempt_count++;
        preempt_latency_sum += (uint64_t)us;
        preempt_latency_max = std::max(preempt_latency_max, us);
        preempt_samples.push_back(us);
    }
    REEF_LOG_INFO("preempt latency: %lld us", (long long)us);

    const uint32_t n = be_queue_cnt.load();
    for (uint32_t i = 0; i < n; i++) {
        auto be_task = be_queues[i]->front();
        if (be_task && be_task->state.load() == TaskState::Executing)
            be_task->state.store(TaskState::Waiting);
    }
}

int64_t REEFScheduler::avg_preempt_latency() const {
    std::lock_guard<std::mutex> lock(stats_mtx);
    return preempt_count ? (int64_t)(preempt_latency_sum / preempt_count) : 0;
}
int64_t REEFScheduler::avg_kernel_sel_latency() const {
    return kernel_sel_count ? (int64_t)(kernel_sel_latency_sum / kernel_sel_count) : 0;
}
size_t REEFScheduler::preempt_latency_samples(int64_t* out, size_t cap) const {
    std::lock_guard<std::mutex> lock(stats_mtx);
    const size_t n = std::min(cap, preempt_samples.size());
    std::copy(preempt_samples.end() - n, preempt_samples.end(), out);
    return n;
}

void REEFScheduler::reset_preempt_flag_async() {
    reef_hal_host_write32(preempt_flag, 0);
}

void REEFScheduler::execute_rt_task(std::shared_ptr<Task>& task) {
    REEF_LOG_INFO("start rt task");
    task->state.store(TaskState::Executing);
    task->start = Clock::now();
    bool be_waiting = false;
    if (mode == ScheduleMode::REEF) {
        const uint32_t n_q = be_queue_cnt.load();
        for (uint32_t q = 0; q < n_q && !be_waiting; q++) be_waiting = !be_queues[q]->empty();
    }
    if (be_waiting) {
        // something to pad with: one launch per kernel, each with its own decision
        dynamic_kernel_padding(task);
        reef_hal_stream_sync(rt_queue->stream);
    } else {
        task->model->executor.execute(rt_queue->stream);
    }
    finish_task(task, Clock::now());
    REEF_LOG_INFO("rt task finish");
    // Off the real-time path, and only when this task preempted something whose device-side
    // sample is still open: complete the samples, with a clock mapping that is renewed first
    // when it is older than 100 ms (the two clocks drift by tens of microseconds per second).
    // The exchange keeps this thread for some tens of microseconds, so a task that has no
    // sample to convert does not pay for it.
    if (clk_valid && !late_samples.empty()) {
        const int64_t now = std::chrono::duration_cast<std::chrono::nanoseconds>(
                                std::chrono::steady_clock::now().time_since_epoch()).count();
        if (now - clk_synced_at_ns > 100000000) sync_clock();
        resolve_late_samples();
    }
}

// ---------------------------------------------------------------- dynamic kernel padding
// Can `be` ride along with `rt`, and with how many workgroups?  (scheduler.cpp:533-602)
//   fits      : occupancy(max resource, max block) >= rt.min_occupancy
//   be_occ    : the largest j+1 <= merged occupancy with be.latency[j] <= rt.total_latency * slack
//   partition : CUs the rt kernel really needs, in whole slots per XCD
//   be_blocks : (CUs left) * (rt_latency * slack / be_latency[be_occ-1]) * be_occ, clamped to what is left
REEFScheduler::PadDecision REEFScheduler::decide_padding(const TransExecutor::KernelArg& rt,
                                                         const TransExecutor::KernelArg& be,
                                                         int be_block_offset,
                                                         const GPUConfig::KernelResource& proxy,
                                                         int num_cus, int num_xcds, int slack_percent) {
    PadDecision d;
    d.rt_occupancy = rt.min_occupancy;
    d.final_occupancy = rt.min_occupancy;
    d.cu_partition = num_cus;
    d.merged_block_size = std::max((int)rt.thread_dim.count(), (int)be.thread_dim.count());
    d.resource = GPUConfig::max_resource(GPUConfig::max_resource(rt.resource, be.resource), proxy);
    // the proxy's LDS is dynamic: it needs the larger of the two sides' static LDS
    d.resource.shared_memory = std::max(rt.resource.shared_memory, be.resource.shared_memory);
    const int merged_occupancy = GPUConfig::calculate_occupancy(d.resource, d.merged_block_size);
    if (merged_occupancy < rt.min_occupancy) return d;

    // latencies in nanoseconds (from the profile's *_ns keys, else microseconds x 1000)
    int be_occupancy = 0;
    const int64_t rt_latency = rt.profile.total_latency_ns;
    const int64_t be_budget = rt_latency * slack_percent / 100;
    const std::vector<int>& be_lat = be.profile.latency_ns;
    for (int j = merged_occupancy - 1; j >= 0; j--) {
        if ((int)be_lat.size() <= j) continue;
        if (be_lat[j] <= be_budget) {
            be_occupancy = j + 1;
            break;
        }
    }
    if (be_occupancy == 0) return d;
    const int64_t be_latency = std::max(be_lat[be_occupancy - 1], 1);

    const int partition = TransExecutor::cu_partition_for(rt.block_num, num_cus, num_xcds);
    const int64_t be_iters = be_budget / be_latency;
    int64_t be_blocks64 = (int64_t)(num_cus - partition) * be_iters * be_occupancy;
    int be_blocks = (int)std::min<int64_t>(be_blocks64, be.block_num - be_block_offset);
    if (be_blocks <= 0) return d;

    d.merge = true;
    d.be_occupancy = be_occupancy;
    d.final_occupancy = std::max(rt.min_occupancy, be_occupancy);
    d.cu_partition = partition;
    d.be_block_num = be_blocks;
    return d;
}

void REEFScheduler::dynamic_kernel_padding(std::shared_ptr<Task>& rt_task) {
    HybridExecutor& rt_exe = rt_task->model->executor;
    const int num_cus = (int)GPUConfig::get_num_cus();
    const int num_xcds = (int)GPUConfig::get_num_xcds();
    std::vector<std::shared_ptr<Task>> complete_be_tasks;
    TimePoint current_time_point = Clock::now();
    const std::vector<TransExecutor::Proxy>& proxies = rt_exe.proxies();

    const int n_rt = (int)rt_exe.num_kernels();
    for (int i = 0; i < n_rt; i++) {
        const auto sel_start = std::chrono::steady_clock::now();
        const TransExecutor::KernelArg& rt_args = rt_exe.trans_args[i];
        PadDecision dec;
        std::shared_ptr<Task> be_task;
        const TransExecutor::KernelArg* be_args = nullptr;
        int proxy_idx = -1;
        const uint32_t n_q = be_queue_cnt.load();
        for (uint32_t q = 0; q < n_q; q++) {   // first queue whose head kernel fits (scheduler.cpp:533-602)
            auto cand = be_queues[q]->front();
            if (!cand || cand->state.load() == TaskState::Finish) continue;
            HybridExecutor& be_exe = cand->model->executor;
            if (cand->kernel_offset >= (int)be_exe.num_kernels()) continue;
            const TransExecutor::KernelArg& ka = be_exe.trans_args[cand->kernel_offset];
            // Cheapest test first: a kernel that is too long at every occupancy cannot be padded
            // (decide_padding would find the same).  This loop runs between two real-time
            // launches, so what it costs per candidate is real-time latency.
            {
                const std::vector<int>& lat = ka.profile.latency_ns;
                const int64_t budget = (int64_t)rt_args.profile.total_latency_ns * dkp_slack_percent / 100;
                if (lat.empty() || *std::min_element(lat.begin(), lat.end()) > budget) continue;
            }
            // the proxy whose two register ranges hold both kernels sets the register budget of
            // the launch (scheduler.cpp:613-642 / trans_executor.cpp:175-199)
            const int px = TransExecutor::select_proxy(proxies, rt_args.resource, ka.resource);
            if (px < 0) continue;
            PadDecision d = decide_padding(rt_args, ka, cand->block_offset, proxies[px].resource, num_cus,
                                           num_xcds, dkp_slack_percent);
            if (!d.merge) continue;
            if (cand->sync_dirty) {
                // An interrupted run left arrival counters behind: pad this task only once its own
                // stream has drained, and clear the counters first -- from the host (a fill on
                // the real-time stream would sit in front of the real-time kernels), and only now
                // that a kernel of the task is really about to be padded.
                if (be_exe.has_sync_storage()) {
                    // (from the stream's counters: a query of the runtime here would put a
                    // marker in front of the real-time kernels)
                    int drained = 0;
                    if (reef_hal_stream_drained(be_queues[q]->stream, &drained) != 0 || !drained) continue;
                    be_exe.reset_sync_storage_from_host(rt_queue->stream);
                }
                cand->sync_dirty = false;
            }
            dec = d;
            proxy_idx = px;
            be_task = cand;
            be_args = &ka;
            break;
        }
        const auto sel_end = std::chrono::steady_clock::now();
        kernel_sel_count++;
        kernel_sel_latency_sum +=
            (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(sel_end - sel_start).count();

        if (!be_task) {
            // nothing fits: the real-time kernel alone, single-sided
            rt_exe.launch_kernel(i, rt_queue->stream);
        } else {
            HybridExecutor& be_exe = be_task->model->executor;
            ReefDkpArgs a;
            std::memset(&a, 0, sizeof(a));
            rt_exe.fill_side(a.l, i, dec.rt_occupancy, rt_args.block_num, rt_args.block_offset);
            be_exe.fill_side(a.r, be_task->kernel_offset, dec.be_occupancy, dec.be_block_num,
                             be_task->block_offset);
            a.cu_partition = dec.cu_partition;
            a.num_cus = num_cus;
            a.num_xcds = num_xcds;
            a.task_slot_r = nullptr;
            a.entry_l = (const void*)(uintptr_t)rt_args.entry;
            a.entry_r = (const void*)(uintptr_t)be_args->entry;
            if (be_task->start.time_since_epoch().count() == 0) be_task->start = current_time_point;
            executor::GPUFunction_t proxy = rt_exe.get_proxy_kernel(proxy_idx);
            const uint32_t grid[3] = {(uint32_t)(dec.final_occupancy * num_cus), 1, 1};
            const uint32_t block[3] = {(uint32_t)dec.merged_block_size, 1, 1};
            reef_hal_launch(proxy, grid, block, (uint32_t)dec.resource.shared_memory, rt_queue->stream,
                            &a, sizeof(a));
            padded_kernel_count++;
            if (be_args->op >= 0 && be_args->op < REEF_OP_COUNT) padded_by_op[be_args->op]++;
        }
        current_time_point += std::chrono::microseconds(rt_args.profile.total_latency);

        // progress of the padded best-effort task (scheduler.cpp:655-672)
        if (be_task) {
            be_task->padding = true;
            // a later restart in best-effort mode re-runs this kernel from its first block
            be_task->sync_touched = true;
            be_task->block_offset += dec.be_block_num;
            if (be_task->block_offset >= be_args->block_num) {
                be_task->block_offset = 0;
                be_task->kernel_offset++;
                if (be_task->kernel_offset >= (int)be_task->model->executor.num_kernels()) {
                    be_task->kernel_offset = 0;
                    be_task->padding_to_finish = true;
                    be_task->end = current_time_point;
                    complete_be_tasks.push_back(be_task);
                    be_queues[be_task->qid]->pop();
                }
            }
        }
    }
    // Tasks that finished inside real-time shadows are reported once the
    // real-time stream has drained (their last workgroups run on it).
    if (!complete_be_tasks.empty()) {
        reef_hal_stream_sync(rt_queue->stream);
        for (auto& t : complete_be_tasks) finish_task(t, t->end);
    }
}

// ---------------------------------------------------------------- best-effort execution
// Incremental launch with a real-time check between launches, completion by
// polling the stream (scheduler.cpp:685-740).
void REEFScheduler::execute_be_task(std::shared_ptr<Task>& task, std::shared_ptr<TaskQueue>& tqueue) {
    switch ((TaskState)task->state.load()) {
        case TaskState::Finish: return;
        case TaskState::Executing: {
            if (executor::GPUStreamEmpty(tqueue->stream)) {
                task->kernel_offset = 0;
                task->block_offset = 0;
                finish_task(task, Clock::now());
            }
            return;
        }
        case TaskState::Init:
        case TaskState::Waiting: {
            auto& exe = task->model->executor;
            const int num_kernels = (int)exe.num_kernels();
            if (task->state.load() == TaskState::Init && task->start.time_since_epoch().count() == 0)
                task->start = Clock::now();
            if (preempted) {
                reset_preempt_flag_async();
                preempted = false;
            }
            if (task->kernel_offset >= num_kernels) {
                task->kernel_offset = 0;
                task->block_offset = 0;
                finish_task(task, Clock::now());
                return;
            }
            task->state.store(TaskState::Executing);
            task->block_offset = 0;
            // Arrival counters of split-K kernels may be left over from an interrupted
            // or partly padded run; the fill is ordered behind anything still draining
            // on this stream.
            if (task->sync_dirty || task->sync_touched) {
                exe.reset_sync_storage(tqueue->stream);
                task->sync_dirty = task->sync_touched = false;
            }
            // wait-based preemption reads the completion counters of this run: the kernels
            // about to be launched start from zero (a model keeps the counts of earlier runs)
            if (mode == ScheduleMode::WaitPreempt) exe.reset_task_slots_from(task->kernel_offset, tqueue->stream);
            for (int i = task->kernel_offset; i < num_kernels; i++) {
                exe.launch_preempt_kernel(i, tqueue->stream);
                task->launch_offset = i;
                if (!rt_queue->empty() && (mode == ScheduleMode::REEF || mode == ScheduleMode::Reset))
                    return;  // preempt during launch
            }
            return;
        }
    }
}

}  // namespace server
}  // namespace reef
