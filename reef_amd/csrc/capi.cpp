// Flat C view of the executors (include/reef_c.h).
#include <algorithm>
#include <chrono>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "client/loadgen.h"
#include "executor/hybrid_executor.h"
#include "executor/op_extents.h"
#include "hal/code_object.h"
#include "reef_c.h"
#include "server/scheduler.h"

using namespace reef;
using namespace reef::executor;

struct reef_executor_s {
    int kind;
    std::unique_ptr<ExecutorBase> exe;
    HybridExecutor* hybrid() { return kind == REEF_EXECUTOR_HYBRID ? static_cast<HybridExecutor*>(exe.get()) : nullptr; }
    TransExecutor* trans() { return kind >= REEF_EXECUTOR_TRANS ? static_cast<TransExecutor*>(exe.get()) : nullptr; }
};

namespace {
// Opens up launch_range / launch_preempt_kernel for the timing helpers.
Status launch_all(reef_executor_s* e, int flavour, int begin, int end) {
    if (flavour == REEF_RUN_PREEMPTIBLE) {
        HybridExecutor* h = e->hybrid();
        if (!h) return Status::Fail;
        for (int i = begin; i < end; ++i) RETURN_STATUS(h->launch_preempt_kernel(i, h->stream()));
        return Status::Succ;
    }
    return e->exe->launch_range(begin, end, e->exe->stream());
}
}  // namespace

extern "C" {

int reef_executor_create(int kind, reef_executor_t* out) {
    reef_executor_s* e = new reef_executor_s;
    e->kind = kind;
    if (kind == REEF_EXECUTOR_BASE) e->exe.reset(new ExecutorBase);
    else if (kind == REEF_EXECUTOR_TRANS) e->exe.reset(new TransExecutor);
    else if (kind == REEF_EXECUTOR_HYBRID) e->exe.reset(new HybridExecutor);
    else { delete e; return Status::OutOfRange; }
    *out = e;
    return Status::Succ;
}
void reef_executor_destroy(reef_executor_t e) { delete e; }

int reef_executor_load(reef_executor_t e, const char* json_path, const char* co_path) {
    return e->exe->load_model_from_file(json_path, co_path);
}
int reef_executor_load_hybrid(reef_executor_t e, const char* json_path, const char* profile_path,
                              const char* trans_co_path, const char* be_co_path) {
    HybridExecutor* h = e->hybrid();
    if (!h) return Status::Fail;
    return h->load_hybrid_model_from_file(json_path, profile_path, trans_co_path, be_co_path);
}
int reef_executor_load_param(reef_executor_t e, const char* p) { return e->exe->load_param_from_file(p); }
int reef_executor_set_input(reef_executor_t e, const char* name, const void* data, size_t len) {
    return e->exe->set_input(std::string(name), data, len);
}
int reef_executor_set_input_idx(reef_executor_t e, int idx, const void* data, size_t len) {
    return e->exe->set_input(idx, data, len);
}
int reef_executor_get_data_size(reef_executor_t e, const char* name, size_t* size) {
    return e->exe->get_data_size(name, *size);
}
int reef_executor_get_output(reef_executor_t e, void* out, size_t len) { return e->exe->get_output(out, len); }
int reef_executor_get_data(reef_executor_t e, int idx, void* out, size_t len) {
    return e->exe->get_data(idx, out, len);
}
void reef_executor_set_graph_launch(reef_executor_t e, int on) { e->exe->set_graph_launch(on != 0); }
int reef_executor_execute(reef_executor_t e) { return e->exe->execute(e->exe->stream()); }
int reef_executor_execute_to(reef_executor_t e, int idx) { return e->exe->execute_to(idx, e->exe->stream()); }
int reef_executor_execute_kernel(reef_executor_t e, int idx) {
    return e->exe->execute_kernel(idx, e->exe->stream());
}
int reef_executor_execute_preemptable(reef_executor_t e) {
    HybridExecutor* h = e->hybrid();
    if (!h) return Status::Fail;
    return h->execute_preemptale(h->stream());
}
int reef_executor_num_kernels(reef_executor_t e) { return (int)e->exe->num_kernels(); }

namespace {
struct HybridPeek : public HybridExecutor {
    GPUDevicePtr_t flag() const { return preempt_flag; }
    GPUDevicePtr_t slots() const { return task_slot_base; }
};
}  // namespace

int reef_executor_poke_preempt_flag(reef_executor_t e, int value) {
    HybridExecutor* h = e->hybrid();
    if (!h) return Status::Fail;
    GPUDevicePtr_t flag = static_cast<HybridPeek*>(h)->flag();
    if (reef_hal_memcpy_h2d(flag, &value, 4) != 0) return Status::Fail;
    return Status::Succ;
}
int reef_executor_read_task_slots(reef_executor_t e, int* out, int n) {
    HybridExecutor* h = e->hybrid();
    if (!h || n > (int)h->num_kernels()) return Status::Fail;
    if (reef_hal_memcpy_d2h(out, static_cast<HybridPeek*>(h)->slots(), (size_t)n * 4) != 0) return Status::Fail;
    return Status::Succ;
}
int reef_executor_kernel_info(reef_executor_t e, int idx, int out[7]) {
    TransExecutor* t = e->trans();
    if (!t || idx < 0 || idx >= (int)t->num_kernels()) return Status::OutOfRange;
    const TransExecutor::KernelArg& ka = t->kernel_args()[idx];
    out[0] = ka.block_num;
    out[1] = ka.min_occupancy;
    out[2] = ka.resource.vgprs;
    out[3] = ka.resource.sgprs;
    out[4] = ka.resource.shared_memory;
    out[5] = ka.resource.stack_size;
    out[6] = ka.op;
    return Status::Succ;
}

int reef_executor_time_kernel(reef_executor_t e, int idx, int flavour, int warmup, int iters,
                              float* avg_us) {
    if (idx < 0 || idx >= (int)e->exe->num_kernels() || iters <= 0) return Status::OutOfRange;
    GPUStream_t s = e->exe->stream();
    for (int i = 0; i < warmup; ++i) RETURN_STATUS(launch_all(e, flavour, idx, idx + 1));
    reef_event_t a, b;
    GPU_RETURN_STATUS(reef_hal_event_create(&a));
    GPU_RETURN_STATUS(reef_hal_event_create(&b));
    GPU_RETURN_STATUS(reef_hal_stream_sync(s));
    GPU_RETURN_STATUS(reef_hal_event_record(a, s));
    for (int i = 0; i < iters; ++i) RETURN_STATUS(launch_all(e, flavour, idx, idx + 1));
    GPU_RETURN_STATUS(reef_hal_event_record(b, s));
    GPU_RETURN_STATUS(reef_hal_event_sync(b));
    float us = 0.f;
    GPU_RETURN_STATUS(reef_hal_event_elapsed_us(a, b, &us));
    *avg_us = us / (float)iters;
    reef_hal_event_destroy(a);
    reef_hal_event_destroy(b);
    return Status::Succ;
}

int reef_executor_time_kernel_in_model(reef_executor_t e, int idx, int flavour, int samples,
                                       float* in_model_us, float* after_itself_us) {
    const int n = (int)e->exe->num_kernels();
    if (idx < 0 || idx >= n || samples <= 0 || !in_model_us || !after_itself_us) return Status::OutOfRange;
    GPUStream_t s = e->exe->stream();
    reef_event_t a, b;
    GPU_RETURN_STATUS(reef_hal_event_create(&a));
    GPU_RETURN_STATUS(reef_hal_event_create(&b));
    std::vector<float> in_model, warm;
    for (int i = 0; i < 2 * samples; ++i) {
        const bool model_order = i < samples;
        RETURN_STATUS(model_order ? launch_all(e, flavour, 0, idx) : launch_all(e, flavour, idx, idx + 1));
        GPU_RETURN_STATUS(reef_hal_event_record(a, s));
        RETURN_STATUS(launch_all(e, flavour, idx, idx + 1));
        GPU_RETURN_STATUS(reef_hal_event_record(b, s));
        if (model_order) RETURN_STATUS(launch_all(e, flavour, idx + 1, n));
        GPU_RETURN_STATUS(reef_hal_stream_sync(s));
        float us = 0.f;
        GPU_RETURN_STATUS(reef_hal_event_elapsed_us(a, b, &us));
        (model_order ? in_model : warm).push_back(us);
    }
    std::sort(in_model.begin(), in_model.end());
    std::sort(warm.begin(), warm.end());
    *in_model_us = in_model[in_model.size() / 2];
    *after_itself_us = warm[warm.size() / 2];
    reef_hal_event_destroy(a);
    reef_hal_event_destroy(b);
    return Status::Succ;
}

int reef_executor_time_kernel_dkp(reef_executor_t e, int idx, int layers, int task_num, int warmup,
                                  int iters, float* avg_us) {
    return reef_executor_time_kernel_dkp_confined(e, idx, layers, task_num, 0, warmup, iters, avg_us);
}
int reef_executor_time_kernel_dkp_confined(reef_executor_t e, int idx, int layers, int task_num, int cus,
                                           int warmup, int iters, float* avg_us) {
    TransExecutor* t = e->trans();
    if (!t || idx < 0 || idx >= (int)t->num_kernels() || iters <= 0 || layers <= 0 || cus < 0)
        return Status::OutOfRange;
    GPUStream_t s = t->stream();
    for (int i = 0; i < warmup; ++i) RETURN_STATUS(t->launch_kernel_dkp(idx, layers, task_num, s, cus));
    reef_event_t a, b;
    GPU_RETURN_STATUS(reef_hal_event_create(&a));
    GPU_RETURN_STATUS(reef_hal_event_create(&b));
    GPU_RETURN_STATUS(reef_hal_stream_sync(s));
    GPU_RETURN_STATUS(reef_hal_event_record(a, s));
    for (int i = 0; i < iters; ++i) RETURN_STATUS(t->launch_kernel_dkp(idx, layers, task_num, s, cus));
    GPU_RETURN_STATUS(reef_hal_event_record(b, s));
    GPU_RETURN_STATUS(reef_hal_event_sync(b));
    float us = 0.f;
    GPU_RETURN_STATUS(reef_hal_event_elapsed_us(a, b, &us));
    *avg_us = us / (float)iters;
    reef_hal_event_destroy(a);
    reef_hal_event_destroy(b);
    return Status::Succ;
}

int reef_executor_time_kernel_dkp_single(reef_executor_t e, int idx, int layers, int task_num, int cus,
                                         void* evict, size_t evict_bytes, int samples, float* single_us) {
    TransExecutor* t = e->trans();
    if (!t || idx < 0 || idx >= (int)t->num_kernels() || samples <= 0 || layers <= 0 || cus < 0 ||
        (evict_bytes && !evict))
        return Status::OutOfRange;
    GPUStream_t s = t->stream();
    reef_event_t a, b;
    GPU_RETURN_STATUS(reef_hal_event_create(&a));
    GPU_RETURN_STATUS(reef_hal_event_create(&b));
    std::vector<float> v;
    for (int i = 0; i < samples; ++i) {
        if (evict_bytes) GPU_RETURN_STATUS(reef_hal_memset_async(evict, i & 1, evict_bytes, s));
        else RETURN_STATUS(t->launch_kernel_dkp(idx, layers, task_num, s, cus));
        GPU_RETURN_STATUS(reef_hal_event_record(a, s));
        RETURN_STATUS(t->launch_kernel_dkp(idx, layers, task_num, s, cus));
        GPU_RETURN_STATUS(reef_hal_event_record(b, s));
        GPU_RETURN_STATUS(reef_hal_event_sync(b));
        float us = 0.f;
        GPU_RETURN_STATUS(reef_hal_event_elapsed_us(a, b, &us));
        v.push_back(us);
    }
    std::sort(v.begin(), v.end());
    *single_us = v[v.size() / 2];
    reef_hal_event_destroy(a);
    reef_hal_event_destroy(b);
    return Status::Succ;
}

int reef_executor_time_model(reef_executor_t e, int flavour, int warmup, int iters, float* lat_us,
                             float* dev_us) {
    GPUStream_t s = e->exe->stream();
    const int n = (int)e->exe->num_kernels();
    reef_event_t a, b;
    GPU_RETURN_STATUS(reef_hal_event_create(&a));
    GPU_RETURN_STATUS(reef_hal_event_create(&b));
    for (int it = -warmup; it < iters; ++it) {
        GPU_RETURN_STATUS(reef_hal_stream_sync(s));
        auto t0 = std::chrono::steady_clock::now();
        GPU_RETURN_STATUS(reef_hal_event_record(a, s));
        if (flavour == REEF_RUN_DEFAULT) RETURN_STATUS(e->exe->launch_model(s));
        else RETURN_STATUS(launch_all(e, flavour, 0, n));
        GPU_RETURN_STATUS(reef_hal_event_record(b, s));
        GPU_RETURN_STATUS(reef_hal_stream_sync(s));
        auto t1 = std::chrono::steady_clock::now();
        if (it >= 0) {
            if (lat_us) lat_us[it] = std::chrono::duration<float, std::micro>(t1 - t0).count();
            if (dev_us) GPU_RETURN_STATUS(reef_hal_event_elapsed_us(a, b, &dev_us[it]));
        }
    }
    reef_hal_event_destroy(a);
    reef_hal_event_destroy(b);
    return Status::Succ;
}

}  // extern "C"

struct reef_scheduler_s {
    std::unique_ptr<reef::server::REEFScheduler> s;
};

extern "C" {

using reef::server::REEFScheduler;

int reef_scheduler_create(int mode, reef_scheduler_t* out) {
    if (mode < 0 || mode > 4) return Status::OutOfRange;
    reef_scheduler_s* h = new reef_scheduler_s;
    h->s.reset(new REEFScheduler((REEFScheduler::ScheduleMode)mode));
    *out = h;
    return Status::Succ;
}
void reef_scheduler_destroy(reef_scheduler_t h) { delete h; }
int reef_scheduler_load_model(reef_scheduler_t h, const char* dir, const char* name, int with_param,
                              uint32_t* mid) {
    if (!with_param) return h->s->load_model(std::string(dir), std::string(name), *mid);
    const std::string base = std::string(dir) + "/" + name;
    return h->s->load_model(base + ".trans.co", base + ".be.co", base + ".json",
                            base + ".profile.json", base + ".param", *mid);
}
int reef_scheduler_load_model_files(reef_scheduler_t h, const char* rt_co, const char* be_co,
                                    const char* json, const char* profile, const char* param,
                                    uint32_t* mid) {
    return h->s->load_model(rt_co, be_co, json, profile, param ? param : "", *mid);
}
int reef_scheduler_create_queue(reef_scheduler_t h, int queue_type, uint32_t* qid) {
    return h->s->create_queue(queue_type == REEF_QUEUE_RT ? REEFScheduler::RealTimeQueue
                                                          : REEFScheduler::BestEffortQueue, *qid);
}
int reef_scheduler_bind_model_queue(reef_scheduler_t h, uint32_t qid, uint32_t mid) {
    return h->s->bind_model_queue(qid, mid);
}
int reef_scheduler_get_data_size(reef_scheduler_t h, uint32_t mid, const char* name, size_t* size) {
    return h->s->get_data_size(mid, name, *size);
}
int reef_scheduler_set_input(reef_scheduler_t h, uint32_t mid, const void* data, size_t len,
                             const char* name) {
    return h->s->set_input(mid, data, len, name ? name : "data");
}
int reef_scheduler_get_data(reef_scheduler_t h, uint32_t mid, int idx, void* data, size_t len) {
    return (int)h->s->get_data(mid, idx, data, len);
}
int reef_scheduler_get_output(reef_scheduler_t h, uint32_t mid, void* data, size_t len) {
    return h->s->get_output(mid, data, len);
}
int reef_scheduler_new_task(reef_scheduler_t h, uint32_t mid, uint32_t* tid) {
    return h->s->new_task(mid, *tid);
}
int reef_scheduler_wait_task(reef_scheduler_t h, uint32_t tid) { return h->s->wait_task(tid); }
int reef_scheduler_task_info(reef_scheduler_t h, uint32_t tid, int* flags, int64_t stamps_ns[3],
                             int* state) {
    std::shared_ptr<REEFScheduler::Task> t;
    Status st = h->s->get_task(tid, t);
    if (st != Status::Succ) return st;
    *flags = (t->is_preempted() ? 1 : 0) | (t->is_padded() ? 2 : 0) | (t->is_padded_to_complete() ? 4 : 0);
    auto ts = t->get_timestamp();
    for (int i = 0; i < 3; ++i)
        stamps_ns[i] = std::chrono::duration_cast<std::chrono::nanoseconds>(ts[i].time_since_epoch()).count();
    *state = (int)t->get_state();
    return Status::Succ;
}
int reef_scheduler_run(reef_scheduler_t h) { return h->s->run(); }
int reef_scheduler_shutdown(reef_scheduler_t h) { return h->s->shutdown(); }
int reef_scheduler_mode(reef_scheduler_t h) { return (int)h->s->sche_mode(); }
void reef_scheduler_set_wait_sync(reef_scheduler_t h, int v) { h->s->set_wait_sync(v != 0); }
int reef_scheduler_set_be_stream_cap(reef_scheduler_t h, int v) { return (int)h->s->set_be_stream_cap(v); }
uint64_t reef_scheduler_pending_tasks(reef_scheduler_t h) { return h->s->num_pending_tasks(); }
void reef_scheduler_set_dkp_slack_percent(reef_scheduler_t h, int v) { h->s->set_dkp_slack_percent(v); }
int64_t reef_scheduler_avg_preempt_latency(reef_scheduler_t h) { return h->s->avg_preempt_latency(); }
int64_t reef_scheduler_max_preempt_latency(reef_scheduler_t h) { return h->s->max_preempt_latency(); }
int64_t reef_scheduler_avg_kernel_sel_latency(reef_scheduler_t h) { return h->s->avg_kernel_sel_latency(); }
uint64_t reef_scheduler_preempt_times(reef_scheduler_t h) { return h->s->preempt_times(); }
uint64_t reef_scheduler_padded_kernels(reef_scheduler_t h) { return h->s->padded_kernels(); }
int reef_scheduler_padded_by_op(reef_scheduler_t h, uint64_t* out, int n) {
    uint64_t v[REEF_OP_COUNT];
    h->s->padded_kernels_by_op(v);
    for (int i = 0; i < n; i++) out[i] = i < REEF_OP_COUNT ? v[i] : 0;
    return REEF_OP_COUNT;
}
size_t reef_scheduler_preempt_device_samples(reef_scheduler_t h, int64_t* out_ns, size_t cap) {
    return h->s->preempt_device_samples(out_ns, cap);
}
size_t reef_scheduler_preempt_device_late(reef_scheduler_t h, uint8_t* out, size_t cap) {
    return h->s->preempt_device_late(out, cap);
}
int64_t reef_scheduler_clock_sync_error_ns(reef_scheduler_t h) { return h->s->clock_sync_error_ns(); }
size_t reef_scheduler_preempt_samples(reef_scheduler_t h, int64_t* out, size_t cap) {
    return h->s->preempt_latency_samples(out, cap);
}

void reef_scheduler_preempt_phases(reef_scheduler_t h, int64_t out_ns[3]) { h->s->preempt_phase_avg_ns(out_ns); }

int reef_loadgen_run(reef_scheduler_t h, const reef_load_config* c, int64_t* rt_latency_ns,
                     int64_t* rt_queue_ns, int64_t* rt_exec_ns, uint64_t* be_completed,
                     uint64_t* be_preempted, uint64_t* be_padded, double* recorded_span_s) {
    if (!h || !c || c->warmup < 0 || c->requests < 0) return Status::OutOfRange;
    reef::client::LoadConfig cfg;
    cfg.rt_model = c->rt_model;
    cfg.be_models.assign(c->be_models, c->be_models + c->n_be);
    cfg.mean_interval_us = c->mean_interval_us;
    cfg.seed = c->seed;
    cfg.warmup = c->warmup;
    cfg.requests = c->requests;
    cfg.be_only_ms = c->be_only_ms;
    reef::client::LoadResult r;
    RETURN_STATUS(reef::client::run_load(*h->s, cfg, r));
    for (size_t i = 0; i < r.rt_latency_ns.size(); i++) {
        if (rt_latency_ns) rt_latency_ns[i] = r.rt_latency_ns[i];
        if (rt_queue_ns) rt_queue_ns[i] = r.rt_queue_ns[i];
        if (rt_exec_ns) rt_exec_ns[i] = r.rt_exec_ns[i];
    }
    for (size_t i = 0; i < r.be_completed.size(); i++) {
        if (be_completed) be_completed[i] = r.be_completed[i];
        if (be_preempted) be_preempted[i] = r.be_preempted[i];
        if (be_padded) be_padded[i] = r.be_padded[i];
    }
    if (recorded_span_s) *recorded_span_s = r.recorded_span_s;
    return Status::Succ;
}

int reef_dkp_decide(const int rt[7], const int be[7], const int* be_latency, int n_lat,
                    int be_block_offset, const int proxy[3], int num_cus, int num_xcds, int out[8]) {
    return reef_dkp_decide_slack(rt, be, be_latency, n_lat, be_block_offset, proxy, num_cus, num_xcds,
                                 100, out);
}
int reef_dkp_decide_slack(const int rt[7], const int be[7], const int* be_latency, int n_lat,
                          int be_block_offset, const int proxy[3], int num_cus, int num_xcds,
                          int slack_percent, int out[8]) {
    auto fill = [](TransExecutor::KernelArg& ka, const int v[7]) {
        ka.block_num = v[0];
        ka.min_occupancy = v[1];
        ka.thread_dim = dim3u((uint32_t)v[2], 1, 1);
        ka.task_dim = dim3u((uint32_t)v[0], 1, 1);
        ka.resource = GPUConfig::KernelResource{v[5], v[3], v[4], 0};
        ka.profile.total_latency = v[6];
        ka.profile.total_latency_ns = v[6] * 1000;
        ka.block_offset = 0;
    };
    TransExecutor::KernelArg rta, bea;
    fill(rta, rt);
    fill(bea, be);
    bea.profile.latency.assign(be_latency, be_latency + n_lat);
    for (int j = 0; j < n_lat; j++) bea.profile.latency_ns.push_back(be_latency[j] * 1000);
    GPUConfig::KernelResource pr{proxy[2], proxy[0], proxy[1], 0};
    REEFScheduler::PadDecision d =
        REEFScheduler::decide_padding(rta, bea, be_block_offset, pr, num_cus, num_xcds, slack_percent);
    out[0] = d.merge; out[1] = d.rt_occupancy; out[2] = d.be_occupancy; out[3] = d.final_occupancy;
    out[4] = d.cu_partition; out[5] = d.be_block_num; out[6] = d.merged_block_size;
    out[7] = d.resource.shared_memory;
    return Status::Succ;
}
int reef_dkp_rollback(int launch_offset, int dropped, int window, int kernel_offset) {
    return REEFScheduler::rollback_kernel_offset(launch_offset, dropped, window, kernel_offset);
}

int reef_gpuconfig_num_cus(void) { return (int)GPUConfig::get_num_cus(); }
int reef_gpuconfig_num_xcds(void) { return (int)GPUConfig::get_num_xcds(); }
void reef_gpuconfig_override_geometry(int num_cus, int num_xcds) {
    GPUConfig::override_geometry((uint32_t)num_cus, (uint32_t)num_xcds);
}
int reef_gpuconfig_calculate_occupancy(int shared_memory, int vgprs, int sgprs, int stack_size,
                                       int block_threads) {
    GPUConfig::KernelResource kr{shared_memory, vgprs, sgprs, stack_size};
    return GPUConfig::calculate_occupancy(kr, block_threads);
}
int reef_dkp_logical_layers(int block_num, int num_cus) {
    return TransExecutor::logical_layers(block_num, num_cus);
}
int reef_dkp_cu_partition(int block_num, int num_cus, int num_xcds) {
    return TransExecutor::cu_partition_for(block_num, num_cus, num_xcds);
}
int reef_dkp_occupancy_class(int vgprs) {
    GPUConfig::KernelResource kr{0, vgprs, 0, 0};
    return TransExecutor::occupancy_class(kr);
}

// Same arithmetic as dkp_walk in kernels/reef_entries.hip, on the host.
int reef_dkp_walk(int b, int C, int X, int cu_partition, int layers_l, int task_num_l,
                  int task_offset_l, int layers_r, int task_num_r, int task_offset_r, int* is_right,
                  int* tasks, int cap) {
    const int layer = b / C, cu = b - layer * C;
    const int xcd = cu % X, slot = cu / X;
    const int rt_slots = cu_partition / X;
    int span, cu_idx, layers, task_num, task_offset;
    if (slot < rt_slots) {
        *is_right = 0;
        span = rt_slots * X; cu_idx = slot * X + xcd;
        layers = layers_l; task_num = task_num_l; task_offset = task_offset_l;
    } else {
        *is_right = 1;
        span = C - rt_slots * X; cu_idx = (slot - rt_slots) * X + xcd;
        layers = layers_r; task_num = task_num_r; task_offset = task_offset_r;
    }
    if (layer >= layers) return 0;
    int n = 0;
    const int step = layers * span, end = task_offset + task_num;
    for (int i = span * layer + cu_idx + task_offset; i < end; i += step) {
        if (n < cap) tasks[n] = i;
        ++n;
    }
    return n;
}

int reef_model_parse_summary(const char* json_path, int* n_storage, int* n_kernels, int* n_args,
                             int* n_shared) {
    std::unique_ptr<Model> m(Model::from_json(json_path));
    if (!m) return Status::NotFound;
    *n_storage = (int)m->storage.size();
    *n_kernels = (int)m->kernels.size();
    *n_args = (int)m->args.size();
    *n_shared = (int)m->shared_memory.size();
    return Status::Succ;
}
int reef_model_check_kernels(const char* json_path, char* why, int why_len) {
    std::unique_ptr<Model> m(Model::from_json(json_path));
    if (why && why_len > 0) why[0] = 0;
    if (!m) return Status::NotFound;
    for (size_t i = 0; i < m->kernels.size(); ++i) {
        std::string reason;
        if (!reef::executor::kernel_fits_storages(*m, i, &reason)) {
            if (why && why_len > 0) {
                std::strncpy(why, reason.c_str(), (size_t)why_len - 1);
                why[why_len - 1] = 0;
            }
            return Status::OutOfRange;
        }
    }
    return Status::Succ;
}
int reef_profile_parse_summary(const char* json_path, int* model_latency, int* n_kernels,
                               int* min_latency, int* n_latency_values) {
    std::unique_ptr<ModelProfile> p(ModelProfile::from_json(json_path));
    if (!p) return Status::NotFound;
    *model_latency = p->model_latency;
    *n_kernels = (int)p->kernel_latency.size();
    int mn = 1 << 30, cnt = 0;
    for (auto& kv : p->kernel_latency)
        for (int v : kv.second.latency) { mn = std::min(mn, v); ++cnt; }
    *min_latency = cnt ? mn : 0;
    *n_latency_values = cnt;
    return Status::Succ;
}
int reef_profile_roundtrip(const char* json_path, char* out, size_t cap) {
    std::unique_ptr<ModelProfile> p(ModelProfile::from_json(json_path));
    if (!p) return Status::NotFound;
    std::string s = p->to_json();
    if (s.size() + 1 > cap) return Status::OutOfRange;
    std::memcpy(out, s.c_str(), s.size() + 1);
    return Status::Succ;
}
int reef_param_parse_summary(const char* param_path, const char* key, uint64_t* n_tensors,
                             uint64_t* key_len, float* first, float* last) {
    std::unique_ptr<ModelParam> p(ModelParamParser::parse_from_file(param_path));
    if (!p) return Status::NotFound;
    *n_tensors = p->size();
    auto it = p->find(key);
    if (it == p->end()) return Status::NotFound;
    *key_len = it->second.size();
    *first = it->second.front();
    *last = it->second.back();
    return Status::Succ;
}
int reef_code_object_kernel_meta(const char* co_path, const char* kernel, int out[6]) {
    std::map<std::string, reef::hal::KernelMeta> meta;
    std::string err;
    if (!reef::hal::read_code_object_metadata(co_path, &meta, &err)) return Status::Fail;
    auto it = meta.find(kernel);
    if (it == meta.end()) return Status::NotFound;
    out[0] = it->second.vgprs; out[1] = it->second.agprs; out[2] = it->second.sgprs;
    out[3] = it->second.lds; out[4] = it->second.scratch; out[5] = it->second.kernarg;
    return Status::Succ;
}

}  // extern "C"
