/*
 * reef_c.h -- flat C view of the executor and scheduler classes, for callers
 * that cannot include C++ headers (the Python tests and benchmark bind it with
 * ctypes).  Each function forwards to the C++ method of the same name, which in
 * turn mirrors the reference class it replaces:
 *   ExecutorBase     src/reef/executor/executor_base.h:17-69
 *   TransExecutor    src/reef/executor/trans_executor.h:41-87
 *   HybridExecutor   src/reef/executor/hybrid_executor.h:18-76
 *   REEFScheduler    src/reef/server/scheduler.h:15-190
 * Return value: reef::Status as an int (0 Succ, 1 Fail, 2 NotFound,
 * 3 OutOfRange, 4 Full), as in src/reef/util/common.h:46-52.
 */
#ifndef REEF_C_H
#define REEF_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct reef_executor_s* reef_executor_t;

enum { REEF_EXECUTOR_BASE = 0, REEF_EXECUTOR_TRANS = 1, REEF_EXECUTOR_HYBRID = 2 };
/* Which flavour a timing helper launches. */
enum { REEF_RUN_DEFAULT = 0, REEF_RUN_PREEMPTIBLE = 1 };

int reef_executor_create(int kind, reef_executor_t* out);
void reef_executor_destroy(reef_executor_t e);
/* ExecutorBase::load_model_from_file (executor_base.cpp:15-27); for a TransExecutor `co` is the trans.co. */
int reef_executor_load(reef_executor_t e, const char* json_path, const char* co_path);
/* HybridExecutor::load_hybrid_model_from_file (hybrid_executor.cpp:14-31) */
int reef_executor_load_hybrid(reef_executor_t e, const char* json_path, const char* profile_path,
                              const char* trans_co_path, const char* be_co_path);
int reef_executor_load_param(reef_executor_t e, const char* param_path);
int reef_executor_set_input(reef_executor_t e, const char* name, const void* data, size_t len);
int reef_executor_set_input_idx(reef_executor_t e, int idx, const void* data, size_t len);
int reef_executor_get_data_size(reef_executor_t e, const char* name, size_t* size);
int reef_executor_get_output(reef_executor_t e, void* out, size_t len);
int reef_executor_get_data(reef_executor_t e, int idx, void* out, size_t len);
/* on: whole-model runs replay a recorded launch sequence (one submission); off (default,
 * unless REEF_GRAPH=1 is in the environment): one launch call per kernel, as
 * executor_base.cpp:191-221 does. */
void reef_executor_set_graph_launch(reef_executor_t e, int on);
int reef_executor_execute(reef_executor_t e);
int reef_executor_execute_to(reef_executor_t e, int idx);
int reef_executor_execute_kernel(reef_executor_t e, int idx);
int reef_executor_execute_preemptable(reef_executor_t e);
int reef_executor_num_kernels(reef_executor_t e);
/* Sets the executor's own 4-byte preemption flag (hybrid only) to `value`. */
int reef_executor_poke_preempt_flag(reef_executor_t e, int value);
/* Reads the per-kernel completion counters (hybrid only) into out[0..n). */
int reef_executor_read_task_slots(reef_executor_t e, int* out, int n);
/* Per-kernel resource record: out = {block_num, min_occupancy, vgprs, sgprs, lds, scratch, op}. */
int reef_executor_kernel_info(reef_executor_t e, int idx, int out[7]);

/*
 * Measurement helpers (device events on the stream the kernels run on).
 * time_kernel: `warmup` untimed launches of kernel idx, then `iters` timed
 *   launches bracketed by two events; *avg_us = elapsed / iters.
 * time_model:  `warmup` whole-model runs, then `iters` runs, each bracketed by
 *   events and by host clocks; lat_us[i] = host-observed latency of run i
 *   (launch of the first kernel to completion of the last), dev_us[i] = device
 *   time between the events.  Either output may be NULL.
 */
int reef_executor_time_kernel(reef_executor_t e, int idx, int flavour, int warmup, int iters,
                              float* avg_us);
/* One launch of kernel idx between two events, `samples` times, medians: in the model's own order
 * (kernels 0..idx-1 before it, the rest after it: operands as cold or warm as a real pass finds
 * them) and directly after a launch of itself (operands cached).  Both carry the same event
 * overhead; in_model - after_itself is what the model's order adds to a back-to-back figure. */
int reef_executor_time_kernel_in_model(reef_executor_t e, int idx, int flavour, int samples,
                                       float* in_model_us, float* after_itself_us);
/* time_kernel_dkp: kernel idx through the DKP flavour with `layers` workgroup layers per CU
 * and the first `task_num` tasks only -- the measurement behind <model>.profile.json
 * (latency[j] = one round of (j+1) x num_cus workgroups; the reference's profiler tool
 * is not in its repository, resource/Makefile:32-36). */
/* The same with the kernel confined to `cus` virtual CUs (0: all), as the best-effort side of a
 * padded launch is: `layers` workgroups then really share each of those CUs.  What a profile's
 * latency[layers - 1] has to describe (scheduler.cpp:565-572,589-590). */
int reef_executor_time_kernel_dkp_confined(reef_executor_t e, int idx, int layers, int task_num, int cus,
                                           int warmup, int iters, float* avg_us);
int reef_executor_time_kernel_dkp(reef_executor_t e, int idx, int layers, int task_num, int warmup,
                                  int iters, float* avg_us);
/* One launch between two events, `samples` times, median in *single_us.  With evict_bytes > 0 the
 * `evict` buffer (device memory of the caller, larger than the device's last-level cache) is
 * overwritten before every sample, so the kernel finds its operands in HBM -- the state a
 * best-effort kernel is in when several models take turns on the device; with evict_bytes == 0 the
 * kernel itself runs once before every sample (operands cached).  The two medians carry the same
 * event overhead, so their difference is what a cold start adds to a back-to-back figure. */
int reef_executor_time_kernel_dkp_single(reef_executor_t e, int idx, int layers, int task_num, int cus,
                                         void* evict, size_t evict_bytes, int samples, float* single_us);
int reef_executor_time_model(reef_executor_t e, int flavour, int warmup, int iters, float* lat_us,
                             float* dev_us);

/* ---- REEFScheduler (src/reef/server/scheduler.h:68-126) ---- */
typedef struct reef_scheduler_s* reef_scheduler_t;
enum { REEF_MODE_NOPREEMPT = 0, REEF_MODE_MULTISTREAM = 1, REEF_MODE_WAITPREEMPT = 2,
       REEF_MODE_REEF = 3, REEF_MODE_RESET = 4 };
enum { REEF_QUEUE_RT = 0, REEF_QUEUE_BE = 1 };
int reef_scheduler_create(int mode, reef_scheduler_t* out);
void reef_scheduler_destroy(reef_scheduler_t s);
/* load_model(dir, name) (scheduler.cpp:57-68); `with_param` != 0 also loads <dir>/<name>.param */
int reef_scheduler_load_model(reef_scheduler_t s, const char* dir, const char* name, int with_param,
                              uint32_t* mid);
int reef_scheduler_load_model_files(reef_scheduler_t s, const char* rt_co, const char* be_co,
                                    const char* json, const char* profile, const char* param,
                                    uint32_t* mid);
int reef_scheduler_create_queue(reef_scheduler_t s, int queue_type, uint32_t* qid);
int reef_scheduler_bind_model_queue(reef_scheduler_t s, uint32_t qid, uint32_t mid);
int reef_scheduler_get_data_size(reef_scheduler_t s, uint32_t mid, const char* name, size_t* size);
int reef_scheduler_set_input(reef_scheduler_t s, uint32_t mid, const void* data, size_t len,
                             const char* name);
int reef_scheduler_get_output(reef_scheduler_t s, uint32_t mid, void* data, size_t len);
/* ExecutorBase::get_data (executor_base.cpp:153-162) of a model the scheduler holds. */
int reef_scheduler_get_data(reef_scheduler_t s, uint32_t mid, int idx, void* data, size_t len);
int reef_scheduler_new_task(reef_scheduler_t s, uint32_t mid, uint32_t* tid);
int reef_scheduler_wait_task(reef_scheduler_t s, uint32_t tid);
/* Task record: flags bit0 preempted, bit1 padded, bit2 padded to completion;
 * stamps = submit, start, end in nanoseconds since the epoch; state = TaskState. */
int reef_scheduler_task_info(reef_scheduler_t s, uint32_t tid, int* flags, int64_t stamps_ns[3],
                             int* state);
int reef_scheduler_run(reef_scheduler_t s);
int reef_scheduler_shutdown(reef_scheduler_t s);
int reef_scheduler_mode(reef_scheduler_t s);
void reef_scheduler_set_wait_sync(reef_scheduler_t s, int value);
/* Launch window of best-effort streams (set_be_stream_cap, scheduler.h:120).  Only while no
 * best-effort queue exists: Fail afterwards (the streams were created with the old window). */
int reef_scheduler_set_be_stream_cap(reef_scheduler_t s, int value);
/* Tasks submitted and not yet finished. */
uint64_t reef_scheduler_pending_tasks(reef_scheduler_t s);
/* Share (percent) of a real-time kernel's profiled latency that padded best-effort workgroups
 * may take; 100 is the reference's rule (scheduler.cpp:565-572). */
void reef_scheduler_set_dkp_slack_percent(reef_scheduler_t s, int value);
int64_t reef_scheduler_avg_preempt_latency(reef_scheduler_t s);
int64_t reef_scheduler_max_preempt_latency(reef_scheduler_t s);
int64_t reef_scheduler_avg_kernel_sel_latency(reef_scheduler_t s);
uint64_t reef_scheduler_preempt_times(reef_scheduler_t s);
uint64_t reef_scheduler_padded_kernels(reef_scheduler_t s);
/* Merged launches by the op of their best-effort side: out[i] for REEF_OP_* = i (reef_kernels.h),
 * i < n.  Returns the number of op ids. */
int reef_scheduler_padded_by_op(reef_scheduler_t s, uint64_t* out, int n);
size_t reef_scheduler_preempt_samples(reef_scheduler_t s, int64_t* out, size_t cap);
/* The same preemptions timed by the device (nanoseconds): flag store -> the last best-effort
 * workgroup that was on the device has left, from the device wall clock that workgroup wrote,
 * mapped to the host clock by a clock exchange whose half-length clock_sync_error_ns returns
 * (-1: this backend has no device clock).  Only with wait_sync on. */
size_t reef_scheduler_preempt_device_samples(reef_scheduler_t s, int64_t* out_ns, size_t cap);
/* For the same samples, in the same order: 1 where a best-effort stream was handing a launch to the
 * runtime when the flag was stored.  That launch reaches the device later (the runtime call may
 * block), finds the flag and leaves; the sample runs until its exit. */
size_t reef_scheduler_preempt_device_late(reef_scheduler_t s, uint8_t* out, size_t cap);
int64_t reef_scheduler_clock_sync_error_ns(reef_scheduler_t s);
/* Average ns per reset-based preemption in: flag store, host-queue drop + rollback, device drain. */
void reef_scheduler_preempt_phases(reef_scheduler_t s, int64_t out_ns[3]);
/* ---- load generator: the request loops of the reference's example clients
 * (src/example/rpc_client.cpp, rpc_client_cont.cpp:20-36) run in-process against a scheduler.
 * One open-loop real-time client (exponential inter-arrival times, mean `mean_interval_us`;
 * <= 0 means closed loop, back to back) and `n_be` closed-loop best-effort clients.  With
 * requests + warmup == 0 only the best-effort clients run, for `be_only_ms`.
 * Output arrays: rt_* hold `requests` entries, be_* hold `n_be`; any may be NULL. ---- */
typedef struct {
    uint32_t rt_model;
    uint32_t n_be;
    const uint32_t* be_models;
    double mean_interval_us;
    uint64_t seed;
    int32_t warmup;
    int32_t requests;
    int32_t be_only_ms;
} reef_load_config;
int reef_loadgen_run(reef_scheduler_t s, const reef_load_config* cfg, int64_t* rt_latency_ns,
                     int64_t* rt_queue_ns, int64_t* rt_exec_ns, uint64_t* be_completed,
                     uint64_t* be_preempted, uint64_t* be_padded, double* recorded_span_s);

/* DKP decision for one (real-time kernel, best-effort kernel) pair (scheduler.cpp:533-602).
 * rt / be = {block_num, min_occupancy, threads, vgprs, sgprs, lds, total_latency};
 * be_latency[n_lat] = best-effort kernel latency per occupancy; proxy = {vgprs, sgprs, lds}.
 * out = {merge, rt_occupancy, be_occupancy, final_occupancy, cu_partition, be_block_num,
 *        merged_block_size, lds}. */
int reef_dkp_decide(const int rt[7], const int be[7], const int* be_latency, int n_lat,
                    int be_block_offset, const int proxy[3], int num_cus, int num_xcds, int out[8]);
/* The same with the share (percent) of rt's latency that best-effort work may take; 100 above. */
int reef_dkp_decide_slack(const int rt[7], const int be[7], const int* be_latency, int n_lat,
                          int be_block_offset, const int proxy[3], int num_cus, int num_xcds,
                          int slack_percent, int out[8]);
int reef_dkp_rollback(int launch_offset, int dropped, int window, int kernel_offset);

/* ---- one fused convolution on plain device pointers ----
 * The call one generated kernel of the reference's fused_nn_conv2d_* family serves
 * (resource/resnet152/resnet152.cu:376,715: in, W, out, bias; :35: in, W, out, residual), for
 * callers that hold tensors of their own instead of a model directory:
 *   out[o][y][x] = act(sum_{c,ky,kx} in[c][y*s+ky-p][x*s+kx-p] * w[o][c][ky][kx] + residual[o][y][x] + bias[o])
 * NCHW / OIHW fp32, batch 1; bias and residual may be NULL.  All pointers are device memory.
 * `stream` is a hipStream_t (NULL: the default stream).  The kernels and the split of K are
 * chosen by the library; a split is folded inside the launch through partial tiles and arrival
 * counters (fixed summation order), which need memory beyond the operands. */
typedef struct {
    int32_t cin, h, w, cout, kh, kw, stride_h, stride_w, pad_h, pad_w;
    int32_t act;   /* REEF_ACT_NONE / REEF_ACT_RELU / REEF_ACT_RELU6 of reef_kernels.h */
} reef_conv2d_desc;
/* Loads the gfx950 kernels (a reef_kernels.raw.co) for the current device. */
int reef_ops_init(const char* kernels_co_path);
/* Takes the partial-tile workspace and the counters from hipMalloc for the duration of the call
 * and returns them before it returns (it waits for the stream then). */
int reef_ops_conv2d(const reef_conv2d_desc* c, const float* in, const float* w, const float* bias,
                    const float* residual, float* out, void* stream);
/* The same convolution for callers that cannot allocate (code under stream capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The partial tiles and arrival counters of a split K live in a fixed array in device memory
 * that belongs to this library (4 MiB of partial tiles + 16384 counters per GPU, held until the
 * process ends); the call allocates and frees nothing, enqueues a small fill kernel that zeroes
 * the counters it needs and then the convolution, and returns without waiting.  A layer whose
 * split needs more than the array holds is refused with Status::Fail and a message saying so
 * (reef_ops_scratch_bytes() = bytes of partial tiles the array holds; the library's own choice
 * of split stays within it for every shape it accepts).  reef_ops_init must have
 * run with the device current.  Every call on a GPU uses that GPU's one array: calls that
 * overlap on one GPU (two streams, two threads) race on it -- serialise them.  Bit-identical
 * to reef_ops_conv2d. */
int reef_ops_conv2d_noalloc(const reef_conv2d_desc* c, const float* in, const float* w, const float* bias,
                            const float* residual, float* out, void* stream);
size_t reef_ops_scratch_bytes(void);

/* GPUConfig (src/reef/executor/hip/hip_impl.cpp:9-74) */
int reef_gpuconfig_num_cus(void);
int reef_gpuconfig_num_xcds(void);
void reef_gpuconfig_override_geometry(int num_cus, int num_xcds);
int reef_gpuconfig_calculate_occupancy(int shared_memory, int vgprs, int sgprs, int stack_size,
                                       int block_threads);
/* DKP arithmetic shared by TransExecutor and the scheduler. */
int reef_dkp_logical_layers(int block_num, int num_cus);
int reef_dkp_cu_partition(int block_num, int num_cus, int num_xcds);
int reef_dkp_occupancy_class(int vgprs);
/* Host replica of the device-side side/task walk (one physical workgroup):
 * returns the number of tasks written to tasks[0..cap), *is_right = side. */
int reef_dkp_walk(int block_idx, int num_cus, int num_xcds, int cu_partition, int layers_l,
                  int task_num_l, int task_offset_l, int layers_r, int task_num_r,
                  int task_offset_r, int* is_right, int* tasks, int cap);

/* Parsers (src/reef/executor/model.cpp), exposed for format tests. */
int reef_model_parse_summary(const char* json_path, int* n_storage, int* n_kernels, int* n_args,
                             int* n_shared);
/* The check every executor makes when it loads a graph file, before anything is launched: each
 * kernel's shape attributes must fit the storages it is given (operand count, bytes behind each
 * operand's start) and the number of workgroups it is launched with.  0 = every kernel fits;
 * otherwise `why` (when given) names the first kernel that does not, the operand and the sizes.
 * No counterpart in the reference: its generated kernels have their shapes compiled in
 * (resource/resnet152/resnet152.cu:315-338), the shape-generic kernels here trust their attributes. */
int reef_model_check_kernels(const char* json_path, char* why, int why_len);
int reef_profile_parse_summary(const char* json_path, int* model_latency, int* n_kernels,
                               int* min_latency, int* n_latency_values);
int reef_profile_roundtrip(const char* json_path, char* out, size_t cap);
int reef_param_parse_summary(const char* param_path, const char* key, uint64_t* n_tensors,
                             uint64_t* key_len, float* first, float* last);
int reef_code_object_kernel_meta(const char* co_path, const char* kernel, int out[6]);

#ifdef __cplusplus
}
#endif
#endif /* REEF_C_H */
