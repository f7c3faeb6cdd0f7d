/*
 * reef_hal.h -- the thin C-ABI layer between REEF's executors / scheduler and
 * the GPU runtime on MI355X.  One function per use the reference makes of its
 * `GPU*` macro table (src/reef/executor/hip/hip_impl.h:5-23), of GPUConfig
 * (src/reef/executor/hip/hip_impl.cpp:9-80) and of the five direct hip* calls
 * in the executors and the scheduler; the citation on each entry names the
 * call it replaces.
 *
 * Conventions: every function returns 0 on success and non-zero on failure;
 * reef_hal_last_error() returns a thread-local message for the last failure
 * on the calling thread.  Handles are opaque and owned by the layer.  No
 * callbacks, no exceptions, no C++ or torch types cross this boundary.
 * Functions may be called from any thread; launches onto one stream must come
 * from one thread at a time (the scheduler thread, as in
 * src/reef/server/scheduler.cpp:237-243).
 *
 * Stock ROCm has no hipStreamCreateWithWindowSize / hipStreamClearQueue /
 * hipResetWavefronts (the reference gets them from a patched runtime and
 * driver).  This layer provides the same contract without patches:
 *   - a stream created with launch_window = w keeps at most w kernels on the
 *     device; further launches wait in a host-side queue of the stream and
 *     move to the device as earlier kernels complete.  In the HIP backend a
 *     feeder thread per windowed stream does that (REEF_HAL_FEEDER=0 in the
 *     environment: the caller's thread does it inside reef_hal_launch /
 *     reef_hal_stream_query / reef_hal_stream_pump instead);
 *   - reef_hal_stream_clear_queue drops the host-side queue and reports how
 *     many launches it dropped, which is what the scheduler's rollback formula
 *     consumes (src/reef/server/scheduler.cpp:313-329);
 *   - reef_hal_reset_cus raises nothing on the device: best-effort kernels
 *     leave on their own when they read the preemption flag, which they poll
 *     at workgroup start and inside their main loops.
 */
#ifndef REEF_HAL_H
#define REEF_HAL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct reef_module_s* reef_module_t;
typedef struct reef_function_s* reef_function_t;
typedef struct reef_stream_s* reef_stream_t;
typedef struct reef_event_s* reef_event_t;
typedef struct reef_graph_s* reef_graph_t;
typedef void* reef_devptr_t;

/* Static properties of the device the occupancy model needs.
 * Replaces GPUConfig::get_num_cus (hard-coded 60, hip_impl.cpp:9-12). */
typedef struct reef_device_info {
    int num_cus;            /* 256 on MI355X */
    int num_xcds;           /* 8 */
    int simds_per_cu;       /* 4 */
    int max_waves_per_simd; /* 8 */
    int vgprs_per_simd;     /* 512 per lane (unified VGPR + AGPR file) */
    int vgpr_granule;       /* 8 */
    int lds_bytes_per_cu;   /* 163840 */
    int lds_granule;        /* 1280 */
    int max_wg_per_cu;      /* 32 */
    int max_threads_per_cu; /* 2048 */
    int clock_khz;
    char arch[32];          /* "gfx950" */
} reef_device_info;

/* Registers / memory one kernel needs (hipFuncGetWGInfo in hip_impl.cpp:34-42). */
typedef struct reef_kernel_resource {
    int shared_memory; /* static LDS bytes */
    int vgprs;         /* arch VGPRs + AGPRs */
    int sgprs;
    int stack_size;    /* scratch bytes per lane */
    int agprs;         /* the accumulation registers among `vgprs` (they sit behind the arch VGPRs) */
} reef_kernel_resource;

/* Completion record of a launch on a windowed stream in REEF_COMPLETE_IN_KERNEL mode: the first
 * 32 bytes of the kernel's argument block.  The caller leaves it zero; the layer fills it when
 * the launch goes to the device.  The kernel's workgroups count themselves out on *exit_count
 * as they leave; the last one sets the counter back to zero, stores the device wall clock to
 * *exit_ticks and then `seq` to *done_word (both host-visible).  A kernel that finds done_word
 * NULL (launched on a stream without that mode) does none of this. */
typedef struct reef_hal_completion {
    uint32_t* done_word;
    uint64_t* exit_ticks;
    uint32_t* exit_count;
    uint32_t seq;
    uint32_t reserved;
} reef_hal_completion;
enum { REEF_COMPLETE_STREAM_WRITE = 0, REEF_COMPLETE_IN_KERNEL = 1 };

enum { REEF_MEM_DEVICE = 0, REEF_MEM_DEVICE_FINEGRAINED = 1, REEF_MEM_HOST_PINNED = 2 };

const char* reef_hal_last_error(void);

/* hipInit + hipDeviceGet            executor_base.cpp:19-22
 * The HIP backend also opens the runtime's pool of hardware queues with idle streams that live as
 * long as the process, so streams created later are spread over different hardware queues instead
 * of sharing one by accident of creation order (REEF_HAL_HOLD_QUEUES=0: off). */
int reef_hal_init(int device);
/* GPUConfig::get_num_cus            hip_impl.cpp:9-12 */
int reef_hal_device_info(reef_device_info* out);

/* hipModuleLoad                     executor_base.cpp:25, hybrid_executor.cpp:22-23 */
int reef_hal_module_load(const char* path, reef_module_t* out);
int reef_hal_module_unload(reef_module_t mod);
/* hipModuleGetFunction              executor_base.cpp:48-50 */
int reef_hal_module_get_function(reef_module_t mod, const char* name, reef_function_t* out);
/* hipFuncGetWGInfo                  hip_impl.cpp:34-42 (read from the code object's metadata) */
int reef_hal_function_resource(reef_function_t fn, reef_kernel_resource* out);
/* Device address of a kernel's first instruction: GPUConfig::get_kernel_address, hip_impl.cpp:16-32
 * (there read out of the kernel descriptor through the patched runtime's hipFuncGetWGInfo; here
 * from the device variable <name>_entry the code object publishes beside each kernel of the
 * padding flavour).  What a merge_framework_<n> proxy jumps to. */
int reef_hal_module_kernel_entry(reef_module_t mod, const char* name, uint64_t* address);
/* GPUConfig::calculate_occupancy    hip_impl.cpp:55-74 -> workgroups resident per CU */
int reef_hal_occupancy(const reef_kernel_resource* res, int block_threads, int dyn_lds,
                       int* blocks_per_cu);

/* hipMalloc / hipHostMalloc / hipFree   executor_base.cpp:61, hybrid_executor.cpp:72,99 */
int reef_hal_malloc(size_t bytes, int kind, reef_devptr_t* out);
int reef_hal_free(reef_devptr_t ptr, int kind);
/* hipMemset / hipMemcpyHtoD / hipMemcpyDtoH   executor_base.cpp:62,90,116,158 */
int reef_hal_memset(reef_devptr_t ptr, int byte, size_t bytes);
int reef_hal_memcpy_h2d(reef_devptr_t dst, const void* src, size_t bytes);
int reef_hal_memcpy_d2h(void* dst, reef_devptr_t src, size_t bytes);
/* hipMemcpyHtoDAsync / hipMemcpyDtoHAsync     hybrid_executor.cpp:134,138; scheduler.cpp:353 */
int reef_hal_memset_async(reef_devptr_t ptr, int byte, size_t bytes, reef_stream_t s);
int reef_hal_memcpy_h2d_async(reef_devptr_t dst, const void* src, size_t bytes, reef_stream_t s);
int reef_hal_memcpy_d2h_async(void* dst, reef_devptr_t src, size_t bytes, reef_stream_t s);

/* hipStreamCreate / hipStreamCreateWithWindowSize   scheduler.cpp:24-25,45-50; executor_base.cpp:78
 * launch_window <= 0: no limit. */
int reef_hal_stream_create(int launch_window, reef_stream_t* out);
int reef_hal_stream_destroy(reef_stream_t s);
/* How a windowed stream learns that a kernel has finished (the reference's patched runtime
 * tracks its launch window inside the driver, scheduler.cpp:45):
 *   REEF_COMPLETE_STREAM_WRITE  the layer appends a stream write of the launch's sequence
 *                               number after every kernel (on this runtime a small kernel of
 *                               its own, about 2 us of device time per launch);
 *   REEF_COMPLETE_IN_KERNEL     every kernel launched on the stream starts its argument block
 *                               with a reef_hal_completion and signals by itself.
 * Set before the first launch on the stream. */
int reef_hal_stream_set_completion(reef_stream_t s, int mode);
/* Launches handed to the device so far on a windowed stream, and how many have signalled. */
int reef_hal_stream_progress(reef_stream_t s, uint32_t* submitted, uint32_t* done);
/* *drained = 1 when nothing of a windowed stream is held back and every launch handed to the
 * device has signalled.  Reads the stream's counters only -- no call into the runtime, whose own
 * query may put a marker into the hardware queue that the kernels of other streams then queue
 * behind; for the real-time launch loop.  A stream without a window: reef_hal_stream_query. */
int reef_hal_stream_drained(reef_stream_t s, int* drained);
/* Device wall clock at which launch `seq` of a windowed stream in REEF_COMPLETE_IN_KERNEL mode
 * left the device (its last workgroup); kept for the 8 most recent launches.  0 if unknown. */
int reef_hal_stream_exit_ticks(reef_stream_t s, uint32_t seq, uint64_t* ticks);
/* One correlated reading of the host's monotonic clock (ns) and the device wall clock (ticks at
 * *ticks_per_us): a probe kernel answers a host-written word with its clock; the host time is
 * the middle of the exchange and *err_ns half its length (best of several exchanges). */
int reef_hal_clock_sync(int64_t* host_ns, uint64_t* device_ticks, int64_t* err_ns, int* ticks_per_us);
/* hipStreamSynchronize / hipStreamQuery / hipDeviceSynchronize   scheduler.cpp:335,339,356; hip_impl.cpp:77-80 */
int reef_hal_stream_sync(reef_stream_t s);
int reef_hal_stream_query(reef_stream_t s, int* idle);
int reef_hal_device_sync(void);
/* Move held launches of a windowed stream to the device while the window has room. */
int reef_hal_stream_pump(reef_stream_t s);

/* hipModuleLaunchKernel             executor_base.cpp:217-221
 * `kernarg` is the packed argument block (C struct layout of the kernel's
 * parameters); it is copied before the call returns. */
int reef_hal_launch(reef_function_t fn, const uint32_t grid[3], const uint32_t block[3],
                    uint32_t dyn_lds, reef_stream_t s, const void* kernarg, size_t kernarg_bytes);

/* hipStreamWriteValue32             scheduler.cpp:27,309,448,458 */
int reef_hal_write_value32(reef_stream_t s, reef_devptr_t ptr, int32_t value);
/* The same write without a stream (scheduler.cpp:309 raises the preemption flag through a
 * stream write and waits for that stream): `ptr` must come from reef_hal_malloc with
 * REEF_MEM_DEVICE_FINEGRAINED.  On a device whose memory is host-visible the word is stored
 * directly from the calling thread and is visible to running kernels about a microsecond later;
 * otherwise the layer falls back to a stream write it waits for.  No ordering against any stream. */
int reef_hal_host_write32(reef_devptr_t ptr, int32_t value);
/* The same for a run of 32-bit words: n_words stores of `value` from the calling thread into
 * REEF_MEM_DEVICE_FINEGRAINED memory, no device work and no stream.  Nothing on the device may
 * be using the words meanwhile.  Returns 2 where device memory cannot be stored to from the host
 * (the caller then fills through a stream). */
int reef_hal_host_fill32(reef_devptr_t ptr, int32_t value, size_t n_words);
/* Wait until the kernels `s` already has ON THE DEVICE have finished; launches the stream still
 * holds on the host stay there (hipStreamSynchronize after hipStreamClearQueue, scheduler.cpp:339).
 * For a windowed stream this spins on the stream's completion counter instead of sleeping in
 * the runtime. */
int reef_hal_stream_wait_device(reef_stream_t s);
/* hipStreamClearQueue (REEF-custom) scheduler.cpp:315 */
int reef_hal_stream_clear_queue(reef_stream_t s, uint64_t* n_dropped);
/* hipResetWavefronts (REEF-custom)  scheduler.cpp:333,341 */
int reef_hal_reset_cus(void);

/* Device-side timing for measurements (no counterpart in the reference, which
 * times on the host with system_clock, scheduler.cpp:378-410): events are
 * recorded on the stream the kernels were launched on. */
int reef_hal_event_create(reef_event_t* out);
int reef_hal_event_destroy(reef_event_t e);
int reef_hal_event_record(reef_event_t e, reef_stream_t s);
int reef_hal_event_sync(reef_event_t e);
int reef_hal_event_elapsed_us(reef_event_t start, reef_event_t stop, float* us);

/* One submission for a recorded sequence of launches (no counterpart in the reference,
 * which issues one hipModuleLaunchKernel per kernel, executor_base.cpp:191-221).  On this
 * device a launch call costs the host 3-4 us; a recorded sequence is replayed by the device
 * at under 2 us per kernel, which matters once kernels are shorter than a launch call.
 *   graph_begin(s): launches issued on `s` by the calling thread are recorded, not run;
 *   graph_end(s, &g): stops recording and builds the replayable sequence;
 *   graph_launch(g, s): enqueues the whole sequence on `s` (any stream without a launch window).
 * Only reef_hal_launch may be called on `s` between begin and end. */
int reef_hal_graph_begin(reef_stream_t s);
int reef_hal_graph_end(reef_stream_t s, reef_graph_t* out);
int reef_hal_graph_launch(reef_graph_t g, reef_stream_t s);
int reef_hal_graph_destroy(reef_graph_t g);

/*
 * Backend table.  The functions above forward to the active backend; the HIP
 * backend is the default and the only one the library ships.  Host-logic tests
 * install a recording backend of their own to drive the executors and the
 * scheduler without a GPU.
 */
typedef struct reef_hal_backend {
    int (*init)(int);
    int (*device_info)(reef_device_info*);
    int (*module_load)(const char*, reef_module_t*);
    int (*module_unload)(reef_module_t);
    int (*module_get_function)(reef_module_t, const char*, reef_function_t*);
    int (*function_resource)(reef_function_t, reef_kernel_resource*);
    int (*malloc_)(size_t, int, reef_devptr_t*);
    int (*free_)(reef_devptr_t, int);
    int (*memset_)(reef_devptr_t, int, size_t);
    int (*memcpy_h2d)(reef_devptr_t, const void*, size_t);
    int (*memcpy_d2h)(void*, reef_devptr_t, size_t);
    int (*memcpy_h2d_async)(reef_devptr_t, const void*, size_t, reef_stream_t);
    int (*memcpy_d2h_async)(void*, reef_devptr_t, size_t, reef_stream_t);
    int (*stream_create)(int, reef_stream_t*);
    int (*stream_destroy)(reef_stream_t);
    int (*stream_sync)(reef_stream_t);
    int (*stream_query)(reef_stream_t, int*);
    int (*device_sync)(void);
    int (*stream_pump)(reef_stream_t);
    int (*launch)(reef_function_t, const uint32_t*, const uint32_t*, uint32_t, reef_stream_t,
                  const void*, size_t);
    int (*write_value32)(reef_stream_t, reef_devptr_t, int32_t);
    int (*stream_clear_queue)(reef_stream_t, uint64_t*);
    int (*reset_cus)(void);
    int (*event_create)(reef_event_t*);
    int (*event_destroy)(reef_event_t);
    int (*event_record)(reef_event_t, reef_stream_t);
    int (*event_sync)(reef_event_t);
    int (*event_elapsed_us)(reef_event_t, reef_event_t, float*);
    int (*memset_async)(reef_devptr_t, int, size_t, reef_stream_t);
    int (*host_write32)(reef_devptr_t, int32_t);
    int (*stream_wait_device)(reef_stream_t);
    int (*graph_begin)(reef_stream_t);
    int (*graph_end)(reef_stream_t, reef_graph_t*);
    int (*graph_launch)(reef_graph_t, reef_stream_t);
    int (*graph_destroy)(reef_graph_t);
    int (*stream_set_completion)(reef_stream_t, int);
    int (*stream_progress)(reef_stream_t, uint32_t*, uint32_t*);
    int (*stream_exit_ticks)(reef_stream_t, uint32_t, uint64_t*);
    int (*clock_sync)(int64_t*, uint64_t*, int64_t*, int*);
    int (*module_kernel_entry)(reef_module_t, const char*, uint64_t*);
    int (*host_fill32)(reef_devptr_t, int32_t, size_t);
    int (*stream_drained)(reef_stream_t, int*);
} reef_hal_backend;

const reef_hal_backend* reef_hal_hip_backend(void);
void reef_hal_set_backend(const reef_hal_backend* b); /* NULL restores the HIP backend */
void reef_hal_set_error(const char* msg);

#ifdef __cplusplus
}
#endif
#endif /* REEF_HAL_H */
