#include "executor/hybrid_executor.h"

#include <cstddef>
#include <cstring>

namespace reef {
namespace executor {

static_assert(sizeof(reef_hal_completion) == 32 && offsetof(ReefBeArgs, preempted) == 32,
              "the best-effort argument block starts with the C-ABI layer's completion record");

HybridExecutor::HybridExecutor()
    : preempt_mod(nullptr), trans_mod(nullptr), preempt_flag(nullptr), owns_flag(false),
      task_slot_base(nullptr), task_slots_host_empty(nullptr), task_slots_host(nullptr),
      sync_ptr(nullptr), sync_bytes(0) {}

HybridExecutor::~HybridExecutor() {
    if (owns_flag && preempt_flag) reef_hal_free(preempt_flag, REEF_MEM_DEVICE_FINEGRAINED);
    if (task_slot_base) reef_hal_free(task_slot_base, REEF_MEM_DEVICE);
    if (task_slots_host) reef_hal_free(task_slots_host, REEF_MEM_HOST_PINNED);
    if (task_slots_host_empty) reef_hal_free(task_slots_host_empty, REEF_MEM_HOST_PINNED);
}

Status HybridExecutor::load_hybrid_model_from_file(const char* json_file_path,
                                                   const char* profile_file_path,
                                                   const char* trans_co_file_path,
                                                   const char* preempt_co_file_path) {
    GPU_RETURN_STATUS(reef_hal_init(0));
    GPUModule_t trans_module, preempt_module;
    REEF_LOG_INFO("%s", trans_co_file_path);
    GPU_RETURN_STATUS(reef_hal_module_load(trans_co_file_path, &trans_module));
    GPU_RETURN_STATUS(reef_hal_module_load(preempt_co_file_path, &preempt_module));
    return load_hybrid_model_from_GPU_module(json_file_path, profile_file_path, trans_module,
                                             preempt_module);
}

Status HybridExecutor::load_hybrid_model_from_GPU_module(const char* json_file_path,
                                                         const char* profile_file_path,
                                                         GPUModule_t trans_module,
                                                         GPUModule_t preempt_module) {
    Status ret = load_model_from_GPU_module(json_file_path, trans_module);
    if (ret != Status::Succ) return ret;
    return init_hybrid_executor(json_file_path, profile_file_path, trans_module, preempt_module);
}

Status HybridExecutor::init_hybrid_executor(const char* json_file_path,
                                            const char* profile_file_path,
                                            GPUModule_t trans_module, GPUModule_t preempt_module) {
    preempt_mod = preempt_module;
    trans_mod = trans_module;
    const size_t n = model->kernels.size();

    // 1. preemptible kernels (hybrid_executor.cpp:60-69)
    preempt_kernels.resize(n);
    std::unordered_map<std::string, GPUFunction_t> seen;
    for (size_t i = 0; i < n; i++) {
        const std::string name = kernel_symbol(model->kernels[i].name);
        auto it = seen.find(name);
        if (it == seen.end()) {
            GPUFunction_t fn;
            GPU_RETURN_STATUS(reef_hal_module_get_function(preempt_mod, name.c_str(), &fn));
            it = seen.emplace(name, fn).first;
        }
        preempt_kernels[i] = it->second;
    }

    // 2. preemption flag and per-kernel completion counters (hybrid_executor.cpp:71-77).
    // The flag is fine-grained device memory: kernels read it past their caches
    // while the host side rewrites it.
    GPU_RETURN_STATUS(reef_hal_malloc(4, REEF_MEM_DEVICE_FINEGRAINED, &preempt_flag));
    owns_flag = true;
    int zero = 0;
    GPU_RETURN_STATUS(reef_hal_memcpy_h2d(preempt_flag, &zero, 4));
    GPU_RETURN_STATUS(reef_hal_malloc(std::max<size_t>(n, 1) * 4, REEF_MEM_DEVICE, &task_slot_base));
    GPU_RETURN_STATUS(reef_hal_memset(task_slot_base, 0, std::max<size_t>(n, 1) * 4));

    size_t sync_idx;
    if (find_storage_idx("reef_sync", sync_idx) == Status::Succ) {
        sync_ptr = storage[sync_idx];
        sync_bytes = storage_bytes(sync_idx);
    }

    // 3. profile (hybrid_executor.cpp:92-97)
    model_profile.reset(ModelProfile::from_json(profile_file_path));
    if (!model_profile) RETURN_STATUS(Status::NotFound);
    for (size_t i = 0; i < n; i++)
        trans_args[i].profile = model_profile->kernel_latency[model->kernels[i].name];

    // 4. pinned mirrors of the counters for wait-based preemption (hybrid_executor.cpp:99-104)
    reef_devptr_t p = nullptr;
    GPU_RETURN_STATUS(reef_hal_malloc(std::max<size_t>(n, 1) * sizeof(int), REEF_MEM_HOST_PINNED, &p));
    task_slots_host = (int*)p;
    GPU_RETURN_STATUS(reef_hal_malloc(std::max<size_t>(n, 1) * sizeof(int), REEF_MEM_HOST_PINNED, &p));
    task_slots_host_empty = (int*)p;
    std::memset(task_slots_host, 0, n * sizeof(int));
    std::memset(task_slots_host_empty, 0, n * sizeof(int));
    return Status::Succ;
}

// The scheduler hands every executor its own shared flag (scheduler.cpp:94).
Status HybridExecutor::set_preempt_flag(GPUDevicePtr_t flag) {
    if (owns_flag && preempt_flag) GPU_RETURN_STATUS(reef_hal_free(preempt_flag, REEF_MEM_DEVICE_FINEGRAINED));
    owns_flag = false;
    preempt_flag = flag;
    return Status::Succ;
}

Status HybridExecutor::execute_preemptale(GPUStream_t stream) {
    for (size_t i = 0; i < model->kernels.size(); i++) {
        Status ret = launch_preempt_kernel((int)i, stream);
        if (ret != Status::Succ) return ret;
    }
    GPU_RETURN_STATUS(reef_hal_stream_sync(stream));
    return Status::Succ;
}

Status HybridExecutor::reset_task_slot_async(int kernel_offset, GPUStream_t stream) {
    GPU_RETURN_STATUS(reef_hal_write_value32(stream, (char*)task_slot_base + kernel_offset * 4, 0));
    return Status::Succ;
}

void HybridExecutor::reset_task_slots(GPUStream_t stream) {
    reef_hal_memcpy_h2d_async(task_slot_base, task_slots_host_empty, 4 * num_kernels(), stream);
}

// Zeroes the completion counters of kernels [first, n) in stream order.
Status HybridExecutor::reset_task_slots_from(int first, GPUStream_t stream) {
    const int n = (int)num_kernels();
    if (first < 0) first = 0;
    if (first >= n) return Status::Succ;
    GPU_RETURN_STATUS(reef_hal_memset_async((char*)task_slot_base + (size_t)first * 4, 0,
                                            (size_t)(n - first) * 4, stream));
    return Status::Succ;
}

void HybridExecutor::copy_be_kernel_offset(GPUStream_t stream) {
    reef_hal_memcpy_d2h_async(task_slots_host, task_slot_base, 4 * num_kernels(), stream);
}

// First kernel at or after `begin` whose workgroups did not all complete
// (hybrid_executor.cpp:141-151).
int HybridExecutor::get_be_kernel_offset(int begin) {
    for (size_t i = begin; i < num_kernels(); i++)
        if (task_slots_host[i] < trans_args[i].block_num) return (int)i;
    return (int)num_kernels();
}

Status HybridExecutor::reset_sync_storage(GPUStream_t stream) {
    if (sync_bytes == 0) return Status::Succ;
    GPU_RETURN_STATUS(reef_hal_memset_async(sync_ptr, 0, sync_bytes, stream));
    return Status::Succ;
}

// The same from the host, with no device operation; `fallback` is the stream the fill goes to
// where the host cannot store into device memory.  No kernel of the model may be running.
Status HybridExecutor::reset_sync_storage_from_host(GPUStream_t fallback) {
    if (sync_bytes == 0) return Status::Succ;
    const int rc = reef_hal_host_fill32(sync_ptr, 0, sync_bytes / 4);
    if (rc == 0) return Status::Succ;
    if (rc != 2) RETURN_STATUS(Status::Fail);
    return reset_sync_storage(fallback);
}

Status HybridExecutor::launch_preempt_kernel(int i, GPUStream_t stream) {
    const KernelArg& ka = trans_args[i];
    ReefBeArgs arg;
    std::memset(&arg, 0, sizeof(reef_hal_completion));   // filled by the layer on a windowed stream
    arg.preempted = (int*)preempt_flag;
    arg.task_slot = (int*)((char*)task_slot_base + i * 4);
    arg.desc = descs[i];
    const uint32_t grid[3] = {ka.task_dim.x, ka.task_dim.y, ka.task_dim.z};
    const uint32_t block[3] = {ka.thread_dim.x, ka.thread_dim.y, ka.thread_dim.z};
    GPU_RETURN_STATUS(reef_hal_launch(preempt_kernels[i], grid, block, 0, stream, &arg, sizeof(arg)));
    return Status::Succ;
}

}  // namespace executor
}  // namespace reef
