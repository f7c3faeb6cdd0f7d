// HybridExecutor: a model in two flavours -- the DKP flavour inherited from
// TransExecutor and the preemptible best-effort flavour whose kernels take
// (int* preempted, int* task_slot, ReefOpDesc).  Same interface as the
// reference (src/reef/executor/hybrid_executor.h:18-76).
#pragma once
#include "executor/trans_executor.h"

namespace reef {
namespace server {
class REEFScheduler;
}
namespace executor {

class HybridExecutor : public TransExecutor {
    friend class server::REEFScheduler;

public:
    HybridExecutor();
    virtual ~HybridExecutor();

    Status load_hybrid_model_from_file(const char* json_file_path, const char* profile_file_path,
                                       const char* trans_co_file_path,
                                       const char* preempt_co_file_path);
    Status load_hybrid_model_from_GPU_module(const char* json_file_path,
                                             const char* profile_file_path,
                                             GPUModule_t trans_module, GPUModule_t preempt_module);

    Status execute_preemptale(GPUStream_t stream = GPUStreamDefault);  // spelling as in the reference
    Status set_preempt_flag(GPUDevicePtr_t flag);

    Status reset_task_slot_async(int kernel_offset, GPUStream_t stream);
    void reset_task_slots(GPUStream_t stream);
    Status reset_task_slots_from(int first_kernel, GPUStream_t stream);
    void copy_be_kernel_offset(GPUStream_t stream);
    int get_be_kernel_offset(int begin);

    Status launch_preempt_kernel(int kernel_offset, GPUStream_t stream);
    // Zeroes the model's "reef_sync" storage (the arrival counters of kernels that
    // fold split-K internally) in stream order.  Needed before kernels of this model
    // run again after an interrupted run; a no-op for models without that storage.
    Status reset_sync_storage(GPUStream_t stream);
    Status reset_sync_storage_from_host(GPUStream_t fallback);
    bool has_sync_storage() const { return sync_bytes > 0; }
    const ModelProfile* profile() const { return model_profile.get(); }

protected:
    Status init_hybrid_executor(const char* json_file_path, const char* profile_file_path,
                                GPUModule_t trans_module, GPUModule_t preempt_module);

protected:
    GPUModule_t preempt_mod;
    GPUModule_t trans_mod;
    std::vector<GPUFunction_t> preempt_kernels;
    GPUDevicePtr_t preempt_flag;
    bool owns_flag;
    GPUDevicePtr_t task_slot_base;
    int* task_slots_host_empty;
    int* task_slots_host;
    std::shared_ptr<ModelProfile> model_profile;
    GPUDevicePtr_t sync_ptr;
    size_t sync_bytes;
};

}  // namespace executor
}  // namespace reef
