// TransExecutor: launches the dynamic-kernel-padding (DKP) flavour of a model.
// Same role as the reference's class (src/reef/executor/trans_executor.h:41-87):
// per kernel call it records the logical grid, the resources, the minimal
// occupancy a real-time run needs and the packed launch arguments; a launch
// covers occupancy x num_cus physical workgroups that walk the logical tasks
// with a persistent loop.
//
// What changed for MI355X: the side descriptor carries a ReefOpDesc (shapes and
// pointers by value) instead of a float** table in device memory, the proxy
// classes are the gfx950 register classes, and the CU geometry (256 virtual
// CUs in 8 XCD groups) comes from the device.
#pragma once
#include "executor/executor_base.h"

namespace reef {
namespace executor {

class TransExecutor : public ExecutorBase {
public:
    TransExecutor();
    virtual ~TransExecutor();
    virtual Status load_model_from_GPU_module(const char* json_file_path, GPUModule_t module) override;

    class KernelArg {  // trans_executor.h:47-63
    public:
        GPUFunction_t kernel;
        int op;                 // REEF_OP_* of this call
        uint64_t entry;         // device address of the kernel's first instruction (funcion_pointer, trans_executor.h:50)
        dim3u task_dim;
        dim3u thread_dim;
        int block_num;
        int block_offset;
        int cu_lower;
        int cu_upper;
        int min_occupancy;      // layers a real-time launch needs
        GPUConfig::KernelResource resource;
        KernelProfile profile;
    };

    // DKP arithmetic (trans_executor.cpp:91-97,138-140; scheduler.cpp:524-526,578).
    static int logical_layers(int block_num, int num_cus);
    static int cu_partition_for(int block_num, int num_cus, int num_xcds);
    static int op_from_name(const std::string& name);

    const std::vector<KernelArg>& kernel_args() const { return trans_args; }
    Status launch_kernel_dkp(int kernel_offset, int layers, int task_num, GPUStream_t stream, int cus = 0);
    // Waves per SIMD a register count allows on gfx950
    // (trans_executor.cpp:175-199 picks among 10 gfx906 classes the same way).
    static int occupancy_class(const GPUConfig::KernelResource& kr);
    // The merge_framework_<n> proxies of the code object, most wavefronts per SIMD first.  A
    // proxy fixes the register file of a merged launch: `resource.vgprs - resource.agprs`
    // architectural VGPRs and `resource.agprs` accumulation registers.
    struct Proxy {
        std::string name;
        GPUFunction_t kernel;
        GPUConfig::KernelResource resource;
    };
    static const char* const kProxyNames[];
    static constexpr int kNumProxies = 9;
    // First proxy (= most wavefronts) whose two register ranges hold both kernels; -1 when a
    // kernel needs scratch memory or more registers than any proxy has
    // (trans_executor.cpp:175-199 picks among 10 + 10 gfx906 classes the same way).
    static int select_proxy(const std::vector<Proxy>& proxies, const GPUConfig::KernelResource& l,
                            const GPUConfig::KernelResource& r);
    int select_proxy(const GPUConfig::KernelResource& l, const GPUConfig::KernelResource& r) const {
        return select_proxy(proxy_kernels, l, r);
    }
    const std::vector<Proxy>& proxies() const { return proxy_kernels; }

protected:
    Status init_rt_executor(const char* json_file_path, GPUModule_t module);
    virtual Status launch_kernel(int kernel_offset, GPUStream_t stream) override;
    GPUFunction_t get_proxy_kernel(int index);
    void fill_side(ReefDkpSide& side, int kernel_offset, int layers, int task_num, int task_offset) const;

protected:
    std::vector<KernelArg> trans_args;
    std::vector<Proxy> proxy_kernels;
    int max_stack_size;

    virtual std::string REEF_PROXY_KERNEL_PREFIX() const { return "merge_framework_"; }
};

}  // namespace executor
}  // namespace reef
