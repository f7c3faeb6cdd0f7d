#include "executor/trans_executor.h"
#include "executor/op_extents.h"

#include <cstring>

namespace reef {
namespace executor {

TransExecutor::TransExecutor() : max_stack_size(0) {}
TransExecutor::~TransExecutor() {}

Status TransExecutor::load_model_from_GPU_module(const char* json_file_path, GPUModule_t module) {
    Status ret = init_executor_base(json_file_path, module);
    if (ret != Status::Succ) return ret;
    return init_rt_executor(json_file_path, module);
}

int TransExecutor::logical_layers(int block_num, int num_cus) {
    return ceil_div(block_num, num_cus);
}

// CUs the kernel really needs: ceil(blocks / layers), rounded up to a whole
// number of slots on every XCD so both sides of a split launch get the same
// share of each XCD.
int TransExecutor::cu_partition_for(int block_num, int num_cus, int num_xcds) {
    const int layers = std::max(logical_layers(block_num, num_cus), 1);
    int part = ceil_div(block_num, layers);
    part = ceil_div(part, num_xcds) * num_xcds;
    return std::min(part, num_cus);
}

int TransExecutor::op_from_name(const std::string& n) { return op_from_symbol(n); }

Status TransExecutor::init_rt_executor(const char* json_file_path, GPUModule_t module) {
    const size_t n = model->kernels.size();
    const int num_cus = (int)GPUConfig::get_num_cus();
    trans_args.resize(n);
    for (size_t i = 0; i < n; i++) {
        KernelArg& ka = trans_args[i];
        const KernelInfo& ki = model->kernels[i];
        const uint32_t* lp = ki.launch_params;
        ka.kernel = kernel_funcs[i];
        ka.op = op_from_name(kernel_symbol(ki.name));
        ka.entry = 0;
        GPU_RETURN_STATUS(reef_hal_module_kernel_entry(module, kernel_symbol(ki.name).c_str(), &ka.entry));
        ka.task_dim = dim3u(lp[0], lp[1], lp[2]);
        ka.thread_dim = dim3u(lp[3], lp[4], lp[5]);
        ka.block_num = (int)ka.task_dim.count();
        ka.block_offset = 0;
        ka.cu_lower = 0;
        ka.cu_upper = num_cus;
        RETURN_STATUS(GPUConfig::get_kernel_resource(ka.kernel, ka.resource));
        // min_occupancy = min(ceil(blocks / CUs), resident blocks per CU)  (trans_executor.cpp:91-97)
        const int max_layers = GPUConfig::calculate_occupancy(ka.resource, ka.thread_dim);
        int layers = logical_layers(ka.block_num, num_cus);
        if (layers > max_layers) layers = max_layers;
        ka.min_occupancy = std::max(layers, 1);
    }

    // proxies: every register class of the code object (trans_executor.cpp:100-124 resolves 20)
    proxy_kernels.clear();
    for (int p = 0; p < kNumProxies; p++) {
        Proxy px;
        px.name = REEF_PROXY_KERNEL_PREFIX() + kProxyNames[p];
        GPU_RETURN_STATUS(reef_hal_module_get_function(module, px.name.c_str(), &px.kernel));
        RETURN_STATUS(GPUConfig::get_kernel_resource(px.kernel, px.resource));
        proxy_kernels.push_back(px);
    }
    max_stack_size = proxy_kernels[0].resource.stack_size;
    return Status::Succ;
}

void TransExecutor::fill_side(ReefDkpSide& side, int i, int layers, int task_num, int task_offset) const {
    side.op = trans_args[i].op;
    side.layers = layers;
    side.task_num = task_num;
    side.task_offset = task_offset;
    side.desc = descs[i];
}

// Single-sided launch: the whole grid belongs to side l (trans_executor.cpp:143-171
// passes cu_partition = num_cus and duplicates the left side into the right one).
Status TransExecutor::launch_kernel(int i, GPUStream_t stream) {
    const KernelArg& ka = trans_args[i];
    const int num_cus = (int)GPUConfig::get_num_cus();
    ReefDkpArgs a;
    std::memset(&a, 0, sizeof(a));
    fill_side(a.l, i, ka.min_occupancy, ka.block_num, ka.block_offset);
    a.r = a.l;
    a.r.task_num = 0;
    a.cu_partition = num_cus;
    a.num_cus = num_cus;
    a.num_xcds = (int)GPUConfig::get_num_xcds();
    a.task_slot_r = nullptr;
    const uint32_t grid[3] = {(uint32_t)(num_cus * ka.min_occupancy), 1, 1};
    const uint32_t block[3] = {ka.thread_dim.count(), 1, 1};
    GPU_RETURN_STATUS(reef_hal_launch(ka.kernel, grid, block, 0, stream, &a, sizeof(a)));
    return Status::Succ;
}

// One single-sided launch with an explicit layer count and task range (profiling).  cus > 0:
// the kernel is confined to that many virtual CUs as the best-effort side of a padded launch is
// (the right side of a partition with nothing on the left), so `layers` workgroups really share
// each of those CUs.
Status TransExecutor::launch_kernel_dkp(int i, int layers, int task_num, GPUStream_t stream, int cus) {
    const KernelArg& ka = trans_args[i];
    const int num_cus = (int)GPUConfig::get_num_cus();
    const int num_xcds = (int)GPUConfig::get_num_xcds();
    ReefDkpArgs a;
    std::memset(&a, 0, sizeof(a));
    fill_side(a.l, i, layers, std::min(task_num, ka.block_num), 0);
    a.r = a.l;
    a.r.task_num = 0;
    a.cu_partition = num_cus;
    if (cus > 0 && cus < num_cus) {
        a.r = a.l;
        a.l.task_num = 0;
        a.cu_partition = num_cus - align_up(cus, num_xcds);
    }
    a.num_cus = num_cus;
    a.num_xcds = num_xcds;
    const uint32_t grid[3] = {(uint32_t)(num_cus * layers), 1, 1};
    const uint32_t block[3] = {ka.thread_dim.count(), 1, 1};
    GPU_RETURN_STATUS(reef_hal_launch(ka.kernel, grid, block, 0, stream, &a, sizeof(a)));
    return Status::Succ;
}

// Waves per SIMD the merged resource allows on gfx950 (512-entry VGPR file in
// granules of 8, at most 8 waves): class n = floor(512 / vgprs) clamped to 1..8.
int TransExecutor::occupancy_class(const GPUConfig::KernelResource& kr) {
    const int v = std::max(align_up(std::max(kr.vgprs, 1), 8), 8);
    return std::max(1, std::min(8, 512 / v));
}

const char* const TransExecutor::kProxyNames[] = {"8", "5", "4", "3", "3b", "2", "2b", "2c", "1"};

int TransExecutor::select_proxy(const std::vector<Proxy>& proxies, const GPUConfig::KernelResource& l,
                                const GPUConfig::KernelResource& r) {
    if (l.stack_size > 0 || r.stack_size > 0) return -1;   // a proxy starts its wavefronts without scratch
    const int arch = std::max(l.vgprs - l.agprs, r.vgprs - r.agprs);
    const int acc = std::max(l.agprs, r.agprs);
    const int sgprs = std::max(l.sgprs, r.sgprs);
    for (size_t p = 0; p < proxies.size(); p++) {
        const GPUConfig::KernelResource& pr = proxies[p].resource;
        if (arch <= pr.vgprs - pr.agprs && acc <= pr.agprs && sgprs <= pr.sgprs) return (int)p;
    }
    return -1;
}

GPUFunction_t TransExecutor::get_proxy_kernel(int index) {
    return proxy_kernels[std::max(0, std::min(index, (int)proxy_kernels.size() - 1))].kernel;
}

}  // namespace executor
}  // namespace reef
