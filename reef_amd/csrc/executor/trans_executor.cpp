#include "executor/trans_executor.h"

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

int TransExecutor::op_from_name(const std::string& n) {
    struct { const char* prefix; int op; } table[] = {
        {"reef_conv2d_", REEF_OP_CONV2D}, {"reef_gemm_", REEF_OP_GEMM},
        {REEF_K_SPLITK_REDUCE, REEF_OP_SPLITK_REDUCE}, {REEF_K_DWCONV2D, REEF_OP_DWCONV2D},
        {REEF_K_POOL2D, REEF_OP_POOL2D}, {REEF_K_GLOBAL_AVGPOOL, REEF_OP_GLOBAL_AVGPOOL},
        {REEF_K_ELTWISE, REEF_OP_ELTWISE}, {REEF_K_DENSE, REEF_OP_DENSE},
        {REEF_K_SOFTMAX, REEF_OP_SOFTMAX}, {REEF_K_LAYERNORM, REEF_OP_LAYERNORM},
        {REEF_K_BIAS_GELU, REEF_OP_BIAS_GELU}, {REEF_K_EMBEDDING, REEF_OP_EMBEDDING},
        {REEF_K_COPY, REEF_OP_COPY}, {REEF_K_TRANSPOSE, REEF_OP_TRANSPOSE},
        {REEF_K_MOCK_ADD, REEF_OP_MOCK_ADD}, {REEF_K_MOCK_MULTIPLY, REEF_OP_MOCK_MULTIPLY},
    };
    for (auto& e : table) {
        const size_t len = std::strlen(e.prefix);
        const bool is_prefix = e.prefix[len - 1] == '_';
        if (is_prefix ? n.compare(0, len, e.prefix) == 0 : n == e.prefix) return e.op;
    }
    return REEF_OP_NONE;
}

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
        int tile = -1, mode = 0, taps = 0;
        if (ka.op == REEF_OP_CONV2D && ki.attrs.size() > REEF_CONV_MODE) {
            tile = ki.attrs[REEF_CONV_TILE];
            mode = ki.attrs[REEF_CONV_MODE];
            taps = ki.attrs[REEF_CONV_KH] * ki.attrs[REEF_CONV_KW];
        }
        ka.proxy_level = proxy_level(ka.op, tile, mode, taps);
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

    // proxies: one per occupancy class that the code object provides
    proxy_kernels.clear();
    for (int level = 0; level < kNumProxyLevels; level++) {
        GPUFunction_t f;
        const std::string name = REEF_PROXY_KERNEL_PREFIX() + std::to_string(proxy_class_of_level(level));
        GPU_RETURN_STATUS(reef_hal_module_get_function(module, name.c_str(), &f));
        proxy_kernels.push_back(f);
    }
    GPUConfig::KernelResource kr;
    RETURN_STATUS(GPUConfig::get_kernel_resource(proxy_kernels[0], kr));
    max_stack_size = kr.stack_size;
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

// One single-sided launch with an explicit layer count and task range (profiling).
Status TransExecutor::launch_kernel_dkp(int i, int layers, int task_num, GPUStream_t stream) {
    const KernelArg& ka = trans_args[i];
    const int num_cus = (int)GPUConfig::get_num_cus();
    ReefDkpArgs a;
    std::memset(&a, 0, sizeof(a));
    fill_side(a.l, i, layers, std::min(task_num, ka.block_num), 0);
    a.r = a.l;
    a.r.task_num = 0;
    a.cu_partition = num_cus;
    a.num_cus = num_cus;
    a.num_xcds = (int)GPUConfig::get_num_xcds();
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

int TransExecutor::proxy_class_of_level(int level) {
    static const int cls[kNumProxyLevels] = {8, 3, 2};
    return cls[std::max(0, std::min(level, kNumProxyLevels - 1))];
}

// Which proxy holds the body of (op, tile, loader family): the bandwidth-bound ops
// are in every proxy, a few matrix-core tiles in the classes whose register budget
// fits them, and everything else in none (-1: that kernel is never merged).
int TransExecutor::proxy_level(int op, int tile, int mode, int taps) {
    if (op == REEF_OP_CONV2D) {
        if (mode == REEF_CONV_MODE_DIRECT)
            return ((tile == REEF_TILE_16x16k4 || tile == REEF_TILE_16x32k4) && (taps == 1 || taps == 9)) ? 1 : -1;
        if (mode != REEF_CONV_MODE_GENERAL && mode != REEF_CONV_MODE_POINTWISE) return -1;
        if (tile == REEF_TILE_64x64 || tile == REEF_TILE_128x32) return 1;
        if (tile == REEF_TILE_128x64) return 2;
        if (tile == REEF_TILE_32x32k4 || tile == REEF_TILE_64x32k2 || tile == REEF_TILE_32x64k2)
            return 2;
        return -1;
    }
    if (op == REEF_OP_GEMM || op == REEF_OP_NONE) return -1;
    return 0;
}

GPUFunction_t TransExecutor::get_proxy_kernel(int level) {
    return proxy_kernels[std::max(0, std::min(level, (int)proxy_kernels.size() - 1))];
}

}  // namespace executor
}  // namespace reef
