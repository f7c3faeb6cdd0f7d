#include "executor/gpu_config.h"

namespace reef {
namespace executor {

namespace {
uint32_t g_cus = 0, g_xcds = 0;      // overrides
uint32_t g_dev_cus = 0, g_dev_xcds = 0;
void query() {
    if (g_dev_cus) return;
    reef_device_info di;
    if (reef_hal_device_info(&di) == 0 && di.num_cus > 0) {
        g_dev_cus = (uint32_t)di.num_cus;
        g_dev_xcds = (uint32_t)std::max(di.num_xcds, 1);
    } else {
        g_dev_cus = 256;
        g_dev_xcds = 8;
    }
}
}  // namespace

uint32_t GPUConfig::get_num_cus() {
    if (g_cus) return g_cus;
    query();
    return g_dev_cus;
}
uint32_t GPUConfig::get_num_xcds() {
    if (g_cus) return g_xcds ? g_xcds : 1;
    query();
    return g_dev_xcds;
}
void GPUConfig::override_geometry(uint32_t num_cus, uint32_t num_xcds) {
    g_cus = num_cus;
    g_xcds = num_xcds;
}

Status GPUConfig::get_kernel_resource(GPUFunction_t func, KernelResource& ret) {
    GPU_RETURN_STATUS(reef_hal_function_resource(func, &ret));
    return Status::Succ;
}

int GPUConfig::calculate_occupancy(const KernelResource& resource, int block_threads) {
    int blocks = 0;
    if (reef_hal_occupancy(&resource, block_threads, 0, &blocks) != 0) return 0;
    return blocks;
}
int GPUConfig::calculate_occupancy(const KernelResource& resource, dim3u block_dim) {
    return calculate_occupancy(resource, (int)block_dim.count());
}

bool GPUStreamEmpty(GPUStream_t s) {
    int idle = 0;
    return reef_hal_stream_query(s, &idle) == 0 && idle != 0;
}

}  // namespace executor
}  // namespace reef
