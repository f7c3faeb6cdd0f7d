// Device/resource model used by the executors and the scheduler.
// Same role and entry points as the reference's GPUConfig
// (src/reef/executor/hip/hip_impl.h:58-75, hip_impl.cpp:9-74), re-derived for
// gfx950 and answered by the C-ABI layer instead of hard-coded for a 60-CU part.
#pragma once
#include <algorithm>
#include <cstdint>

#include "reef_hal.h"
#include "util/common.h"

namespace reef {
namespace executor {

typedef reef_devptr_t GPUDevicePtr_t;
typedef reef_function_t GPUFunction_t;
typedef reef_module_t GPUModule_t;
typedef reef_stream_t GPUStream_t;
#define GPUStreamDefault ((::reef::executor::GPUStream_t) nullptr)

struct dim3u {
    uint32_t x, y, z;
    dim3u(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
    uint32_t count() const { return x * y * z; }
};

class GPUConfig {
public:
    typedef reef_kernel_resource KernelResource;

    // Virtual CUs a DKP launch is laid out over (hip_impl.cpp:9-12 returns 60).
    static uint32_t get_num_cus();
    static uint32_t get_num_xcds();
    // Tests may pin the geometry (0 restores the device's own).
    static void override_geometry(uint32_t num_cus, uint32_t num_xcds);

    static Status get_kernel_resource(GPUFunction_t func, KernelResource& ret);  // hip_impl.cpp:34-42

    static KernelResource max_resource(const KernelResource& a, const KernelResource& b) {  // :45-53
        // registers: the architectural VGPRs and the accumulation registers behind them are
        // two ranges of one file, so the union needs the larger of each
        KernelResource r;
        r.sgprs = std::max(a.sgprs, b.sgprs);
        r.agprs = std::max(a.agprs, b.agprs);
        const int arch = std::max(a.vgprs - a.agprs, b.vgprs - b.agprs);
        r.vgprs = std::max(std::max(a.vgprs, b.vgprs), r.agprs ? align_up(arch, 4) + r.agprs : arch);
        r.shared_memory = std::max(a.shared_memory, b.shared_memory);
        r.stack_size = std::max(a.stack_size, b.stack_size);
        return r;
    }

    // Workgroups resident per CU (hip_impl.cpp:55-74).
    static int calculate_occupancy(const KernelResource& resource, dim3u block_dim);
    static int calculate_occupancy(const KernelResource& resource, int block_threads);
};

bool GPUStreamEmpty(GPUStream_t s);  // hip_impl.cpp:77-80

}  // namespace executor
}  // namespace reef
