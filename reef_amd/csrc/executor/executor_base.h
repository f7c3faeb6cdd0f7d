// ExecutorBase: loads one model (graph JSON + code object), owns its device
// storages and launches its kernels in JSON order.  Same public interface as
// the reference (src/reef/executor/executor_base.h:17-69).
//
// HBM layout: every storage entry lives in ONE device arena (a single
// allocation, each storage at a 256-byte aligned offset, zero-filled at load as
// executor_base.cpp:55-64 does per buffer).  Each kernel launch carries a
// ReefOpDesc by value: storage pointers in JSON `args` order plus the JSON
// `attrs` integers (include/reef_kernels.h).
#pragma once
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "executor/gpu_config.h"
#include "executor/model.h"
#include "reef_kernels.h"
#include "util/common.h"

namespace reef {
namespace executor {

class ExecutorBase {
public:
    ExecutorBase();
    virtual ~ExecutorBase();

    Status load_model_from_file(const char* json_file_path, const char* co_file_path);
    virtual Status load_model_from_GPU_module(const char* json_file_path, GPUModule_t module);
    Status load_param_from_file(const char* param_file_path);

    Status set_input(const std::string& key, const std::vector<float>& value);
    Status set_input(int idx, const void* value, size_t len);
    Status set_input(const std::string& key, const void* value, size_t len);
    Status get_data_size(const std::string& key, size_t& size);
    Status get_output(std::vector<float>& out);
    Status get_output(void* out, size_t len);
    Status get_data(int idx, void* out, size_t len);

    Status execute(GPUStream_t stream = GPUStreamDefault);
    Status execute_to(int idx, GPUStream_t stream = GPUStreamDefault);
    Status execute_kernel(int idx, GPUStream_t stream = GPUStreamDefault);

    size_t num_kernels() const;
    void set_stream(GPUStream_t stream);
    GPUStream_t stream();

    // Launches kernels [begin, end) without synchronising (for timing loops).
    Status launch_range(int begin, int end, GPUStream_t stream);
    // Enqueues the whole model without synchronising.  The kernel sequence of a model
    // never changes between runs (same functions, same argument blocks, same storages),
    // so it can be recorded once and replayed as ONE submission: the host then pays one
    // call instead of one per kernel.  Off by default (set_graph_launch(true), or
    // REEF_GRAPH=1 in the environment, turns it on): a launch call costs the host 3-4 us,
    // which hides behind kernels that run 5-15 us each, while a replay starts about
    // 0.1 ms later than the first direct launch would.  It pays for models whose kernels
    // are shorter than a launch call.
    Status launch_model(GPUStream_t stream);
    void set_graph_launch(bool on);
    bool graph_launch() const { return use_graph; }

    // Entry symbol of a graph-JSON kernel name ("symbol" or "symbol#instance").
    static std::string kernel_symbol(const std::string& name);

    std::unique_ptr<Model> model;

protected:
    Status init_executor_base(const char* json_file_path, GPUModule_t module);
    virtual Status launch_kernel(int kernel_offset, GPUStream_t stream);
    Status find_storage_idx(const std::string& name, size_t& idx);
    size_t storage_bytes(size_t idx) const;

protected:
    std::vector<GPUDevicePtr_t> storage;            // device address per storage entry
    std::vector<GPUFunction_t> kernel_funcs;        // per kernel call
    std::unordered_map<std::string, GPUFunction_t> kernels;  // by name
    std::vector<ReefOpDesc> descs;                  // per kernel call
    GPUDevicePtr_t arena;
    size_t arena_bytes;
    GPUDevicePtr_t sync_mem;   // the "reef_sync" storage (fine-grained memory of its own), or null
    GPUModule_t base_mod;
    GPUStream_t s;
    bool owns_stream;
    bool use_graph;
    reef_graph_t model_graph;
    void drop_graph();
};

}  // namespace executor
}  // namespace reef
