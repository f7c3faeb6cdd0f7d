#include "executor/executor_base.h"
#include "executor/op_extents.h"

#include <cstdlib>

#include <cstring>

namespace reef {
namespace executor {

ExecutorBase::ExecutorBase()
    : arena(nullptr), arena_bytes(0), sync_mem(nullptr), base_mod(nullptr), s(nullptr), owns_stream(false),
      use_graph(std::getenv("REEF_GRAPH") != nullptr), model_graph(nullptr) {}

ExecutorBase::~ExecutorBase() {
    drop_graph();
    if (owns_stream && s) reef_hal_stream_destroy(s);
    if (arena) reef_hal_free(arena, REEF_MEM_DEVICE);
    if (sync_mem) reef_hal_free(sync_mem, REEF_MEM_DEVICE_FINEGRAINED);
}

Status ExecutorBase::load_model_from_file(const char* json_file_path, const char* co_file_path) {
    GPU_RETURN_STATUS(reef_hal_init(0));
    GPUModule_t mod;
    GPU_RETURN_STATUS(reef_hal_module_load(co_file_path, &mod));
    return this->load_model_from_GPU_module(json_file_path, mod);
}

Status ExecutorBase::load_model_from_GPU_module(const char* json_file_path, GPUModule_t mod) {
    return init_executor_base(json_file_path, mod);
}

std::string ExecutorBase::kernel_symbol(const std::string& name) {
    const size_t p = name.find('#');
    return p == std::string::npos ? name : name.substr(0, p);
}

size_t ExecutorBase::storage_bytes(size_t idx) const {
    const StorageInfo& si = model->storage[idx];
    return Model::get_stype_size(si.stype) * si.size;
}

Status ExecutorBase::init_executor_base(const char* json_file_path, GPUModule_t mod) {
    base_mod = mod;
    model.reset(Model::from_json(json_file_path));
    if (model.get() == nullptr) RETURN_STATUS(Status::NotFound);

    // kernels: one lookup per distinct name
    kernel_funcs.clear();
    for (KernelInfo& ki : model->kernels) {
        // "symbol#instance": the part before '#' is the entry symbol, the whole
        // string keys the per-kernel profile (one symbol serves many layers here).
        const std::string sym = kernel_symbol(ki.name);
        auto it = kernels.find(sym);
        if (it == kernels.end()) {
            GPUFunction_t fn;
            GPU_RETURN_STATUS(reef_hal_module_get_function(mod, sym.c_str(), &fn));
            it = kernels.emplace(sym, fn).first;
        }
        kernel_funcs.push_back(it->second);
        if (ki.args.size() > REEF_MAX_PTRS || ki.attrs.size() > REEF_MAX_ATTRS) {
            REEF_LOG_ERROR("kernel %s: too many args/attrs", ki.name.c_str());
            return Status::OutOfRange;
        }
    }

    // every kernel must fit the storages it is given and the grid it is launched with
    for (size_t i = 0; i < model->kernels.size(); ++i) {
        std::string why;
        if (!kernel_fits_storages(*model, i, &why)) {
            REEF_LOG_ERROR("%s: %s", json_file_path, why.c_str());
            return Status::OutOfRange;
        }
    }

    // storages: one zero-filled arena
    std::vector<size_t> offs(model->storage.size());
    size_t total = 0;
    // The arrival counters of folded split-K launches ("reef_sync") live in fine-grained memory
    // of their own: the scheduler clears them from the host, without a device operation, before
    // it pads a kernel of a model whose last run was cut short.
    size_t sync_idx = model->storage.size();
    for (size_t i = 0; i < model->storage.size(); ++i) {
        if (Model::get_stype_size(model->storage[i].stype) == 0) return Status::Fail;
        if (model->storage[i].name == "reef_sync" && sync_idx == model->storage.size()) {
            sync_idx = i;
            continue;
        }
        offs[i] = total;
        total += align_up<size_t>(std::max<size_t>(storage_bytes(i), 4), 256);
    }
    arena_bytes = std::max<size_t>(total, 256);
    GPU_RETURN_STATUS(reef_hal_malloc(arena_bytes, REEF_MEM_DEVICE, &arena));
    GPU_RETURN_STATUS(reef_hal_memset(arena, 0, arena_bytes));
    storage.resize(model->storage.size());
    for (size_t i = 0; i < storage.size(); ++i) storage[i] = (char*)arena + offs[i];
    if (sync_idx < model->storage.size()) {
        const size_t bytes = align_up<size_t>(std::max<size_t>(storage_bytes(sync_idx), 4), 256);
        GPU_RETURN_STATUS(reef_hal_malloc(bytes, REEF_MEM_DEVICE_FINEGRAINED, &sync_mem));
        GPU_RETURN_STATUS(reef_hal_memset(sync_mem, 0, bytes));
        storage[sync_idx] = sync_mem;
    }

    // per-call descriptors
    descs.assign(model->kernels.size(), ReefOpDesc());
    for (size_t i = 0; i < model->kernels.size(); ++i) {
        const KernelInfo& ki = model->kernels[i];
        ReefOpDesc& d = descs[i];
        std::memset(&d, 0, sizeof(d));
        for (size_t j = 0; j < ki.args.size(); ++j)
            d.ptr[j] = (char*)storage[ki.args[j]] + (ki.arg_offsets.empty() ? 0 : ki.arg_offsets[j]);
        for (size_t j = 0; j < ki.attrs.size(); ++j) d.attr[j] = ki.attrs[j];
    }

    return Status::Succ;
}

Status ExecutorBase::load_param_from_file(const char* param_file_path) {
    std::unique_ptr<ModelParam> params(ModelParamParser::parse_from_file(param_file_path));
    if (!params) RETURN_STATUS(Status::NotFound);
    for (size_t i = 0; i < storage.size(); i++) {
        auto it = params->find(model->storage[i].name);
        if (it == params->end()) continue;
        // The reference copies the whole tensor without a size check
        // (executor_base.cpp:90-92); never write past the storage here.
        size_t bytes = std::min(it->second.size() * sizeof(float), storage_bytes(i));
        GPU_RETURN_STATUS(reef_hal_memcpy_h2d(storage[i], it->second.data(), bytes));
    }
    return Status::Succ;
}

Status ExecutorBase::get_data_size(const std::string& key, size_t& size) {
    size_t idx;
    if (find_storage_idx(key, idx) != Status::Succ) RETURN_STATUS(Status::NotFound);
    size = storage_bytes(idx);
    return Status::Succ;
}

Status ExecutorBase::set_input(const std::string& key, const std::vector<float>& value) {
    return set_input(key, (const void*)value.data(), value.size() * sizeof(float));
}

Status ExecutorBase::set_input(const std::string& key, const void* value, size_t len) {
    size_t idx;
    if (find_storage_idx(key, idx) != Status::Succ) RETURN_STATUS(Status::NotFound);
    return set_input((int)idx, value, len);
}

Status ExecutorBase::set_input(int idx, const void* value, size_t len) {
    if (idx < 0 || (size_t)idx >= storage.size()) RETURN_STATUS(Status::OutOfRange);
    const size_t bytes = storage_bytes(idx);
    if (len < bytes) RETURN_STATUS(Status::OutOfRange);
    GPU_RETURN_STATUS(reef_hal_memcpy_h2d(storage[idx], value, bytes));
    return Status::Succ;
}

Status ExecutorBase::get_output(std::vector<float>& out) {
    size_t idx;
    if (find_storage_idx("output", idx) != Status::Succ) RETURN_STATUS(Status::NotFound);
    if (Model::get_stype_size(model->storage[idx].stype) != sizeof(float)) RETURN_STATUS(Status::Fail);
    out.resize(model->storage[idx].size);
    return get_data((int)idx, (void*)out.data(), out.size() * sizeof(float));
}

Status ExecutorBase::get_output(void* out, size_t len) {
    size_t idx;
    if (find_storage_idx("output", idx) != Status::Succ) RETURN_STATUS(Status::NotFound);
    if (len < storage_bytes(idx)) RETURN_STATUS(Status::Fail);
    return get_data((int)idx, out, len);
}

Status ExecutorBase::get_data(int idx, void* out, size_t len) {
    if (idx < 0 || (size_t)idx >= storage.size()) RETURN_STATUS(Status::OutOfRange);
    const size_t bytes = storage_bytes(idx);
    if (len < bytes) RETURN_STATUS(Status::Fail);
    GPU_RETURN_STATUS(reef_hal_memcpy_d2h(out, storage[idx], bytes));
    return Status::Succ;
}

Status ExecutorBase::find_storage_idx(const std::string& name, size_t& idx) {
    for (size_t i = 0; i < model->storage.size(); i++) {
        if (model->storage[i].name == name) {
            idx = i;
            return Status::Succ;
        }
    }
    return Status::NotFound;
}

size_t ExecutorBase::num_kernels() const { return model->kernels.size(); }
void ExecutorBase::set_stream(GPUStream_t stream) {
    if (owns_stream && s) reef_hal_stream_destroy(s);
    owns_stream = false;
    s = stream;
}
// The model's own stream is made on first use: an executor that a scheduler drives
// runs on the scheduler's streams and never needs one, and every stream that exists
// takes a share of the few hardware queues.
GPUStream_t ExecutorBase::stream() {
    if (!s) {
        REEF_LOG_INFO("create base model stream");
        if (reef_hal_stream_create(0, &s) == 0) owns_stream = true;
    }
    return s;
}

// The reference's execute(stream) drops its argument and runs on the default
// stream (executor_base.cpp:191-194); here the stream is honoured.
Status ExecutorBase::execute(GPUStream_t stream) { return execute_to((int)num_kernels(), stream); }

Status ExecutorBase::execute_to(int idx, GPUStream_t stream) {
    if (idx < 0 || (size_t)idx > num_kernels()) RETURN_STATUS(Status::OutOfRange);
    if ((size_t)idx == num_kernels()) RETURN_STATUS(launch_model(stream));
    else for (int i = 0; i < idx; i++) RETURN_STATUS(launch_kernel(i, stream));
    GPU_RETURN_STATUS(reef_hal_stream_sync(stream));
    return Status::Succ;
}

void ExecutorBase::set_graph_launch(bool on) {
    use_graph = on;
    if (!on) drop_graph();
}

void ExecutorBase::drop_graph() {
    if (model_graph) reef_hal_graph_destroy(model_graph);
    model_graph = nullptr;
}

Status ExecutorBase::launch_model(GPUStream_t stream) {
    const int n = (int)num_kernels();
    if (!use_graph || !stream || n == 0) return launch_range(0, n, stream);
    if (!model_graph) {
        GPU_RETURN_STATUS(reef_hal_graph_begin(stream));
        Status st = launch_range(0, n, stream);
        reef_graph_t g = nullptr;
        const int rc = reef_hal_graph_end(stream, &g);
        if (st != Status::Succ) {
            if (rc == 0) reef_hal_graph_destroy(g);
            RETURN_STATUS(st);
        }
        GPU_RETURN_STATUS(rc);
        model_graph = g;
    }
    GPU_RETURN_STATUS(reef_hal_graph_launch(model_graph, stream));
    return Status::Succ;
}

Status ExecutorBase::execute_kernel(int idx, GPUStream_t stream) {
    if (idx < 0 || (size_t)idx >= num_kernels()) RETURN_STATUS(Status::OutOfRange);
    RETURN_STATUS(launch_kernel(idx, stream));
    GPU_RETURN_STATUS(reef_hal_stream_sync(stream));
    return Status::Succ;
}

Status ExecutorBase::launch_range(int begin, int end, GPUStream_t stream) {
    if (begin < 0 || end < begin || (size_t)end > num_kernels()) RETURN_STATUS(Status::OutOfRange);
    for (int i = begin; i < end; i++) RETURN_STATUS(launch_kernel(i, stream));
    return Status::Succ;
}

Status ExecutorBase::launch_kernel(int i, GPUStream_t stream) {
    const uint32_t* lp = model->kernels[i].launch_params;
    GPU_RETURN_STATUS(reef_hal_launch(kernel_funcs[i], lp, lp + 3, 0, stream, &descs[i],
                                      sizeof(ReefOpDesc)));
    return Status::Succ;
}

}  // namespace executor
}  // namespace reef
