// Model resource formats: graph JSON, per-kernel profile JSON, binary .param.
// Same types and entry points as the reference (src/reef/executor/model.h:14-58);
// files written for either implementation load in the other.  Differences:
// a malformed file yields nullptr (the reference asserts), and a kernel entry
// may carry an "attrs" integer list, which the shape-generic gfx950 kernels
// need and the reference's parser ignores (model.cpp:23-51 looks up known keys only).
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace reef {
namespace executor {

class StorageInfo {
public:
    std::string name;
    size_t size;  // element count
    std::string stype;
};

class KernelInfo {
public:
    std::string name;
    uint32_t launch_params[6];  // grid x,y,z, block x,y,z
    std::vector<size_t> args;   // storage indices, bound positionally
    std::vector<int32_t> attrs; // per-launch shape attributes (may be empty)
    // Optional "arg_offsets": per argument the byte at which the operand starts inside its
    // storage (empty = every operand starts at its storage's first byte).  A channel range of a
    // tensor is one contiguous piece of its storage, so a kernel can read or write a part of a
    // larger buffer without a variant of its own.  The reference's reader ignores the key.
    std::vector<size_t> arg_offsets;
};

class Model {
public:
    std::vector<StorageInfo> storage;
    std::vector<KernelInfo> kernels;
    std::vector<uint32_t> args;
    std::unordered_map<std::string, size_t> shared_memory;

    // model.cpp:13-55.  Caller owns the result; nullptr on error.
    static Model* from_json(const char* json_file);
    static Model* from_json_text(const std::string& text, std::string* err);
    // model.cpp:147-156.  0 for an unknown stype.
    static size_t get_stype_size(const std::string& stype);
};

class KernelProfile {
public:
    std::vector<int> latency;  // microseconds at occupancy 1, 2, ...
    int total_latency = 0;
    // The same in nanoseconds, from the optional keys "latency_ns" / "total_latency_ns" (kernels on
    // this device run for a few microseconds, so whole microseconds are too coarse to decide what
    // fits beside what; the reference's reader ignores keys it does not look up, model.cpp:57-80).
    // Filled from the microsecond values when the keys are absent.
    std::vector<int> latency_ns;
    int total_latency_ns = 0;
    bool has_ns = false;
};

class ModelProfile {
public:
    int model_latency = 0;
    std::unordered_map<std::string, KernelProfile> kernel_latency;
    std::string to_json() const;                              // model.cpp:123-145
    static ModelProfile* from_json(const char* json_file);    // model.cpp:57-80
    static ModelProfile* from_json_text(const std::string& text, std::string* err);
};

typedef std::unordered_map<std::string, std::vector<float>> ModelParam;

class ModelParamParser {
public:
    // model.cpp:82-121: "TVM_MODEL_PARAMS\0", u64 n, n x {key\0, u64 len, f32[len]}.
    static ModelParam* parse_from_file(const char* param_file);
    // Writer of the same format (script/tvm_generate_model.py:66-76).
    static bool write_to_file(const char* param_file,
                              const std::vector<std::pair<std::string, std::vector<float>>>& params);
};

}  // namespace executor
}  // namespace reef
