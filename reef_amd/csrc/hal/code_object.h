// Reads per-kernel resource usage out of an AMDGPU code object (optionally
// wrapped in a clang offload bundle): the NT_AMDGPU_METADATA note holds a
// MessagePack map whose "amdhsa.kernels" list carries .name, .vgpr_count,
// .agpr_count, .sgpr_count, .group_segment_fixed_size,
// .private_segment_fixed_size and .kernarg_segment_size for every kernel.
// This replaces the reference's hipFuncGetWGInfo, a call that exists only in
// its patched runtime (src/reef/executor/hip/hip_impl.cpp:34-42).
// Pure host code: works without a GPU.
#pragma once
#include <cstdint>
#include <map>
#include <string>

namespace reef {
namespace hal {

struct KernelMeta {
    int vgprs = 0;    // unified register count: arch VGPRs (rounded to 4) + AGPRs
    int agprs = 0;    // accumulation VGPRs, included in vgprs
    int sgprs = 0;
    int lds = 0;      // static group segment bytes
    int scratch = 0;  // private segment bytes per lane
    int kernarg = 0;  // kernarg segment bytes
    int max_threads = 0;
};

// name -> metadata.  Returns false and fills err when the file cannot be parsed.
bool read_code_object_metadata(const char* path, std::map<std::string, KernelMeta>* out,
                               std::string* err);

}  // namespace hal
}  // namespace reef
