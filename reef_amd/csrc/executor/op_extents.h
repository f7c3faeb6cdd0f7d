// What a kernel of the graph file touches, worked out on the host from its shape attributes
// before anything is launched: the bytes each operand needs behind its pointer and the number
// of workgroups the launch must have.  The kernels are shape-generic and trust their
// attributes, and all storages of a model share one allocation, so an attribute that does not
// fit its storages would read or write a neighbouring tensor (or fault past the end of the
// allocation).  The reference has no such check: its generated kernels have their shapes
// compiled in (resource/resnet152/resnet152.cu:315-338) and the graph file only names them.
#pragma once
#include <string>

#include "executor/model.h"

namespace reef {
namespace executor {

// REEF_OP_* of an entry symbol (the part of a kernel name before '#'), REEF_OP_NONE if the
// symbol is not one of this library's.
int op_from_symbol(const std::string& symbol);

// True when kernel `index` of `m` fits its storages and its grid.  On false `why` says which
// kernel, which operand and by how much.  Kernels whose symbol is not one of this library's
// (another code object's) are not judged.
bool kernel_fits_storages(const Model& m, size_t index, std::string* why);

}  // namespace executor
}  // namespace reef
