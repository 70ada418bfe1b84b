// Row maps kept across calls (mluOpExtBuildRowMap / mluOpExtUseRowMap): the operator side.
#ifndef MLUOP_AMD_SPARSE_CONV_ROW_MAP_H_
#define MLUOP_AMD_SPARSE_CONV_ROW_MAP_H_

#include <string>

#include "core/core.h"
#include "sparse_conv/indice_conv.h"

namespace mluop {
namespace sparse_conv {

// Checks that the announced map (may be null: nothing to do) was built from this pair tensor
// for this direction and shape (BAD_PARAM otherwise) and hands it to the launch.
mluOpStatus_t takeRowMap(const std::string &api, mluOpHandle_t handle, const void *announced,
                         GatherDirection dir, ConvProblem *p);

// The map announced for the next call; the announcement ends here whatever the call does.
inline const void *announcedRowMap(mluOpHandle_t handle) {
  if (handle == nullptr) return nullptr;
  const void *map = handle->pending_row_map;
  handle->pending_row_map = nullptr;
  return map;
}

}  // namespace sparse_conv
}  // namespace mluop

#endif  // MLUOP_AMD_SPARSE_CONV_ROW_MAP_H_
