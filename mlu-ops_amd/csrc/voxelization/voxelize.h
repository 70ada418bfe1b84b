// Host-side interface of the hard-voxelization kernel set.
#ifndef MLUOP_AMD_VOXELIZATION_VOXELIZE_H_
#define MLUOP_AMD_VOXELIZATION_VOXELIZE_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "core/launch.h"

namespace mluop {
namespace voxelization {

struct VoxelizeShape {
  int64_t num_points;
  int num_features;
  int max_points;
  int max_voxels;
};

// Most points one call accepts (the hash table has twice as many slots and is
// indexed with 32 bits).
constexpr int64_t kMaxPoints = (int64_t)1 << 28;

// Bytes of device workspace: the per-point arrays and the cell table, plus
// `library_bytes` for the sort and the scan (from libraryWorkspaceBytes).
size_t voxelizeWorkspaceBytes(const VoxelizeShape &s, size_t library_bytes);

// Counters the sort and the scan want at this size.
hipError_t libraryWorkspaceBytes(const VoxelizeShape &s, hipStream_t stream, size_t *bytes);

// Enqueues the whole operator: outputs zero-filled, then written.
hipError_t launchVoxelize(const LaunchCtx &lc, const VoxelizeShape &s, const float *points,
                          const float *voxel_size, const float *coors_range, void *workspace,
                          size_t workspace_bytes, float *voxels, int32_t *coors,
                          int32_t *num_points_per_voxel, int32_t *voxel_num);

}  // namespace voxelization
}  // namespace mluop

#endif  // MLUOP_AMD_VOXELIZATION_VOXELIZE_H_
