// Host-side interface of the dynamic point-to-voxel (forward) kernel set.
#ifndef MLUOP_AMD_DYNAMIC_POINT_TO_VOXEL_SCATTER_POINTS_H_
#define MLUOP_AMD_DYNAMIC_POINT_TO_VOXEL_SCATTER_POINTS_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "core/launch.h"

namespace mluop {
namespace dynamic_point_to_voxel {

struct ScatterShape {
  int num_points;    // N
  int num_features;  // C
  int voxel_rows;    // rows of the voxel_* output tensors (<= N)
  bool reduce_max;   // max, else mean
};

// Per-point arrays only; the sort's counters come on top (libraryWorkspaceBytes).
size_t scatterWorkspaceBytes(const ScatterShape &s, size_t library_bytes);
hipError_t libraryWorkspaceBytes(const ScatterShape &s, hipStream_t stream, size_t *bytes);

// Enqueues the operator.  It synchronises the stream once to read the largest
// coordinate of every axis back into `pinned_host` (three ints of pinned host
// memory), which sizes the radix sorts.
hipError_t launchScatterPoints(const LaunchCtx &lc, const ScatterShape &s, const float *feats,
                               int32_t *coors, void *workspace, size_t workspace_bytes,
                               int32_t *pinned_host, float *voxel_feats, int32_t *voxel_coors,
                               int32_t *point2voxel_map, int32_t *voxel_points_count,
                               int32_t *voxel_num);

// Backward of the max reduction: `from` is [voxel_rows, num_features] ints of workspace.
hipError_t launchScatterPointsBackward(const LaunchCtx &lc, int num_points, int num_features,
                                       int voxel_rows, const float *grad_voxel_feats,
                                       const float *feats, const float *voxel_feats,
                                       const int32_t *point2voxel_map, const int32_t *voxel_num,
                                       int32_t *from, float *grad_feats);

}  // namespace dynamic_point_to_voxel
}  // namespace mluop

#endif  // MLUOP_AMD_DYNAMIC_POINT_TO_VOXEL_SCATTER_POINTS_H_
