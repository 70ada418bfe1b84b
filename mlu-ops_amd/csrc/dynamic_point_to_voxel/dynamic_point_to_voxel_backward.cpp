// mluOpDynamicPointToVoxelBackward and its workspace query: parameter checks with
// the reference's status conventions
// (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_backward/
//  dynamic_point_to_voxel_backward.cpp:33-175), then the backward kernels of
// scatter_points.hip.  The reference also refuses shapes whose working set
// exceeds one core's on-chip memory (5 N + 20 C + 4 bytes, :118-136); there is no
// such limit here.
#include "core/core.h"
#include "core/gen_case.h"
#include "dynamic_point_to_voxel/scatter_points.h"

namespace {

bool archOk(const char *api, mluOpHandle_t handle) {
  if (handle->arch == 950) return true;
  MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported, this handle is on gfx"
                   << handle->arch << ".";
  return false;
}

}  // namespace

mluOpStatus_t MLUOP_WIN_API mluOpGetDynamicPointToVoxelBackwardWorkspaceSize(
    const mluOpHandle_t handle, const mluOpReduceMode_t reduce_type,
    const mluOpTensorDescriptor_t grad_voxel_feats_desc, const mluOpTensorDescriptor_t feats_desc,
    const mluOpTensorDescriptor_t voxel_feats_desc,
    const mluOpTensorDescriptor_t point2voxel_map_desc,
    const mluOpTensorDescriptor_t voxel_points_count_desc,
    const mluOpTensorDescriptor_t voxel_num_desc, size_t *workspace_size) {
  const char *api = "[mluOpGetDynamicPointToVoxelBackwardWorkspaceSize]";
  (void)reduce_type;
  PARAM_CHECK(api, handle != NULL);
  if (!archOk(api, handle)) return MLUOP_STATUS_ARCH_MISMATCH;
  PARAM_CHECK(api, grad_voxel_feats_desc != NULL);
  PARAM_CHECK(api, feats_desc != NULL);
  PARAM_CHECK(api, voxel_feats_desc != NULL);
  PARAM_CHECK(api, point2voxel_map_desc != NULL);
  PARAM_CHECK(api, voxel_points_count_desc != NULL);
  PARAM_CHECK(api, voxel_num_desc != NULL);
  PARAM_CHECK(api, workspace_size != NULL);
  PARAM_CHECK(api, feats_desc->getDim() == 2);
  // N * C ints, the reference's size (:361-363); voxel rows never exceed N
  *workspace_size = (size_t)feats_desc->getDimIndex(0) * feats_desc->getDimIndex(1) * sizeof(int);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpDynamicPointToVoxelBackward(
    const mluOpHandle_t handle, const mluOpReduceMode_t reduce_type,
    const mluOpTensorDescriptor_t grad_voxel_feats_desc, const void *grad_voxel_feats,
    const mluOpTensorDescriptor_t feats_desc, const void *feats,
    const mluOpTensorDescriptor_t voxel_feats_desc, const void *voxel_feats,
    const mluOpTensorDescriptor_t point2voxel_map_desc, const void *point2voxel_map,
    const mluOpTensorDescriptor_t voxel_points_count_desc, const void *voxel_points_count,
    const mluOpTensorDescriptor_t voxel_num_desc, const void *voxel_num, void *workspace,
    const size_t workspace_size, const mluOpTensorDescriptor_t grad_feats_desc,
    void *grad_feats) {
  const char *api = "[mluOpDynamicPointToVoxelBackward]";
  PARAM_CHECK(api, handle != NULL);
  if (!archOk(api, handle)) return MLUOP_STATUS_ARCH_MISMATCH;
  PARAM_CHECK(api, grad_voxel_feats_desc != NULL);
  PARAM_CHECK(api, feats_desc != NULL);
  PARAM_CHECK(api, voxel_feats_desc != NULL);
  PARAM_CHECK(api, point2voxel_map_desc != NULL);
  PARAM_CHECK(api, voxel_points_count_desc != NULL);
  PARAM_CHECK(api, voxel_num_desc != NULL);
  PARAM_CHECK(api, grad_feats_desc != NULL);
  STRIDE_TENSOR_CHECK(api, grad_voxel_feats_desc, "grad_voxel_feats_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, feats_desc, "feats_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, voxel_feats_desc, "voxel_feats_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, point2voxel_map_desc, "point2voxel_map_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, voxel_points_count_desc, "voxel_points_count_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, voxel_num_desc, "voxel_num_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, grad_feats_desc, "grad_feats_desc must be contiguous");
  PARAM_CHECK(api, grad_voxel_feats_desc->getDtype() == MLUOP_DTYPE_FLOAT);
  PARAM_CHECK(api, feats_desc->getDtype() == MLUOP_DTYPE_FLOAT);
  PARAM_CHECK(api, voxel_feats_desc->getDtype() == MLUOP_DTYPE_FLOAT);
  PARAM_CHECK(api, grad_feats_desc->getDtype() == MLUOP_DTYPE_FLOAT);
  PARAM_CHECK(api, point2voxel_map_desc->getDtype() == MLUOP_DTYPE_INT32);
  PARAM_CHECK(api, voxel_points_count_desc->getDtype() == MLUOP_DTYPE_INT32);
  PARAM_CHECK(api, voxel_num_desc->getDtype() == MLUOP_DTYPE_INT32);
  PARAM_CHECK(api, grad_voxel_feats_desc->getDim() == 2);
  PARAM_CHECK(api, feats_desc->getDim() == 2);
  PARAM_CHECK(api, voxel_feats_desc->getDim() == 2);
  PARAM_CHECK(api, point2voxel_map_desc->getDim() == 1);
  PARAM_CHECK(api, voxel_points_count_desc->getDim() == 1);
  PARAM_CHECK(api, voxel_num_desc->getDim() == 1);
  PARAM_CHECK(api, grad_feats_desc->getDim() == 2);
  PARAM_CHECK(api, feats_desc->getDimIndex(1) == grad_voxel_feats_desc->getDimIndex(1));
  PARAM_CHECK(api, voxel_feats_desc->getDimIndex(0) == grad_voxel_feats_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_feats_desc->getDimIndex(1) == grad_voxel_feats_desc->getDimIndex(1));
  PARAM_CHECK(api, point2voxel_map_desc->getDimIndex(0) == feats_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_points_count_desc->getDimIndex(0) == grad_voxel_feats_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_num_desc->getDimIndex(0) == 1);
  PARAM_CHECK(api, grad_feats_desc->getDimIndex(0) == feats_desc->getDimIndex(0));
  PARAM_CHECK(api, grad_feats_desc->getDimIndex(1) == grad_voxel_feats_desc->getDimIndex(1));
  PARAM_CHECK(api, feats_desc->getDimIndex(0) >= grad_voxel_feats_desc->getDimIndex(0));
  if (reduce_type != MLUOP_REDUCE_DMAX) {
    MLUOP_LOG(ERROR) << api << " only supports max reduce in current version. ";
    return MLUOP_STATUS_BAD_PARAM;
  }
  const uint64_t grad_voxel_num = mluOpGetTensorElementNum(grad_voxel_feats_desc);
  const uint64_t feats_num = mluOpGetTensorElementNum(feats_desc);
  TENSOR_NUM_CHECK(api, grad_voxel_num, LARGE_TENSOR_NUM, "");
  TENSOR_NUM_CHECK(api, feats_num, LARGE_TENSOR_NUM, "");
  if (mluOpGetTensorElementNum(grad_feats_desc) == 0) return MLUOP_STATUS_SUCCESS;
  if (grad_voxel_num != 0) {
    PARAM_CHECK(api, grad_voxel_feats != NULL);
  }
  PARAM_CHECK(api, feats != NULL);
  if (mluOpGetTensorElementNum(voxel_feats_desc) != 0) {
    PARAM_CHECK(api, voxel_feats != NULL);
  }
  PARAM_CHECK(api, point2voxel_map != NULL);
  if (mluOpGetTensorElementNum(voxel_points_count_desc) != 0) {
    PARAM_CHECK(api, voxel_points_count != NULL);
  }
  PARAM_CHECK(api, voxel_num != NULL);
  PARAM_CHECK(api, grad_feats != NULL);
  if (workspace_size != 0) {
    PARAM_CHECK(api, workspace != NULL);
  }
  if (mluop::gen_case::mode() != 0) {
    // (reference kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_backward/
    // dynamic_point_to_voxel_backward.cpp:254-270)
    mluop::gen_case::CaseWriter c(handle, "dynamic_point_to_voxel_backward", "dynamic_point_to_voxel_backward_param");
    c.input("grad_voxel_feats", grad_voxel_feats_desc, grad_voxel_feats);
    c.input("feats", feats_desc, feats);
    c.input("voxel_feats", voxel_feats_desc, voxel_feats);
    c.input("point2voxel_map", point2voxel_map_desc, point2voxel_map);
    c.input("voxel_points_count", voxel_points_count_desc, voxel_points_count);
    c.input("voxel_num", voxel_num_desc, voxel_num);
    c.output("grad_feats", grad_feats_desc);
    c.paramName("reduce_type", reduce_type == MLUOP_REDUCE_DMAX ? "REDUCE_MODE_MAX" : "REDUCE_MODE_MEAN");
    c.finish(0.003);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  HIP_CHECK_RETURN(api, hipSetDevice(handle->device));

  const int n = (int)feats_desc->getDimIndex(0);
  const int c = (int)feats_desc->getDimIndex(1);
  const int rows = (int)grad_voxel_feats_desc->getDimIndex(0);
  const size_t need = (size_t)rows * c * sizeof(int);
  PARAM_CHECK_V2(api, workspace_size >= need,
                 "workspace_size " << workspace_size << " is below the " << need << " bytes needed.");
  if (need > 0) {
    PARAM_CHECK(api, workspace != NULL);
  }
  HIP_CHECK_RETURN(api, mluop::dynamic_point_to_voxel::launchScatterPointsBackward(
                            handle->launchCtx(), n, c, rows,
                            static_cast<const float *>(grad_voxel_feats),
                            static_cast<const float *>(feats),
                            static_cast<const float *>(voxel_feats),
                            static_cast<const int32_t *>(point2voxel_map),
                            static_cast<const int32_t *>(voxel_num),
                            static_cast<int32_t *>(workspace), static_cast<float *>(grad_feats)));
  return MLUOP_STATUS_SUCCESS;
}
