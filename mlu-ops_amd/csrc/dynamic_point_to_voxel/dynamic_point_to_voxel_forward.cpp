// mluOpDynamicPointToVoxelForward and its workspace query: parameter checks with
// the reference's status conventions
// (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_forward/
//  dynamic_point_to_voxel_forward.cpp:72-193), then the kernel set of
// scatter_points.hip.
#include <string>

#include "core/core.h"
#include "dynamic_point_to_voxel/scatter_points.h"

namespace {

using mluop::dynamic_point_to_voxel::ScatterShape;

bool archOk(const std::string &api, mluOpHandle_t handle) {
  if (handle->arch == 950) return true;
  MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported, this handle is on gfx"
                   << handle->arch << ".";
  return false;
}

mluOpStatus_t paramCheck(const std::string &api, const mluOpHandle_t handle,
                         const mluOpReduceMode_t reduce_type, const void *feats, const void *coors,
                         const void *voxel_feats, const void *voxel_coors,
                         const void *point2voxel_map, const void *voxel_points_count,
                         const void *voxel_num, void *workspace, const size_t workspace_size,
                         const mluOpTensorDescriptor_t feats_desc,
                         const mluOpTensorDescriptor_t coors_desc,
                         const mluOpTensorDescriptor_t voxel_feats_desc,
                         const mluOpTensorDescriptor_t voxel_coors_desc,
                         const mluOpTensorDescriptor_t point2voxel_map_desc,
                         const mluOpTensorDescriptor_t voxel_points_count_desc,
                         const mluOpTensorDescriptor_t voxel_num_desc, bool *zero_element) {
  PARAM_CHECK(api, handle != NULL);
  if (!archOk(api, handle)) return MLUOP_STATUS_ARCH_MISMATCH;
  PARAM_CHECK(api, feats_desc != NULL);
  PARAM_CHECK(api, coors_desc != NULL);
  PARAM_CHECK(api, voxel_feats_desc != NULL);
  PARAM_CHECK(api, voxel_coors_desc != NULL);
  PARAM_CHECK(api, point2voxel_map_desc != NULL);
  PARAM_CHECK(api, voxel_points_count_desc != NULL);
  PARAM_CHECK(api, voxel_num_desc != NULL);
  PARAM_CHECK(api, feats_desc->getDim() == 2);
  PARAM_CHECK(api, coors_desc->getDim() == 2);
  PARAM_CHECK(api, voxel_feats_desc->getDim() == 2);
  PARAM_CHECK(api, voxel_coors_desc->getDim() == 2);
  PARAM_CHECK(api, point2voxel_map_desc->getDim() == 1);
  PARAM_CHECK(api, voxel_points_count_desc->getDim() == 1);
  PARAM_CHECK(api, voxel_num_desc->getDim() == 1);
  STRIDE_TENSOR_CHECK(api + ":", feats_desc, "feats_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", coors_desc, "coors_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", voxel_feats_desc, "voxel_feats_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", voxel_coors_desc, "voxel_coors_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", point2voxel_map_desc, "point2voxel_map_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", voxel_points_count_desc,
                      "voxel_points_count_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api + ":", voxel_num_desc, "voxel_num_desc must be contiguous");
  PARAM_CHECK_V2(api, (feats_desc->getDtype() == MLUOP_DTYPE_FLOAT),
                 "Only float are supported in feats tensor, but the data type of tensor is "
                     << mluop::getNameOfDataType(feats_desc->getDtype()) << ".");
  PARAM_CHECK_V2(api, (coors_desc->getDtype() == MLUOP_DTYPE_INT32),
                 "Only int32 are supported in coors tensor, but the data type of tensor is "
                     << mluop::getNameOfDataType(coors_desc->getDtype()) << ".");
  PARAM_CHECK_V2(api, (point2voxel_map_desc->getDtype() == MLUOP_DTYPE_INT32),
                 "Only int32 are supported in point2voxel_map tensor, but the data type of tensor is "
                     << mluop::getNameOfDataType(point2voxel_map_desc->getDtype()) << ".");
  PARAM_CHECK(api, voxel_feats_desc->getDtype() == feats_desc->getDtype());
  PARAM_CHECK(api, voxel_coors_desc->getDtype() == coors_desc->getDtype());
  PARAM_CHECK(api, voxel_points_count_desc->getDtype() == point2voxel_map_desc->getDtype());
  PARAM_CHECK(api, voxel_num_desc->getDtype() == point2voxel_map_desc->getDtype());
  if (reduce_type != MLUOP_REDUCE_DMAX && reduce_type != MLUOP_REDUCE_DMEAN) {
    MLUOP_LOG(ERROR) << api << " Only support max and mean. Please check reduce_type!";
    return MLUOP_STATUS_BAD_PARAM;
  }
  PARAM_CHECK(api, feats_desc->getDimIndex(0) == coors_desc->getDimIndex(0));
  PARAM_CHECK(api, feats_desc->getDimIndex(0) == point2voxel_map_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_feats_desc->getDimIndex(0) == voxel_coors_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_feats_desc->getDimIndex(0) == voxel_points_count_desc->getDimIndex(0));
  PARAM_CHECK(api, voxel_num_desc->getDimIndex(0) == 1);
  PARAM_CHECK(api, feats_desc->getDimIndex(1) == voxel_feats_desc->getDimIndex(1));
  PARAM_CHECK(api, coors_desc->getDimIndex(1) == voxel_coors_desc->getDimIndex(1));
  PARAM_CHECK(api, coors_desc->getDimIndex(1) == 3);
  PARAM_CHECK(api, feats_desc->getDimIndex(0) >= voxel_feats_desc->getDimIndex(0));

  const size_t feats_element_num = mluOpGetTensorElementNum(feats_desc);
  const size_t coors_element_num = mluOpGetTensorElementNum(coors_desc);
  TENSOR_NUM_CHECK(api, feats_element_num, LARGE_TENSOR_NUM, "");
  TENSOR_NUM_CHECK(api, coors_element_num, LARGE_TENSOR_NUM, "");
  if (feats_element_num == 0 || coors_element_num == 0) {
    *zero_element = true;
    return MLUOP_STATUS_SUCCESS;
  }
  if (workspace_size > 0) {
    PARAM_CHECK(api, workspace != NULL);
  }
  PARAM_CHECK(api, feats != NULL);
  PARAM_CHECK(api, coors != NULL);
  PARAM_CHECK(api, voxel_feats != NULL);
  PARAM_CHECK(api, voxel_coors != NULL);
  PARAM_CHECK(api, point2voxel_map != NULL);
  PARAM_CHECK(api, voxel_points_count != NULL);
  PARAM_CHECK(api, voxel_num != NULL);
  return MLUOP_STATUS_SUCCESS;
}

}  // namespace

mluOpStatus_t MLUOP_WIN_API mluOpGetDynamicPointToVoxelForwardWorkspaceSize(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t feats_desc,
    const mluOpTensorDescriptor_t coors_desc, size_t *workspace_size) {
  const std::string api = "[mluOpGetDynamicPointToVoxelForwardWorkspaceSize]";
  PARAM_CHECK(api, handle != NULL);
  if (!archOk(api, handle)) return MLUOP_STATUS_ARCH_MISMATCH;
  PARAM_CHECK(api, feats_desc != NULL);
  PARAM_CHECK(api, coors_desc != NULL);
  PARAM_CHECK(api, workspace_size != NULL);
  PARAM_CHECK(api, coors_desc->getDim() == 2);
  ScatterShape s{};
  s.num_points = (int)coors_desc->getDimIndex(0);
  size_t library_bytes = 0;
  if (handle->device >= 0 && s.num_points > 0) {
    HIP_CHECK_RETURN(api, hipSetDevice(handle->device));
    HIP_CHECK_RETURN(api, mluop::dynamic_point_to_voxel::libraryWorkspaceBytes(s, handle->queue,
                                                                               &library_bytes));
  }
  *workspace_size = mluop::dynamic_point_to_voxel::scatterWorkspaceBytes(s, library_bytes);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpDynamicPointToVoxelForward(
    const mluOpHandle_t handle, const mluOpReduceMode_t reduce_type,
    const mluOpTensorDescriptor_t feats_desc, const void *feats,
    const mluOpTensorDescriptor_t coors_desc, void *coors, void *workspace,
    const size_t workspace_size, const mluOpTensorDescriptor_t voxel_feats_desc,
    void *voxel_feats, const mluOpTensorDescriptor_t voxel_coors_desc, void *voxel_coors,
    const mluOpTensorDescriptor_t point2voxel_map_desc, void *point2voxel_map,
    const mluOpTensorDescriptor_t voxel_points_count_desc, void *voxel_points_count,
    const mluOpTensorDescriptor_t voxel_num_desc, void *voxel_num) {
  const std::string api = "[mluOpDynamicPointToVoxelForward]";
  bool zero_element = false;
  mluOpStatus_t ret = paramCheck(api, handle, reduce_type, feats, coors, voxel_feats, voxel_coors,
                                 point2voxel_map, voxel_points_count, voxel_num, workspace,
                                 workspace_size, feats_desc, coors_desc, voxel_feats_desc,
                                 voxel_coors_desc, point2voxel_map_desc, voxel_points_count_desc,
                                 voxel_num_desc, &zero_element);
  if (ret != MLUOP_STATUS_SUCCESS) {
    MLUOP_LOG(ERROR) << api << " Error found during element verification, please check.";
    return ret;
  }
  if (zero_element) return MLUOP_STATUS_SUCCESS;
  DEVICE_HANDLE_CHECK(api, handle);
  HIP_CHECK_RETURN(api, hipSetDevice(handle->device));

  ScatterShape s;
  s.num_points = (int)feats_desc->getDimIndex(0);
  s.num_features = (int)feats_desc->getDimIndex(1);
  s.voxel_rows = (int)voxel_feats_desc->getDimIndex(0);
  s.reduce_max = reduce_type == MLUOP_REDUCE_DMAX;
  size_t library_bytes = 0;
  HIP_CHECK_RETURN(api, mluop::dynamic_point_to_voxel::libraryWorkspaceBytes(s, handle->queue,
                                                                             &library_bytes));
  const size_t need = mluop::dynamic_point_to_voxel::scatterWorkspaceBytes(s, library_bytes);
  PARAM_CHECK_V2(api, workspace_size >= need,
                 "workspace_size " << workspace_size << " is below the " << need
                                   << " bytes mluOpGetDynamicPointToVoxelForwardWorkspaceSize reports.");
  PARAM_CHECK(api, workspace != NULL);
  PARAM_CHECK(api, handle->pinned_scalar != NULL);

  HIP_CHECK_RETURN(api, mluop::dynamic_point_to_voxel::launchScatterPoints(
                            handle->launchCtx(), s, static_cast<const float *>(feats),
                            static_cast<int32_t *>(coors), workspace, workspace_size,
                            handle->pinned_scalar, static_cast<float *>(voxel_feats),
                            static_cast<int32_t *>(voxel_coors),
                            static_cast<int32_t *>(point2voxel_map),
                            static_cast<int32_t *>(voxel_points_count),
                            static_cast<int32_t *>(voxel_num)));
  return MLUOP_STATUS_SUCCESS;
}
