// mluOpDynamicPointToVoxelForward and its workspace query: parameter checks with
// the reference's status conventions
// (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_forward/
//  dynamic_point_to_voxel_forward.cpp:72-193), then the kernel set of
// scatter_points.hip.
#include <string>

#include "core/core.h"
#include "core/gen_case.h"
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

  // The seven tensors in argument order, with the rank and element type each must have;
  // the checks run in the reference's order: all descriptors, all ranks, all strides, all types.
  struct Expect {
    const mluOpTensorDescriptor_t desc;
    const char *name;
    int rank;
    mluOpDataType_t dtype;
  };
  const Expect tensors[] = {
      {feats_desc, "feats", 2, MLUOP_DTYPE_FLOAT},
      {coors_desc, "coors", 2, MLUOP_DTYPE_INT32},
      {voxel_feats_desc, "voxel_feats", 2, MLUOP_DTYPE_FLOAT},
      {voxel_coors_desc, "voxel_coors", 2, MLUOP_DTYPE_INT32},
      {point2voxel_map_desc, "point2voxel_map", 1, MLUOP_DTYPE_INT32},
      {voxel_points_count_desc, "voxel_points_count", 1, MLUOP_DTYPE_INT32},
      {voxel_num_desc, "voxel_num", 1, MLUOP_DTYPE_INT32},
  };
  for (const Expect &t : tensors)
    PARAM_CHECK_V2(api, t.desc != NULL, "descriptor of " << t.name << " is NULL.");
  for (const Expect &t : tensors)
    PARAM_CHECK_V2(api, t.desc->getDim() == t.rank, t.name << " must have " << t.rank << " dimensions.");
  for (const Expect &t : tensors)
    STRIDE_TENSOR_CHECK(api + ":", t.desc, t.name << " must be contiguous");
  for (const Expect &t : tensors)
    PARAM_CHECK_V2(api, t.desc->getDtype() == t.dtype,
                   t.name << " must be " << mluop::getNameOfDataType(t.dtype) << ", but is "
                          << mluop::getNameOfDataType(t.desc->getDtype()) << ".");
  if (reduce_type != MLUOP_REDUCE_DMAX && reduce_type != MLUOP_REDUCE_DMEAN) {
    MLUOP_LOG(ERROR) << api << " reduce_type must be max or mean.";
    return MLUOP_STATUS_BAD_PARAM;
  }

  // N points, M voxel rows, C features, three coordinates
  const int64_t n = feats_desc->getDimIndex(0), c = feats_desc->getDimIndex(1);
  const int64_t m = voxel_feats_desc->getDimIndex(0);
  PARAM_CHECK(api, coors_desc->getDimIndex(0) == n && point2voxel_map_desc->getDimIndex(0) == n);
  PARAM_CHECK(api, voxel_coors_desc->getDimIndex(0) == m && voxel_points_count_desc->getDimIndex(0) == m);
  PARAM_CHECK(api, voxel_num_desc->getDimIndex(0) == 1);
  PARAM_CHECK(api, voxel_feats_desc->getDimIndex(1) == c);
  PARAM_CHECK(api, coors_desc->getDimIndex(1) == 3 && voxel_coors_desc->getDimIndex(1) == 3);
  PARAM_CHECK(api, n >= m);

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
  const void *const data[] = {feats, coors, voxel_feats, voxel_coors, point2voxel_map, voxel_points_count,
                              voxel_num};
  for (size_t i = 0; i < sizeof(data) / sizeof(data[0]); ++i)
    PARAM_CHECK_V2(api, data[i] != NULL, tensors[i].name << " is NULL.");
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
  if (mluop::gen_case::mode() != 0) {
    // (reference kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_forward/
    // dynamic_point_to_voxel_forward.cpp:264-279)
    mluop::gen_case::CaseWriter c(handle, "dynamic_point_to_voxel_forward", "dynamic_point_to_voxel_forward_param");
    c.input("feats", feats_desc, feats);
    c.input("coors", coors_desc, coors);
    c.output("voxel_feats", voxel_feats_desc);
    c.output("voxel_coors", voxel_coors_desc);
    c.output("point2voxel_map", point2voxel_map_desc);
    c.output("voxel_points_count", voxel_points_count_desc);
    c.output("voxel_num", voxel_num_desc);
    c.paramName("reduce_type", reduce_type == MLUOP_REDUCE_DMAX ? "REDUCE_MODE_MAX" : "REDUCE_MODE_MEAN");
    c.finish(0.003);
  }
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
