// mluOpVoxelization and its workspace query: parameter checks with the
// reference's status conventions (kernels/voxelization/voxelization.cpp:55-172),
// then the kernel set of voxelize.hip.
#include "core/core.h"
#include "core/gen_case.h"
#include "voxelization/voxelize.h"

namespace {

using mluop::voxelization::VoxelizeShape;

mluOpStatus_t voxelizationParamCheck(const char *api, const mluOpHandle_t handle,
                                     const mluOpTensorDescriptor_t points_desc,
                                     const mluOpTensorDescriptor_t voxel_size_desc,
                                     const mluOpTensorDescriptor_t coors_range_desc,
                                     const int32_t max_points, const int32_t max_voxels,
                                     const int32_t NDim, const bool deterministic,
                                     const mluOpTensorDescriptor_t voxels_desc,
                                     const mluOpTensorDescriptor_t coors_desc,
                                     const mluOpTensorDescriptor_t num_points_per_voxel_desc,
                                     const mluOpTensorDescriptor_t voxel_num_desc,
                                     bool *is_zero_element) {
  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported, this handle is on gfx"
                     << handle->arch << ".";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }
  if (!deterministic) {
    // the reference has no non-deterministic mode either (voxelization.cpp:166-170)
    MLUOP_LOG(ERROR) << api << " Non-deterministic mode is not supported.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  // points [N, F]; voxel_size [3]; coors_range [6]; voxels [max_voxels, max_points, F];
  // coors [max_voxels, 3]; num_points_per_voxel [max_voxels]; voxel_num [1].
  // -1 in `dims` = "whatever the tensor says" (N and F come from points).
  struct Expect {
    const mluOpTensorDescriptor_t desc;
    const char *name;
    int rank;
    int64_t dims[3];
    mluOpDataType_t dtype;
  };
  const int64_t features = points_desc->getDim() == 2 ? points_desc->getDimIndex(1) : -1;
  const Expect tensors[] = {
      {points_desc, "points", 2, {-1, -1, 0}, MLUOP_DTYPE_FLOAT},
      {voxel_size_desc, "voxel_size", 1, {3, 0, 0}, MLUOP_DTYPE_FLOAT},
      {coors_range_desc, "coors_range", 1, {6, 0, 0}, MLUOP_DTYPE_FLOAT},
      {voxels_desc, "voxels", 3, {max_voxels, max_points, features}, MLUOP_DTYPE_FLOAT},
      {coors_desc, "coors", 2, {max_voxels, 3, 0}, MLUOP_DTYPE_INT32},
      {num_points_per_voxel_desc, "num_points_per_voxel", 1, {max_voxels, 0, 0}, MLUOP_DTYPE_INT32},
      {voxel_num_desc, "voxel_num", 1, {1, 0, 0}, MLUOP_DTYPE_INT32},
  };
  for (const Expect &t : tensors) {
    PARAM_CHECK_V2(api, t.desc->getDim() == t.rank, t.name << " must have " << t.rank << " dimensions.");
    for (int a = 0; a < t.rank; ++a)
      PARAM_CHECK_V2(api, t.dims[a] < 0 || t.desc->getDimIndex(a) == t.dims[a],
                     "dimension " << a << " of " << t.name << " must be " << t.dims[a] << ".");
  }
  PARAM_CHECK_EQ(api, NDim, 3);
  for (const Expect &t : tensors) STRIDE_TENSOR_CHECK(api, t.desc, t.name << " must be contiguous");
  for (const Expect &t : tensors)
    PARAM_CHECK_V2(api, t.desc->getDtype() == t.dtype,
                   t.name << " must be " << mluop::getNameOfDataType(t.dtype) << ".");

  const uint64_t points_num = mluOpGetTensorElementNum(points_desc);
  const uint64_t voxel_size_num = mluOpGetTensorElementNum(voxel_size_desc);
  const uint64_t coors_range_num = mluOpGetTensorElementNum(coors_range_desc);
  if (points_num >= LARGE_TENSOR_NUM || voxel_size_num >= LARGE_TENSOR_NUM ||
      coors_range_num >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(coors_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(num_points_per_voxel_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(voxel_num_desc) >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " Overflow max tensor num."
                     << " Tensors of fewer than 2^31 elements are supported.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  if (points_desc->getDimIndex(0) > mluop::voxelization::kMaxPoints) {
    MLUOP_LOG(ERROR) << api << " At most " << mluop::voxelization::kMaxPoints
                     << " points per call are supported.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  // the voxels tensor is indexed with size_t on the device; its byte size must still be sane
  if (mluOpGetTensorElementNum(voxels_desc) >= ((uint64_t)1 << 40)) {
    MLUOP_LOG(ERROR) << api << " voxels tensor too large.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  *is_zero_element = false;
  if (points_num == 0 || voxel_size_num == 0 || coors_range_num == 0) {
    MLUOP_LOG(ERROR) << api << " Check failed: Input zero element tensor.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (max_points == 0 || max_voxels == 0) *is_zero_element = true;
  return MLUOP_STATUS_SUCCESS;
}

VoxelizeShape shapeOf(const mluOpTensorDescriptor_t points_desc, int32_t max_points,
                      int32_t max_voxels) {
  VoxelizeShape s;
  s.num_points = points_desc->getDimIndex(0);
  s.num_features = (int)points_desc->getDimIndex(1);
  s.max_points = max_points;
  s.max_voxels = max_voxels;
  return s;
}

}  // namespace

mluOpStatus_t MLUOP_WIN_API mluOpGetVoxelizationWorkspaceSize(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t points_desc,
    const mluOpTensorDescriptor_t voxel_size_desc, const mluOpTensorDescriptor_t coors_range_desc,
    const int32_t max_points, const int32_t max_voxels, const int32_t NDim,
    const bool deterministic, const mluOpTensorDescriptor_t voxels_desc,
    const mluOpTensorDescriptor_t coors_desc,
    const mluOpTensorDescriptor_t num_points_per_voxel_desc,
    const mluOpTensorDescriptor_t voxel_num_desc, size_t *size) {
  const char *api = "[mluOpGetVoxelizationWorkspaceSize]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, points_desc != NULL);
  PARAM_CHECK(api, voxel_size_desc != NULL);
  PARAM_CHECK(api, coors_range_desc != NULL);
  PARAM_CHECK(api, voxels_desc != NULL);
  PARAM_CHECK(api, coors_desc != NULL);
  PARAM_CHECK(api, num_points_per_voxel_desc != NULL);
  PARAM_CHECK(api, voxel_num_desc != NULL);
  PARAM_CHECK(api, size != NULL);

  bool is_zero_element = false;
  mluOpStatus_t status = voxelizationParamCheck(
      "[mluOpVoxelization]", handle, points_desc, voxel_size_desc, coors_range_desc, max_points,
      max_voxels, NDim, deterministic, voxels_desc, coors_desc, num_points_per_voxel_desc,
      voxel_num_desc, &is_zero_element);
  if (status != MLUOP_STATUS_SUCCESS) return status;
  if (is_zero_element) return MLUOP_STATUS_SUCCESS;  // *size untouched, as in the reference

  const VoxelizeShape s = shapeOf(points_desc, max_points, max_voxels);
  size_t library_bytes = 0;
  if (handle->device >= 0) {
    HIP_CHECK_RETURN(api, hipSetDevice(handle->device));
    HIP_CHECK_RETURN(api,
                     mluop::voxelization::libraryWorkspaceBytes(s, handle->queue, &library_bytes));
  }
  *size = mluop::voxelization::voxelizeWorkspaceBytes(s, library_bytes);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpVoxelization(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t points_desc, const void *points,
    const mluOpTensorDescriptor_t voxel_size_desc, const void *voxel_size,
    const mluOpTensorDescriptor_t coors_range_desc, const void *coors_range,
    const int32_t max_points, const int32_t max_voxels, const int32_t NDim,
    const bool deterministic, void *workspace, size_t workspace_size,
    const mluOpTensorDescriptor_t voxels_desc, void *voxels,
    const mluOpTensorDescriptor_t coors_desc, void *coors,
    const mluOpTensorDescriptor_t num_points_per_voxel_desc, void *num_points_per_voxel,
    const mluOpTensorDescriptor_t voxel_num_desc, void *voxel_num) {
  const char *api = "[mluOpVoxelization]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, points_desc != NULL);
  PARAM_CHECK(api, voxel_size_desc != NULL);
  PARAM_CHECK(api, coors_range_desc != NULL);
  PARAM_CHECK(api, voxels_desc != NULL);
  PARAM_CHECK(api, coors_desc != NULL);
  PARAM_CHECK(api, num_points_per_voxel_desc != NULL);
  PARAM_CHECK(api, voxel_num_desc != NULL);

  bool is_zero_element = false;
  mluOpStatus_t status = voxelizationParamCheck(
      api, handle, points_desc, voxel_size_desc, coors_range_desc, max_points, max_voxels, NDim,
      deterministic, voxels_desc, coors_desc, num_points_per_voxel_desc, voxel_num_desc,
      &is_zero_element);
  if (status != MLUOP_STATUS_SUCCESS) return status;
  if (workspace_size > 0) {
    PARAM_CHECK(api, workspace != NULL);
  }
  if (is_zero_element) return MLUOP_STATUS_SUCCESS;

  PARAM_CHECK(api, points != NULL);
  PARAM_CHECK(api, voxel_size != NULL);
  PARAM_CHECK(api, coors_range != NULL);
  PARAM_CHECK(api, voxels != NULL);
  PARAM_CHECK(api, coors != NULL);
  PARAM_CHECK(api, num_points_per_voxel != NULL);
  PARAM_CHECK(api, voxel_num != NULL);
  if (mluop::gen_case::mode() != 0) {
    // as the reference's call site lists them (kernels/voxelization/voxelization.cpp:269-284)
    mluop::gen_case::CaseWriter c(handle, "voxelization", "voxelization_param");
    c.input("points", points_desc, points);
    c.input("voxel_size", voxel_size_desc, voxel_size);
    c.input("coors_range", coors_range_desc, coors_range);
    c.output("voxels", voxels_desc);
    c.output("coors", coors_desc);
    c.output("num_points_per_voxel", num_points_per_voxel_desc);
    c.output("voxel_num", voxel_num_desc);
    c.param("max_points", max_points);
    c.param("max_voxels", max_voxels);
    c.param("ndim", NDim);
    c.param("deterministic", deterministic ? 1 : 0);
    c.finish(0.0);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  HIP_CHECK_RETURN(api, hipSetDevice(handle->device));

  const VoxelizeShape s = shapeOf(points_desc, max_points, max_voxels);
  size_t library_bytes = 0;
  HIP_CHECK_RETURN(api,
                   mluop::voxelization::libraryWorkspaceBytes(s, handle->queue, &library_bytes));
  const size_t need = mluop::voxelization::voxelizeWorkspaceBytes(s, library_bytes);
  PARAM_CHECK_V2(api, workspace_size >= need,
                 "workspace_size " << workspace_size << " is below the " << need
                                   << " bytes mluOpGetVoxelizationWorkspaceSize reports.");
  PARAM_CHECK(api, workspace != NULL);

  HIP_CHECK_RETURN(api, mluop::voxelization::launchVoxelize(
                            handle->launchCtx(), s, static_cast<const float *>(points),
                            static_cast<const float *>(voxel_size),
                            static_cast<const float *>(coors_range), workspace, workspace_size,
                            static_cast<float *>(voxels), static_cast<int32_t *>(coors),
                            static_cast<int32_t *>(num_points_per_voxel),
                            static_cast<int32_t *>(voxel_num)));
  return MLUOP_STATUS_SUCCESS;
}
