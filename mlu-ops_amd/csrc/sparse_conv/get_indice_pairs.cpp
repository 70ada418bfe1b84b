// mluOpGetIndicePairs / mluOpGetIndicePairsWorkspaceSize: parameter checks in
// the order (and with the status codes) of reference
// kernels/sparse_conv/get_indice_pairs/get_indice_pairs.cpp:78-277, then the
// HIP rulebook kernel set.
#include <string>

#include "core/core.h"
#include "sparse_conv/rulebook.h"

namespace {

using mluop::sparse_conv::RulebookGeom;

mluOpStatus_t internalGetIndicePairs(mluOpHandle_t handle, const std::string &api,
                                     mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
                                     const mluOpTensorDescriptor_t indices_desc,
                                     const void *indices, void *workspace, size_t workspace_size,
                                     const mluOpTensorDescriptor_t indice_pairs_desc,
                                     void *indice_pairs,
                                     const mluOpTensorDescriptor_t out_indices_desc,
                                     void *out_indices,
                                     const mluOpTensorDescriptor_t indice_num_desc,
                                     void *indice_num, const bool is_get_workspace,
                                     size_t *return_ws) {
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, sparse_conv_desc != NULL);
  PARAM_CHECK(api, indices_desc != NULL);
  PARAM_CHECK(api, indice_pairs_desc != NULL);
  PARAM_CHECK(api, out_indices_desc != NULL);
  PARAM_CHECK(api, indice_num_desc != NULL);

  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported, this handle is on gfx"
                     << handle->arch << ".";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }

  const int conv_dim = sparse_conv_desc->dimNb;
  PARAM_CHECK(api, conv_dim == 5);  // descriptor was never set otherwise

  PARAM_CHECK(api, indices_desc->getDim() == 2);
  PARAM_CHECK(api, indice_pairs_desc->getDim() == 3);
  PARAM_CHECK(api, out_indices_desc->getDim() == 2);
  PARAM_CHECK(api, indice_num_desc->getDim() == 1);
  PARAM_CHECK(api, indices_desc->getDimIndex(1) == 4);
  PARAM_CHECK(api, out_indices_desc->getDimIndex(1) == 4);
  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(1) == 2);

  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(2) == indices_desc->getDimIndex(0));
  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(0) == indice_num_desc->getDimIndex(0));
  int64_t kernel_volume = 1;
  int64_t output_spaces = sparse_conv_desc->batch;
  int64_t input_spaces = sparse_conv_desc->batch;
  for (int i = 0; i < conv_dim - 2; ++i) {
    kernel_volume *= sparse_conv_desc->filter_space[i];
    output_spaces *= sparse_conv_desc->output_space[i];
    input_spaces *= sparse_conv_desc->input_space[i];
  }
  PARAM_CHECK_LE(api, indices_desc->getDimIndex(0), input_spaces);
  for (int i = 0; i < conv_dim - 2; ++i) {
    std::string where = "i: " + std::to_string(i) + ".";
    PARAM_CHECK_V2(api, sparse_conv_desc->pad[i] >= 0, where);
    PARAM_CHECK_V2(api, sparse_conv_desc->dilation[i] >= 1, where);
    PARAM_CHECK_V2(api, sparse_conv_desc->stride[i] >= 1, where);
    if (sparse_conv_desc->dilation[i] != 1 && sparse_conv_desc->stride[i] != 1) {
      MLUOP_LOG(ERROR) << api << " dilation[" << i << "] and stride[" << i
                       << "] cannot both be larger than 1.";
      return MLUOP_STATUS_BAD_PARAM;
    }
  }
  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(0) == kernel_volume);
  PARAM_CHECK_LE(api, kernel_volume, 4096);
  PARAM_CHECK_LE(api, out_indices_desc->getDimIndex(0), output_spaces);

  STRIDE_TENSOR_CHECK(api, indices_desc, "indices_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, indice_pairs_desc, "indice_pairs_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, out_indices_desc, "out_indices_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, indice_num_desc, "indice_num_desc must be contiguous");

  PARAM_CHECK_LE(api, indices_desc->getDimIndex(0), INDICE_IN_LARGE_TENSOR_NUM);
  if (mluOpGetTensorElementNum(indices_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(out_indices_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(indice_pairs_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(indice_num_desc) >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " Overflow max tensor num. Tensors must hold fewer than 2^31 "
                     << "elements.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  // Linear cell indices are 32-bit: batch * volume must stay below 2^31 (the
  // reference multiplies plain ints here without a check).
  if ((uint64_t)output_spaces >= LARGE_TENSOR_NUM || (uint64_t)input_spaces >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " batch * spatial volume must be smaller than 2^31.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  PARAM_CHECK_EQ(api, indices_desc->getDtype(), MLUOP_DTYPE_INT32);
  PARAM_CHECK_EQ(api, indice_pairs_desc->getDtype(), MLUOP_DTYPE_INT32);
  PARAM_CHECK_EQ(api, out_indices_desc->getDtype(), MLUOP_DTYPE_INT32);
  PARAM_CHECK_EQ(api, indice_num_desc->getDtype(), MLUOP_DTYPE_INT32);

  const int sub_m = sparse_conv_desc->sub_m;
  if (sub_m) {
    for (int i = 0; i < conv_dim - 2; ++i) {
      std::string where = "i: " + std::to_string(i) + ".";
      PARAM_CHECK_V2(api, sparse_conv_desc->input_space[i] == sparse_conv_desc->output_space[i],
                     where);
      PARAM_CHECK_V2(api, sparse_conv_desc->stride[i] == 1, where);
      PARAM_CHECK_V2(api, sparse_conv_desc->dilation[i] == 1, where);
    }
  }

  if (mluOpGetTensorElementNum(indices_desc) == 0 ||
      mluOpGetTensorElementNum(indice_pairs_desc) == 0 ||
      mluOpGetTensorElementNum(out_indices_desc) == 0 ||
      mluOpGetTensorElementNum(indice_num_desc) == 0) {
    sparse_conv_desc->num_act_out = 0;
    return MLUOP_STATUS_SUCCESS;
  }

  if (!is_get_workspace) {
    PARAM_CHECK(api, indices != NULL);
    PARAM_CHECK(api, indice_pairs != NULL);
    PARAM_CHECK(api, out_indices != NULL);
    PARAM_CHECK(api, indice_num != NULL);
    if (workspace_size != 0) {
      PARAM_CHECK(api, workspace != NULL);
    }
  }

  RulebookGeom g;
  g.batch = sparse_conv_desc->batch;
  for (int a = 0; a < 3; ++a) {
    g.in_space[a] = sparse_conv_desc->input_space[a];
    g.out_space[a] = sparse_conv_desc->output_space[a];
    g.ksize[a] = sparse_conv_desc->filter_space[a];
    g.pad[a] = sparse_conv_desc->pad[a];
    g.stride[a] = sparse_conv_desc->stride[a];
    g.dilation[a] = sparse_conv_desc->dilation[a];
  }
  g.K = (int)kernel_volume;
  g.L = (int)indices_desc->getDimIndex(0);
  g.out_rows = (int)out_indices_desc->getDimIndex(0);
  g.sub_m = sub_m != 0;

  const size_t need = mluop::sparse_conv::rulebookWorkspaceBytes(g);
  if (is_get_workspace) {
    *return_ws = need;
    return MLUOP_STATUS_SUCCESS;
  }
  if (workspace_size < need || workspace == NULL) {
    MLUOP_LOG(ERROR) << api << " workspace of " << workspace_size << " bytes is smaller than the "
                     << need << " bytes mluOpGetIndicePairsWorkspaceSize reports.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  DEVICE_HANDLE_CHECK(api, handle);

  if (g.sub_m) {
    HIP_CHECK_RETURN(api, mluop::sparse_conv::launchSubmRulebook(
                              handle->launchCtx(), g, static_cast<const int32_t *>(indices), workspace,
                              static_cast<int32_t *>(indice_pairs),
                              static_cast<int32_t *>(out_indices),
                              static_cast<int32_t *>(indice_num)));
    // Submanifold mode leaves num_act_out untouched, as the reference does
    // (normal_get_indice_pairs.cpp:848-975): the caller uses the input row count.
    return MLUOP_STATUS_SUCCESS;
  }

  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchRegularRulebook(
                            handle->launchCtx(), g, static_cast<const int32_t *>(indices), workspace,
                            static_cast<int32_t *>(indice_pairs),
                            static_cast<int32_t *>(out_indices),
                            static_cast<int32_t *>(indice_num), handle->pinned_scalar));
  // The output row count travels back through the host descriptor, which needs
  // one wait on the queue (the reference waits at normal_get_indice_pairs.cpp:531-533).
  HIP_CHECK_RETURN(api, hipStreamSynchronize(handle->queue));
  const int num_act_out = handle->pinned_scalar[0];
  sparse_conv_desc->num_act_out = num_act_out;
  if (num_act_out > g.out_rows) {
    MLUOP_LOG(ERROR) << api << " out_indices holds " << g.out_rows << " rows but "
                     << num_act_out << " output cells are active; rows beyond the tensor "
                     << "were dropped.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  return MLUOP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpGetIndicePairs(
    mluOpHandle_t handle, const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
    const mluOpTensorDescriptor_t indices_desc, const void *indices, void *workspace,
    const size_t workspace_size, const mluOpTensorDescriptor_t indice_pairs_desc,
    void *indice_pairs, const mluOpTensorDescriptor_t out_indices_desc, void *out_indices,
    const mluOpTensorDescriptor_t indice_num_desc, void *indice_num) {
  return internalGetIndicePairs(handle, "[mluOpGetIndicesPairs]", sparse_conv_desc, indices_desc,
                                indices, workspace, workspace_size, indice_pairs_desc,
                                indice_pairs, out_indices_desc, out_indices, indice_num_desc,
                                indice_num, false, NULL);
}

mluOpStatus_t MLUOP_WIN_API mluOpGetIndicePairsWorkspaceSize(
    mluOpHandle_t handle, const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
    const mluOpTensorDescriptor_t indices_desc, const mluOpTensorDescriptor_t indice_pairs_desc,
    const mluOpTensorDescriptor_t out_indices_desc, const mluOpTensorDescriptor_t indice_num_desc,
    size_t *workspace_size) {
  const char *api = "[mluOpGetIndicePairsWorkspaceSize]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, sparse_conv_desc != NULL);
  PARAM_CHECK(api, indices_desc != NULL);
  PARAM_CHECK(api, indice_pairs_desc != NULL);
  PARAM_CHECK(api, out_indices_desc != NULL);
  PARAM_CHECK(api, indice_num_desc != NULL);
  PARAM_CHECK(api, workspace_size != NULL);
  if (mluOpGetTensorElementNum(indices_desc) == 0 ||
      mluOpGetTensorElementNum(indice_pairs_desc) == 0 ||
      mluOpGetTensorElementNum(out_indices_desc) == 0 ||
      mluOpGetTensorElementNum(indice_num_desc) == 0) {
    workspace_size[0] = 0;
    return MLUOP_STATUS_SUCCESS;
  }
  return internalGetIndicePairs(handle, api, sparse_conv_desc, indices_desc, NULL, NULL, 0,
                                indice_pairs_desc, NULL, out_indices_desc, NULL, indice_num_desc,
                                NULL, true, workspace_size);
}

}  // extern "C"
