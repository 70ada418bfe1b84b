// Sparse-convolution descriptor: a host-side POD describing one 3-D sparse
// convolution (spaces, padding, stride, dilation, submanifold flag) plus the
// number of active outputs that regular-mode rulebook construction returns.
// Status codes follow reference get_indice_pairs_structs.cpp:31-134.
#include <new>
#include <string>

#include "core/core.h"

extern "C" {

mluOpStatus_t MLUOP_WIN_API
mluOpCreateSparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t *desc) {
  if (desc == NULL) {
    MLUOP_LOG(ERROR) << "mluOpCreateSparseConvolutionDescriptor failed, "
                     << "can't create desc when desc == NULL.";
    return MLUOP_STATUS_NOT_INITIALIZED;
  }
  *desc = new (std::nothrow) mluOpSparseConvolutionStruct();
  return *desc ? MLUOP_STATUS_SUCCESS : MLUOP_STATUS_ALLOC_FAILED;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetSparseConvolutionDescriptor(
    mluOpSparseConvolutionDescriptor_t sparse_conv_desc, int dimNb, int batch, const int pad[],
    const int stride[], const int dilation[], const int input_space[], const int filter_space[],
    const int output_space[], const int sub_m, const int transpose, const int inverse) {
  const char *api = "[mluOpSetSparseConvolutionDescriptor]";
  PARAM_CHECK(api, sparse_conv_desc != NULL);
  PARAM_CHECK(api, pad != NULL);
  PARAM_CHECK(api, stride != NULL);
  PARAM_CHECK(api, dilation != NULL);
  PARAM_CHECK(api, input_space != NULL);
  PARAM_CHECK(api, filter_space != NULL);
  PARAM_CHECK(api, output_space != NULL);
  if (dimNb != 5) {
    MLUOP_LOG(ERROR) << api << " only supports 3-D convolution, dimNb should be 5, now "
                     << dimNb << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  sparse_conv_desc->dimNb = dimNb;
  if (batch <= 0) {
    MLUOP_LOG(ERROR) << api << " only supports positive batch, now " << batch << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  sparse_conv_desc->batch = batch;
  sparse_conv_desc->sub_m = sub_m;
  if (transpose != 0) {
    MLUOP_LOG(ERROR) << api << " transpose is not supported, now " << transpose << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  sparse_conv_desc->transpose = transpose;
  if (inverse != 0) {
    MLUOP_LOG(ERROR) << api << " inverse is not supported, now " << inverse << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  sparse_conv_desc->inverse = inverse;

  const int kernel_dim = dimNb - 2;
  for (int idx = 0; idx < kernel_dim; ++idx) {
    std::string where = "idx: " + std::to_string(idx) + ".";
    PARAM_CHECK_V2(api, pad[idx] >= 0, where);
    sparse_conv_desc->pad[idx] = pad[idx];
    PARAM_CHECK_V2(api, stride[idx] >= 1, where);
    sparse_conv_desc->stride[idx] = stride[idx];
    PARAM_CHECK_V2(api, dilation[idx] >= 1, where);
    sparse_conv_desc->dilation[idx] = dilation[idx];
    PARAM_CHECK_V2(api, input_space[idx] >= 1, where);
    sparse_conv_desc->input_space[idx] = input_space[idx];
    PARAM_CHECK_V2(api, filter_space[idx] >= 1, where);
    sparse_conv_desc->filter_space[idx] = filter_space[idx];
    PARAM_CHECK_V2(api, output_space[idx] >= 1, where);
    sparse_conv_desc->output_space[idx] = output_space[idx];
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API
mluOpGetSparseConvolutionNumActOut(mluOpSparseConvolutionDescriptor_t desc, int *num_act_out) {
  if (desc == NULL || num_act_out == NULL) {
    MLUOP_LOG(ERROR) << "mluOpGetSparseConvolutionNumActOut: passing NULL ptr to this API.";
    return MLUOP_STATUS_NOT_INITIALIZED;
  }
  *num_act_out = desc->num_act_out;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API
mluOpDestroySparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t desc) {
  if (desc == NULL) {
    MLUOP_LOG(ERROR) << "mluOpDestroySparseConvolutionDescriptor fail. Passing NULL ptr.";
    return MLUOP_STATUS_EXECUTION_FAILED;
  }
  delete desc;
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
