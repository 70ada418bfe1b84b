// Sparse-convolution descriptor: a host-side record of one 3-D sparse convolution (spaces,
// padding, stride, dilation, submanifold flag) plus the number of active outputs that the
// regular-mode rulebook leaves in it.  Which arguments are refused, and with which status,
// follows the reference (get_indice_pairs_structs.cpp:31-134); how they are checked does
// not: the setter looks at every argument first and writes the descriptor only when all of
// them passed, so a refused call leaves the descriptor as it was.
#include <new>

#include "core/core.h"

namespace {

constexpr int kSpatialAxes = 3;

// One per-axis argument of the setter: its values, the least value allowed, and where in
// the descriptor the three values go.
struct AxisArgument {
  const char *name;
  const int *values;
  int least;
  int *destination;
};

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API
mluOpCreateSparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t *desc) {
  if (desc == NULL) {
    MLUOP_LOG(ERROR) << "[mluOpCreateSparseConvolutionDescriptor] no place to return the descriptor "
                        "(desc is NULL).";
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

  // pass 1: look at everything, write nothing
  mluOpSparseConvolutionStruct filled = *sparse_conv_desc;
  const AxisArgument per_axis[] = {
      {"pad", pad, 0, filled.pad},
      {"stride", stride, 1, filled.stride},
      {"dilation", dilation, 1, filled.dilation},
      {"input_space", input_space, 1, filled.input_space},
      {"filter_space", filter_space, 1, filled.filter_space},
      {"output_space", output_space, 1, filled.output_space},
  };
  for (const AxisArgument &arg : per_axis) {
    if (arg.values == NULL) {
      MLUOP_LOG(ERROR) << api << " " << arg.name << " is NULL.";
      return MLUOP_STATUS_BAD_PARAM;
    }
  }
  if (dimNb != kSpatialAxes + 2) {
    MLUOP_LOG(ERROR) << api << " dimNb is " << dimNb << "; a 3-D convolution has " << kSpatialAxes + 2
                     << " dimensions (batch, three spatial axes, channels).";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (batch <= 0) {
    MLUOP_LOG(ERROR) << api << " batch is " << batch << ", it must be positive.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (transpose != 0 || inverse != 0) {
    MLUOP_LOG(ERROR) << api << " transposed and inverse convolutions are not supported (transpose "
                     << transpose << ", inverse " << inverse << ").";
    return MLUOP_STATUS_BAD_PARAM;
  }
  for (int axis = 0; axis < kSpatialAxes; ++axis) {
    for (const AxisArgument &arg : per_axis) {
      if (arg.values[axis] < arg.least) {
        MLUOP_LOG(ERROR) << api << " " << arg.name << "[" << axis << "] is " << arg.values[axis]
                         << ", below " << arg.least << ".";
        return MLUOP_STATUS_BAD_PARAM;
      }
      arg.destination[axis] = arg.values[axis];
    }
  }
  filled.dimNb = dimNb;
  filled.batch = batch;
  filled.sub_m = sub_m;
  filled.transpose = transpose;
  filled.inverse = inverse;

  // pass 2: all of it passed
  *sparse_conv_desc = filled;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API
mluOpGetSparseConvolutionNumActOut(mluOpSparseConvolutionDescriptor_t desc, int *num_act_out) {
  if (desc == NULL || num_act_out == NULL) {
    MLUOP_LOG(ERROR) << "[mluOpGetSparseConvolutionNumActOut] "
                     << (desc == NULL ? "the descriptor" : "num_act_out") << " is NULL.";
    return MLUOP_STATUS_NOT_INITIALIZED;
  }
  *num_act_out = desc->num_act_out;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API
mluOpDestroySparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t desc) {
  if (desc == NULL) {
    MLUOP_LOG(ERROR) << "[mluOpDestroySparseConvolutionDescriptor] nothing to destroy (NULL).";
    return MLUOP_STATUS_EXECUTION_FAILED;
  }
  delete desc;
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
