// mluOpIndiceConvolutionBackwardData and its workspace query.  Checks follow
// the order and status codes of reference
// kernels/sparse_conv/indice_convolution_backward_data/
// indice_convolution_backward_data.cpp:34-241 (foolCheckNoPtr), :279-306
// (pointer checks) and :358-617 (entry points); bfloat16 is accepted too.
#include <string>

#include "core/core.h"
#include "core/gen_case.h"
#include "sparse_conv/indice_conv.h"
#include "sparse_conv/row_map.h"
#include "sparse_conv/rulebook_notes.h"

namespace {

using mluop::sparse_conv::ConvProblem;
using mluop::sparse_conv::ElemType;
using mluop::sparse_conv::FilterView;
using mluop::sparse_conv::GatherDirection;

bool isConvFloatType(mluOpDataType_t t) {
  return t == MLUOP_DTYPE_FLOAT || t == MLUOP_DTYPE_HALF || t == MLUOP_DTYPE_BFLOAT16;
}

ElemType toElemType(mluOpDataType_t t) {
  return t == MLUOP_DTYPE_FLOAT ? ElemType::kFloat
                                : (t == MLUOP_DTYPE_HALF ? ElemType::kHalf : ElemType::kBFloat16);
}

struct FilterDims {
  int64_t kd = 1, kh = 1, kw = 1, dyc = 1, dxc = 1;
  int64_t K() const { return kd * kh * kw; }
};

// dyc = output channels (Co), dxc = input channels (Ci).
FilterDims filterDims(const mluOpTensorDescriptor_t filters_desc) {
  FilterDims d;
  if (filters_desc->getLayout() != MLUOP_LAYOUT_ARRAY) {
    d.kh = mluop::dimH(filters_desc);
    d.kw = mluop::dimW(filters_desc);
    d.dyc = mluop::dimN(filters_desc);
    d.dxc = mluop::dimC(filters_desc);
    if (filters_desc->getDim() == 5) d.kd = mluop::dimD(filters_desc);
  } else {
    const int n = filters_desc->getDim();
    if (n == 5) d.kd = filters_desc->getDimIndex(0);
    d.kh = filters_desc->getDimIndex(n - 4);
    d.kw = filters_desc->getDimIndex(n - 3);
    d.dxc = filters_desc->getDimIndex(n - 2);
    d.dyc = filters_desc->getDimIndex(n - 1);
  }
  return d;
}

int64_t maxCount(const int64_t *indice_num, int64_t K) {
  int64_t m = indice_num[0];
  for (int64_t i = 1; i < K; ++i) m = indice_num[i] > m ? indice_num[i] : m;
  return m;
}

mluOpStatus_t foolCheckNoPtr(mluOpHandle_t handle, const mluOpTensorDescriptor_t output_grad_desc,
                             const mluOpTensorDescriptor_t filters_desc,
                             const mluOpTensorDescriptor_t indice_pairs_desc,
                             const int64_t indice_num[], const int64_t inverse,
                             const int64_t sub_m, const mluOpTensorDescriptor_t input_grad_desc,
                             bool *is_zero) {
  const std::string api = "[mluOpIndiceConvolutionBackwardData]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, output_grad_desc != NULL);
  PARAM_CHECK(api, filters_desc != NULL);
  PARAM_CHECK(api, indice_pairs_desc != NULL);
  PARAM_CHECK(api, input_grad_desc != NULL);
  // The reference reads indice_num without testing it; a NULL array is a bad
  // parameter here rather than a crash.
  PARAM_CHECK(api, indice_num != NULL);

  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported.";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }

  PARAM_CHECK_EQ(api, output_grad_desc->getDim(), 2);
  PARAM_CHECK(api, filters_desc->getDim() == 4 || filters_desc->getDim() == 5);
  PARAM_CHECK_EQ(api, indice_pairs_desc->getDim(), 3);
  PARAM_CHECK_EQ(api, input_grad_desc->getDim(), 2);

  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(1) == 2);
  if (indice_pairs_desc->getDimIndex(2) > INDICE_IN_LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " indice_pairs_desc->getDimIndex(2) cannot be greater than "
                     << INDICE_IN_LARGE_TENSOR_NUM << ".";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  PARAM_CHECK(api, isConvFloatType(output_grad_desc->getDtype()));
  PARAM_CHECK(api, isConvFloatType(filters_desc->getDtype()));
  PARAM_CHECK(api, isConvFloatType(input_grad_desc->getDtype()));
  PARAM_CHECK(api, indice_pairs_desc->getDtype() == MLUOP_DTYPE_INT32);

  const mluOpTensorLayout_t layout = filters_desc->getLayout();
  const bool layout_ok = layout == MLUOP_LAYOUT_NHWC || layout == MLUOP_LAYOUT_NCHW ||
                         layout == MLUOP_LAYOUT_HWCN || layout == MLUOP_LAYOUT_NCDHW ||
                         layout == MLUOP_LAYOUT_NDHWC || layout == MLUOP_LAYOUT_ARRAY;
  if (!layout_ok) {
    MLUOP_LOG(ERROR) << api
                     << " The filters tensor only supports NHWC/NCHW/HWCN/NCDHW/NDHWC/ARRAY "
                     << "layout.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  STRIDE_TENSOR_CHECK(api, output_grad_desc, "output_grad_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, filters_desc, "filters_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, indice_pairs_desc, "indice_pairs_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, input_grad_desc, "input_grad_desc must be contiguous");

  const FilterDims fd = filterDims(filters_desc);
  const int64_t K = fd.K();

  PARAM_CHECK(api, inverse == 0 || inverse == 1);
  PARAM_CHECK(api, sub_m == 0 || sub_m == 1);
  for (int64_t kk = 0; kk < K; ++kk) {
    PARAM_CHECK(api, indice_num[kk] >= 0);
  }
  // Rejected as in the reference unless the handle was switched to the extended
  // modes (mluOpExtSetSparseConvExtendedModes).
  if (inverse == 1 && !handle->sparse_conv_extended) {
    MLUOP_LOG(ERROR) << api << " Not support inverse == 1 yet.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  // The tensor pair column 0 indexes has indice_pairs.dim[2] rows: input_grad,
  // or output_grad of an inverse convolution.
  const mluOpTensorDescriptor_t col0_desc = inverse == 1 ? output_grad_desc : input_grad_desc;
  const char *col0_name = inverse == 1 ? "output_grad" : "input_grad";

  if (K != indice_pairs_desc->getDimIndex(0)) {
    MLUOP_LOG(ERROR) << api << " The dims[0] of indice_pairs should be equal to kd*kh*kw.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (output_grad_desc->getDimIndex(1) != fd.dyc) {
    MLUOP_LOG(ERROR) << api << " The dims[1] of output_grad should be equal to dyc of filters.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (input_grad_desc->getDimIndex(1) != fd.dxc) {
    MLUOP_LOG(ERROR) << api << " The dims[1] of input_grad should be equal to dxc of filters.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (col0_desc->getDimIndex(0) != indice_pairs_desc->getDimIndex(2)) {
    MLUOP_LOG(ERROR) << api << " The dims[0] of " << col0_name
                     << " should be equal to the dims[2] of indice_pairs.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  const int64_t max_indice_num = K > 0 ? maxCount(indice_num, K) : 0;
  if (indice_pairs_desc->getDimIndex(2) < max_indice_num) {
    MLUOP_LOG(ERROR) << api << " The data in indice_num array should be smaller or equal to the "
                     << "dims[2] of indice_pairs.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (sub_m == 1) {
    if (input_grad_desc->getDimIndex(0) != output_grad_desc->getDimIndex(0)) {
      MLUOP_LOG(ERROR) << api << " The dims[0] of input_grad should be equal to the dims[0] of "
                       << "output_grad when sub_m is 1.";
      return MLUOP_STATUS_BAD_PARAM;
    }
    if (K > 0 && indice_num[K / 2] < max_indice_num) {
      MLUOP_LOG(ERROR) << api << " The middle number of the indice_num array should be the "
                       << "maximum of the array when sub_m is 1.";
      return MLUOP_STATUS_BAD_PARAM;
    }
  }
  // (the reference's rule for output_grad; an inverse convolution's input_grad may have fewer
  // rows than an offset has pairs when the partner layer's coordinates repeat)
  if (inverse == 0 && output_grad_desc->getDimIndex(0) < max_indice_num) {
    MLUOP_LOG(ERROR) << api << " The dims[0] of output_grad should be larger than or equal to "
                     << "the maximum number of indice_num.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (sub_m == 1 && K % 2 == 0) {
    MLUOP_LOG(ERROR) << api << " When sub_m value is 1, the filters dims (Kd, Kh & Kw) should be "
                     << "odd numbers.";
    return MLUOP_STATUS_BAD_PARAM;
  }

  PARAM_CHECK(api, output_grad_desc->getDtype() == input_grad_desc->getDtype());
  PARAM_CHECK(api, output_grad_desc->getDtype() == filters_desc->getDtype());

  const uint64_t input_grad_count = mluOpGetTensorElementNum(input_grad_desc);
  TENSOR_NUM_CHECK(api, input_grad_count, LARGE_TENSOR_NUM, "input_grad tensor num is too large. ");
  const uint64_t output_grad_count = mluOpGetTensorElementNum(output_grad_desc);
  TENSOR_NUM_CHECK(api, output_grad_count, LARGE_TENSOR_NUM,
                   "output_grad tensor num is too large. ");
  const uint64_t filter_count = mluOpGetTensorElementNum(filters_desc);
  TENSOR_NUM_CHECK(api, filter_count, LARGE_TENSOR_NUM, "filters tensor num is too large. ");
  const uint64_t indice_pairs_count = mluOpGetTensorElementNum(indice_pairs_desc);
  TENSOR_NUM_CHECK(api, indice_pairs_count, LARGE_TENSOR_NUM,
                   "indice_pairs tensor num is too large. ");

  if (input_grad_count == 0 || output_grad_count == 0 || filter_count == 0 ||
      indice_pairs_count == 0) {
    *is_zero = true;
  }
  return MLUOP_STATUS_SUCCESS;
}

ConvProblem makeProblem(const mluOpTensorDescriptor_t output_grad_desc,
                        const mluOpTensorDescriptor_t filters_desc,
                        const mluOpTensorDescriptor_t indice_pairs_desc,
                        const mluOpTensorDescriptor_t input_grad_desc, const int64_t indice_num[],
                        int64_t inverse, const void *indice_pairs) {
  const FilterDims fd = filterDims(filters_desc);
  ConvProblem p;
  p.dtype = toElemType(filters_desc->getDtype());
  p.K = (int)indice_pairs_desc->getDimIndex(0);
  p.L = (int)indice_pairs_desc->getDimIndex(2);
  p.inverse = inverse != 0;
  p.num_out = (int)(p.inverse ? input_grad_desc : output_grad_desc)->getDimIndex(0);
  p.Ci = (int)fd.dxc;
  p.Co = (int)fd.dyc;
  p.indice_pairs = static_cast<const int32_t *>(indice_pairs);
  p.indice_num = indice_num;
  return p;
}

FilterView filterView(const mluOpTensorDescriptor_t filters_desc, const void *filters,
                      const ConvProblem &p) {
  // Element strides of W(k, ci, co): N = Co, C = Ci in the named layouts;
  // HWCN and ARRAY are (kd,)kh,kw,Ci,Co.
  FilterView f;
  f.base = filters;
  switch (filters_desc->getLayout()) {
    case MLUOP_LAYOUT_NHWC:
    case MLUOP_LAYOUT_NDHWC:
      f.stride_k = p.Ci;
      f.stride_ci = 1;
      f.stride_co = (int64_t)p.K * p.Ci;
      break;
    case MLUOP_LAYOUT_NCHW:
    case MLUOP_LAYOUT_NCDHW:
      f.stride_k = 1;
      f.stride_ci = p.K;
      f.stride_co = (int64_t)p.Ci * p.K;
      break;
    default:
      f.stride_k = (int64_t)p.Ci * p.Co;
      f.stride_ci = p.Co;
      f.stride_co = 1;
      break;
  }
  return f;
}

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t output_grad_desc,
    const mluOpTensorDescriptor_t filters_desc, const mluOpTensorDescriptor_t indice_pairs_desc,
    const mluOpTensorDescriptor_t input_grad_desc, const int64_t indice_num[],
    const int64_t inverse, size_t *workspace_size) {
  const char *api = "[mluOpGetIndiceConvolutionBackwardDataWorkspaceSize]";
  if (workspace_size == NULL) {
    MLUOP_LOG(ERROR) << api << " The pointer workspace_size should not be nullptr.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  bool is_zero = false;
  mluOpStatus_t st = foolCheckNoPtr(handle, output_grad_desc, filters_desc, indice_pairs_desc,
                                    indice_num, inverse, 0, input_grad_desc, &is_zero);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (is_zero) return MLUOP_STATUS_SUCCESS;
  const ConvProblem p =
      makeProblem(output_grad_desc, filters_desc, indice_pairs_desc, input_grad_desc, indice_num,
                  inverse, nullptr);
  *workspace_size =
      mluop::sparse_conv::gatherConvWorkspaceBytes(p, GatherDirection::kBackwardData);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpIndiceConvolutionBackwardData(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t output_grad_desc,
    const void *output_grad, const mluOpTensorDescriptor_t filters_desc, const void *filters,
    const mluOpTensorDescriptor_t indice_pairs_desc, const void *indice_pairs,
    const int64_t indice_num[], const int64_t inverse, const int64_t sub_m, void *workspace,
    const size_t workspace_size, const mluOpTensorDescriptor_t input_grad_desc,
    void *input_grad) {
  const std::string api = "[mluOpIndiceConvolutionBackwardData]";
  const void *announced_map = mluop::sparse_conv::announcedRowMap(handle);
  bool is_zero = false;
  mluOpStatus_t st = foolCheckNoPtr(handle, output_grad_desc, filters_desc, indice_pairs_desc,
                                    indice_num, inverse, sub_m, input_grad_desc, &is_zero);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (is_zero) return MLUOP_STATUS_SUCCESS;

  PARAM_CHECK(api, output_grad != NULL);
  PARAM_CHECK(api, filters != NULL);
  PARAM_CHECK(api, indice_pairs != NULL);
  PARAM_CHECK(api, input_grad != NULL);
  if (workspace_size > 0) {
    PARAM_CHECK(api, workspace != NULL);
  }

  ConvProblem p = makeProblem(output_grad_desc, filters_desc, indice_pairs_desc, input_grad_desc,
                              indice_num, inverse, indice_pairs);
  p.distinct_pairs = handle->distinct_pairs_promised;
  st = mluop::sparse_conv::takeRowMap(api, handle, announced_map, GatherDirection::kBackwardData, &p);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  // what this call overwrites is no pair tensor any more, whatever the handle noted there
  mluop::sparse_conv::forgetRulebookNotesIn(handle, input_grad, input_grad_desc->total_tensor_size);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, workspace, workspace_size);
  // result rows are named by pair column 0 (the other one in an inverse convolution)
  mluop::sparse_conv::consultRulebookNotes(handle, p.inverse ? 1 : 0, &p);
  const size_t need =
      mluop::sparse_conv::gatherConvWorkspaceBytes(p, GatherDirection::kBackwardData);
  if (workspace_size < need || workspace == NULL) {
    MLUOP_LOG(ERROR) << api << " workspace of " << workspace_size
                     << " bytes is smaller than the " << need
                     << " bytes mluOpGetIndiceConvolutionBackwardDataWorkspaceSize reports.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (mluop::gen_case::mode() != 0) {
    // (reference indice_convolution_backward_data.cpp:316-332)
    mluop::gen_case::CaseWriter c(handle, "indice_convolution_backward_data",
                                  "indice_convolution_backward_data_param");
    c.input("output_grad", output_grad_desc, output_grad);
    c.input("filters", filters_desc, filters);
    c.input("indice_pairs", indice_pairs_desc, indice_pairs);
    c.output("input_grad", input_grad_desc);
    c.params("indice_num", indice_num, p.K);
    c.param("sub_m", sub_m);
    c.param("inverse", inverse);
    c.finish(0.003);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  const FilterView f = filterView(filters_desc, filters, p);
  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchGatherConv(
                            handle->launchCtx(), p, GatherDirection::kBackwardData, output_grad, f,
                            workspace, input_grad));
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
