// mluOpIndiceConvolutionForward and its workspace query.  Checks follow the
// order and status codes of reference
// kernels/sparse_conv/indice_convolution_forward/indice_convolution_forward.cpp:37-169
// and :581-686; bfloat16 is accepted in addition to half and float.
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
  int64_t ci = 0, co = 0, num_filter = 0;
};

FilterDims forwardFilterDims(const mluOpTensorDescriptor_t filters_desc) {
  FilterDims d;
  if (filters_desc->getLayout() == MLUOP_LAYOUT_ARRAY) {
    d.ci = filters_desc->getDimIndex(3);
    d.num_filter =
        filters_desc->getDimIndex(0) * filters_desc->getDimIndex(1) * filters_desc->getDimIndex(2);
    d.co = filters_desc->getDimIndex(4);
  } else {
    d.ci = mluop::dimC(filters_desc);
    d.num_filter =
        mluop::dimD(filters_desc) * mluop::dimH(filters_desc) * mluop::dimW(filters_desc);
    d.co = mluop::dimN(filters_desc);
  }
  return d;
}

mluOpStatus_t foolProof(const std::string &api, mluOpHandle_t handle,
                        const mluOpTensorDescriptor_t features_desc,
                        const mluOpTensorDescriptor_t filters_desc,
                        const mluOpTensorDescriptor_t indice_pairs_desc,
                        const int64_t indice_num[], const int64_t num_act_out,
                        const int64_t inverse, const int64_t sub_m,
                        const mluOpTensorDescriptor_t features_out_desc) {
  PARAM_CHECK(api, handle != nullptr);
  PARAM_CHECK(api, features_desc != nullptr);
  PARAM_CHECK(api, filters_desc != nullptr);
  PARAM_CHECK(api, indice_pairs_desc != nullptr);
  PARAM_CHECK(api, indice_num != nullptr);
  PARAM_CHECK(api, features_out_desc != nullptr);

  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported.";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }

  PARAM_CHECK(api, isConvFloatType(features_desc->getDtype()));
  PARAM_CHECK(api, isConvFloatType(filters_desc->getDtype()));
  PARAM_CHECK(api, indice_pairs_desc->getDtype() == MLUOP_DTYPE_INT32);
  PARAM_CHECK(api, isConvFloatType(features_out_desc->getDtype()));
  PARAM_CHECK(api, features_desc->getDtype() == features_out_desc->getDtype() &&
                       features_desc->getDtype() == filters_desc->getDtype());

  PARAM_CHECK(api, sub_m == 0 || sub_m == 1);
  PARAM_CHECK(api, inverse == 0 || inverse == 1);
  // The reference rejects inverse = 1; so does this library unless the handle
  // was switched to the extended modes (mluOpExtSetSparseConvExtendedModes).
  if (inverse != 0 && !handle->sparse_conv_extended) {
    MLUOP_LOG(ERROR) << api << " inverse is: " << inverse << ", which is not supported now.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  if (filters_desc->getLayout() != MLUOP_LAYOUT_NDHWC &&
      filters_desc->getLayout() != MLUOP_LAYOUT_NCDHW &&
      filters_desc->getLayout() != MLUOP_LAYOUT_ARRAY) {
    MLUOP_LOG(ERROR) << api << " The layout of filters is: "
                     << mluop::getNameOfTensorLayout(filters_desc->getLayout())
                     << ", which is not supported now.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  PARAM_CHECK(api, features_desc->getDim() == 2);
  PARAM_CHECK(api, indice_pairs_desc->getDim() == 3);
  PARAM_CHECK(api, features_out_desc->getDim() == 2);
  if (indice_pairs_desc->getDimIndex(2) > INDICE_IN_LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " indice_pairs_desc->getDimIndex(2) cannot be greater than "
                     << INDICE_IN_LARGE_TENSOR_NUM << ".";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  if (filters_desc->getDim() != 5) {
    MLUOP_LOG(ERROR) << api << " The filters dimension number only support 5 currently, but is "
                     << filters_desc->getDim() << ".";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  STRIDE_TENSOR_CHECK(api, features_desc, "features_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, filters_desc, "filters_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, indice_pairs_desc, "indice_pairs_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, features_out_desc, "features_out_desc must be contiguous");

  if (mluOpGetTensorElementNum(features_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(filters_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(indice_pairs_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(features_out_desc) >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " Max tensor number overflow: tensors must hold fewer than 2^31 "
                     << "elements.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }

  const FilterDims fd = forwardFilterDims(filters_desc);
  // indice_pairs.dim[2] is the row count of the tensor pair column 0 indexes:
  // the input features, or the output of an inverse convolution.
  if (inverse == 0) {
    PARAM_CHECK(api, features_desc->getDimIndex(0) == indice_pairs_desc->getDimIndex(2));
  } else {
    PARAM_CHECK(api, num_act_out == indice_pairs_desc->getDimIndex(2));
  }
  PARAM_CHECK(api, features_desc->getDimIndex(1) == fd.ci);
  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(0) == fd.num_filter);
  PARAM_CHECK(api, indice_pairs_desc->getDimIndex(1) == 2);
  PARAM_CHECK(api, features_out_desc->getDimIndex(0) == num_act_out);
  PARAM_CHECK(api, features_out_desc->getDimIndex(1) == fd.co);

  for (int64_t i = 0; i < fd.num_filter; ++i) {
    std::string where = "i: " + std::to_string(i) + ".";
    // (no more pairs than the pair lists are long: features_desc->getDimIndex(0) in the
    // reference, which is the same number unless the convolution is an inverse one)
    PARAM_CHECK_V2(api, indice_num[i] >= 0 && indice_num[i] <= indice_pairs_desc->getDimIndex(2),
                   where);
  }
  return MLUOP_STATUS_SUCCESS;
}

bool anyZeroElement(const mluOpTensorDescriptor_t a, const mluOpTensorDescriptor_t b,
                    const mluOpTensorDescriptor_t c, const mluOpTensorDescriptor_t d) {
  return mluOpGetTensorElementNum(a) == 0 || mluOpGetTensorElementNum(b) == 0 ||
         mluOpGetTensorElementNum(c) == 0 || mluOpGetTensorElementNum(d) == 0;
}

ConvProblem makeProblem(const mluOpTensorDescriptor_t features_desc,
                        const mluOpTensorDescriptor_t filters_desc,
                        const mluOpTensorDescriptor_t indice_pairs_desc,
                        const int64_t indice_num[], int64_t num_act_out, int64_t inverse,
                        const void *indice_pairs) {
  const FilterDims fd = forwardFilterDims(filters_desc);
  ConvProblem p;
  p.dtype = toElemType(features_desc->getDtype());
  p.K = (int)indice_pairs_desc->getDimIndex(0);
  p.L = (int)indice_pairs_desc->getDimIndex(2);
  p.inverse = inverse != 0;
  p.num_out = p.inverse ? (int)features_desc->getDimIndex(0) : (int)num_act_out;
  p.Ci = (int)fd.ci;
  p.Co = (int)fd.co;
  p.indice_pairs = static_cast<const int32_t *>(indice_pairs);
  p.indice_num = indice_num;
  return p;
}

FilterView forwardFilterView(const mluOpTensorDescriptor_t filters_desc, const void *filters,
                             const ConvProblem &p) {
  // Element strides of W(k, ci, co) in the three accepted layouts:
  // ARRAY [kd,kh,kw,Ci,Co], NDHWC [Co,kd,kh,kw,Ci], NCDHW [Co,Ci,kd,kh,kw].
  FilterView f;
  f.base = filters;
  switch (filters_desc->getLayout()) {
    case MLUOP_LAYOUT_NDHWC:
      f.stride_k = p.Ci;
      f.stride_ci = 1;
      f.stride_co = (int64_t)p.K * p.Ci;
      break;
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

mluOpStatus_t MLUOP_WIN_API mluOpGetIndiceConvolutionForwardWorkspaceSize(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc,
    const mluOpTensorDescriptor_t filters_desc, const mluOpTensorDescriptor_t indice_pairs_desc,
    const mluOpTensorDescriptor_t features_out_desc, const int64_t indice_num[],
    const int64_t num_act_out, const int64_t inverse, const int64_t sub_m, size_t *size) {
  const std::string api = "[mluOpGetIndiceConvolutionForwardWorkspaceSize]";
  mluOpStatus_t st = foolProof(api, handle, features_desc, filters_desc, indice_pairs_desc,
                               indice_num, num_act_out, inverse, sub_m, features_out_desc);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (anyZeroElement(features_desc, indice_pairs_desc, filters_desc, features_out_desc)) {
    return MLUOP_STATUS_SUCCESS;
  }
  PARAM_CHECK(api, size != nullptr);
  const ConvProblem p = makeProblem(features_desc, filters_desc, indice_pairs_desc, indice_num,
                                    num_act_out, inverse, nullptr);
  *size = mluop::sparse_conv::gatherConvWorkspaceBytes(p, GatherDirection::kForward);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpIndiceConvolutionForward(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc, const void *features,
    const mluOpTensorDescriptor_t filters_desc, const void *filters,
    const mluOpTensorDescriptor_t indice_pairs_desc, const void *indice_pairs,
    const int64_t indice_num[], const int64_t num_act_out, const int64_t inverse,
    const int64_t sub_m, void *workspace, size_t workspace_size,
    const mluOpTensorDescriptor_t features_out_desc, void *features_out) {
  const std::string api = "[mluOpIndiceConvolutionForward]";
  const void *announced_map = mluop::sparse_conv::announcedRowMap(handle);
  mluOpStatus_t st = foolProof(api, handle, features_desc, filters_desc, indice_pairs_desc,
                               indice_num, num_act_out, inverse, sub_m, features_out_desc);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (anyZeroElement(filters_desc, features_desc, indice_pairs_desc, features_out_desc)) {
    return MLUOP_STATUS_SUCCESS;
  }
  PARAM_CHECK(api, features != nullptr);
  PARAM_CHECK(api, filters != nullptr);
  PARAM_CHECK(api, indice_pairs != nullptr);
  PARAM_CHECK(api, features_out != nullptr);
  if (workspace_size > 0) {
    PARAM_CHECK(api, workspace != nullptr);
  }

  ConvProblem p = makeProblem(features_desc, filters_desc, indice_pairs_desc, indice_num,
                              num_act_out, inverse, indice_pairs);
  p.distinct_pairs = handle->distinct_pairs_promised;
  st = mluop::sparse_conv::takeRowMap(api, handle, announced_map, GatherDirection::kForward, &p);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  // what this call overwrites is no pair tensor any more, whatever the handle noted there
  mluop::sparse_conv::forgetRulebookNotesIn(handle, features_out, features_out_desc->total_tensor_size);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, workspace, workspace_size);
  // result rows are named by pair column 1 (the other one in an inverse convolution)
  mluop::sparse_conv::consultRulebookNotes(handle, p.inverse ? 0 : 1, &p);
  const size_t need = mluop::sparse_conv::gatherConvWorkspaceBytes(p, GatherDirection::kForward);
  if (workspace_size < need || workspace == nullptr) {
    MLUOP_LOG(ERROR) << api << " workspace of " << workspace_size
                     << " bytes is smaller than the " << need
                     << " bytes mluOpGetIndiceConvolutionForwardWorkspaceSize reports.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (mluop::gen_case::mode() != 0) {
    // (reference indice_convolution_forward.cpp:657-675; tensor ids as the test runner's executor reads them)
    mluop::gen_case::CaseWriter c(handle, "indice_convolution_forward", "indice_convolution_forward_param");
    c.input("features", features_desc, features);
    c.input("filters", filters_desc, filters);
    c.input("indice_pairs", indice_pairs_desc, indice_pairs);
    c.output("features_out", features_out_desc);
    c.params("indice_num", indice_num, p.K);
    c.param("num_active_out", num_act_out);
    c.param("sub_m", sub_m);
    c.param("inverse", inverse);
    c.finish(0.003);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  const FilterView f = forwardFilterView(filters_desc, filters, p);
  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchGatherConv(handle->launchCtx(), p,
                                                            GatherDirection::kForward, features,
                                                            f, workspace, features_out));
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
