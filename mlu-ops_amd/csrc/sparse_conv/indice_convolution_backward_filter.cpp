// mluOpIndiceConvolutionBackwardFilter and its workspace query.  Checks follow
// the order and status codes of reference
// kernels/sparse_conv/indice_convolution_backward_filter/
// indice_convolution_backward_filter.cpp:100-258 and :536-620; bfloat16 is
// accepted in addition to half and float.
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "core/core.h"
#include "core/gen_case.h"
#include "mlu_op_ext.h"
#include "sparse_conv/indice_conv.h"
#include "sparse_conv/rulebook_notes.h"
#include "sparse_conv/no_alloc_scratch.h"

namespace {

// Device memory of mluOpExtIndiceConvolutionBackwardFilterNoAlloc: the fp32 partial tiles
// that the ordinary entry point keeps in the caller's workspace.  One copy per GPU, held
// until the process ends.  The name is a host-side stand-in: host code uses the address
// hipGetSymbolAddress returned for the device in question, never the name.
static __device__ __align__(256) unsigned char scratch[MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES];

constexpr int kMaxScratchDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxScratchDevices] = {nullptr};

using mluop::sparse_conv::ConvProblem;
using mluop::sparse_conv::ElemType;

bool isFloatDtype(mluOpDataType_t t) {
  return t == MLUOP_DTYPE_HALF || t == MLUOP_DTYPE_FLOAT || t == MLUOP_DTYPE_BFLOAT16;
}

ElemType toElemType(mluOpDataType_t t) {
  return t == MLUOP_DTYPE_FLOAT ? ElemType::kFloat
                                : (t == MLUOP_DTYPE_HALF ? ElemType::kHalf : ElemType::kBFloat16);
}

mluOpStatus_t dtypeValid(const std::string &api, const mluOpTensorDescriptor_t features_desc,
                         const mluOpTensorDescriptor_t output_grad_desc,
                         const mluOpTensorDescriptor_t indice_pairs_desc,
                         const mluOpTensorDescriptor_t filters_grad_desc) {
  const mluOpDataType_t input_dtype = features_desc->getDtype();
  const mluOpDataType_t diffy_dtype = output_grad_desc->getDtype();
  const mluOpDataType_t filters_grad_dtype = filters_grad_desc->getDtype();
  const mluOpDataType_t pairs_dtype = indice_pairs_desc->getDtype();
  if (pairs_dtype != MLUOP_DTYPE_INT32) {
    MLUOP_LOG(ERROR) << api << " indice_pairs_desc only supports data type int32, now "
                     << mluop::getNameOfDataType(pairs_dtype) << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (input_dtype != diffy_dtype || input_dtype != filters_grad_dtype ||
      !isFloatDtype(input_dtype) || !isFloatDtype(diffy_dtype) ||
      !isFloatDtype(filters_grad_dtype)) {
    MLUOP_LOG(ERROR) << api << " The data type of features_desc, output_grad_desc and "
                     << "filters_grad_desc should be the same floating-point type. Now "
                     << mluop::getNameOfDataType(input_dtype) << "-"
                     << mluop::getNameOfDataType(diffy_dtype) << "-"
                     << mluop::getNameOfDataType(filters_grad_dtype) << ".";
    return MLUOP_STATUS_BAD_PARAM;
  }
  const mluOpDataType_t input_on = features_desc->getOnchipDtype();
  const mluOpDataType_t diffy_on = output_grad_desc->getOnchipDtype();
  const mluOpDataType_t grad_on = filters_grad_desc->getOnchipDtype();
  const mluOpDataType_t pairs_on = indice_pairs_desc->getOnchipDtype();
  if ((input_on != MLUOP_DTYPE_INVALID && input_on != input_dtype) ||
      (diffy_on != MLUOP_DTYPE_INVALID && diffy_on != diffy_dtype) ||
      (pairs_on != MLUOP_DTYPE_INVALID && pairs_on != pairs_dtype)) {
    MLUOP_LOG(ERROR) << api << " For features_desc, output_grad_desc and indice_pairs_desc the "
                     << "on-chip data type, when set, must equal the off-chip data type.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if ((grad_on != MLUOP_DTYPE_INVALID && !isFloatDtype(grad_on)) ||
      (filters_grad_dtype == MLUOP_DTYPE_FLOAT && grad_on == MLUOP_DTYPE_HALF)) {
    MLUOP_LOG(ERROR) << api << " The on-chip data type of filters_grad_desc, when set, must be a "
                     << "floating-point type at least as wide as the off-chip data type.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  return MLUOP_STATUS_SUCCESS;
}

// Extents and element strides of dW(k, ci, co) in filters_grad.  The reference takes the
// dimensions positionally as (kd,) kh, kw, Ci, Co whatever the layout tag says
// (indice_convolution_backward_filter.cpp:227-242); with the extended modes on,
// a tensor tagged N(D)HWC is [Co, (kd,) kh, kw, Ci] and one tagged NC(D)HW is
// [Co, Ci, (kd,) kh, kw], as the forward and backward-data operators read their filters.
struct GradDims {
  int64_t K, ci, co;
  int64_t stride_k, stride_ci, stride_co;
};

GradDims gradDims(const mluOpTensorDescriptor_t desc, bool extended) {
  const int n = desc->getDim();
  auto volume = [&](int first) {
    int64_t v = 1;
    for (int i = first; i < first + n - 2; ++i) v *= desc->getDimIndex(i);
    return v;
  };
  const mluOpTensorLayout_t layout = desc->getLayout();
  GradDims g;
  if (extended && (layout == MLUOP_LAYOUT_NHWC || layout == MLUOP_LAYOUT_NDHWC)) {
    g.co = desc->getDimIndex(0); g.ci = desc->getDimIndex(n - 1); g.K = volume(1);
    g.stride_k = g.ci; g.stride_ci = 1; g.stride_co = g.K * g.ci;
  } else if (extended && (layout == MLUOP_LAYOUT_NCHW || layout == MLUOP_LAYOUT_NCDHW)) {
    g.co = desc->getDimIndex(0); g.ci = desc->getDimIndex(1); g.K = volume(2);
    g.stride_k = 1; g.stride_ci = g.K; g.stride_co = g.ci * g.K;
  } else {
    g.ci = desc->getDimIndex(n - 2); g.co = desc->getDimIndex(n - 1); g.K = volume(0);
    g.stride_k = g.ci * g.co; g.stride_ci = g.co; g.stride_co = 1;
  }
  return g;
}

mluOpStatus_t baseParamCheck(const std::string &api, mluOpHandle_t handle,
                             const mluOpTensorDescriptor_t features_desc,
                             const mluOpTensorDescriptor_t output_grad_desc,
                             const mluOpTensorDescriptor_t indice_pairs_desc,
                             const mluOpTensorDescriptor_t filters_grad_desc,
                             const int64_t indice_num[], const int64_t inverse) {
  PARAM_CHECK(api, handle != nullptr);
  PARAM_CHECK(api, features_desc != nullptr);
  PARAM_CHECK(api, output_grad_desc != nullptr);
  PARAM_CHECK(api, indice_pairs_desc != nullptr);
  PARAM_CHECK(api, filters_grad_desc != nullptr);
  PARAM_CHECK(api, indice_num != nullptr);
  // inverse = 1 is a bad parameter in the reference, and here unless the handle was
  // switched to the extended modes (mluOpExtSetSparseConvExtendedModes).
  PARAM_CHECK(api, inverse == 0 || (inverse == 1 && handle->sparse_conv_extended));

  STRIDE_TENSOR_CHECK(api, features_desc, "features_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, output_grad_desc, "output_grad_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, indice_pairs_desc, "indice_pairs_desc must be contiguous");
  STRIDE_TENSOR_CHECK(api, filters_grad_desc, "filters_grad_desc must be contiguous");

  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported.";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }

  mluOpStatus_t st =
      dtypeValid(api, features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc);
  if (st != MLUOP_STATUS_SUCCESS) return st;

  if (mluOpGetTensorElementNum(features_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(output_grad_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(indice_pairs_desc) >= LARGE_TENSOR_NUM ||
      mluOpGetTensorElementNum(filters_grad_desc) >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " Overflow max tensor num: tensors must hold fewer than 2^31 "
                     << "elements.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  bool shape_check = true;
  if (2 != features_desc->getDim() || 2 != output_grad_desc->getDim() ||
      3 != indice_pairs_desc->getDim() ||
      (4 != filters_grad_desc->getDim() && 5 != filters_grad_desc->getDim())) {
    shape_check = false;
  }
  if (shape_check) {
    const GradDims g = gradDims(filters_grad_desc, handle->sparse_conv_extended);
    // indice_pairs.dim[2] is the row count of the tensor pair column 0 indexes:
    // features, or output_grad of an inverse convolution.
    const mluOpTensorDescriptor_t col0_desc = inverse == 1 ? output_grad_desc : features_desc;
    if (g.ci != features_desc->getDimIndex(1) || g.co != output_grad_desc->getDimIndex(1) ||
        col0_desc->getDimIndex(0) != indice_pairs_desc->getDimIndex(2) ||
        2 != indice_pairs_desc->getDimIndex(1) || g.K != indice_pairs_desc->getDimIndex(0)) {
      shape_check = false;
    }
    PARAM_CHECK_LE(api, indice_pairs_desc->getDimIndex(2), INDICE_IN_LARGE_TENSOR_NUM);
  }
  if (!shape_check) {
    MLUOP_LOG(ERROR) << api << " Shape check failed!";
    return MLUOP_STATUS_BAD_PARAM;
  }
  return MLUOP_STATUS_SUCCESS;
}

bool anyZeroElement(const mluOpTensorDescriptor_t a, const mluOpTensorDescriptor_t b,
                    const mluOpTensorDescriptor_t c, const mluOpTensorDescriptor_t d) {
  return a->getTotalElementNum() == 0 || b->getTotalElementNum() == 0 ||
         c->getTotalElementNum() == 0 || d->getTotalElementNum() == 0;
}

ConvProblem makeProblem(mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc,
                        const mluOpTensorDescriptor_t output_grad_desc,
                        const mluOpTensorDescriptor_t indice_pairs_desc,
                        const mluOpTensorDescriptor_t filters_grad_desc,
                        const int64_t indice_num[], int64_t inverse, const void *indice_pairs) {
  ConvProblem p;
  p.dtype = toElemType(features_desc->getDtype());
  p.K = (int)indice_pairs_desc->getDimIndex(0);
  p.L = (int)indice_pairs_desc->getDimIndex(2);
  p.inverse = inverse != 0;
  p.num_out = (int)(p.inverse ? features_desc : output_grad_desc)->getDimIndex(0);
  const GradDims g = gradDims(filters_grad_desc, handle->sparse_conv_extended);
  p.grad_stride_k = g.stride_k;
  p.grad_stride_ci = g.stride_ci;
  p.grad_stride_co = g.stride_co;
  p.Ci = (int)features_desc->getDimIndex(1);
  p.Co = (int)output_grad_desc->getDimIndex(1);
  p.indice_pairs = static_cast<const int32_t *>(indice_pairs);
  p.indice_num = indice_num;
  return p;
}

}  // namespace

namespace mluop {
namespace sparse_conv {

hipError_t lookUpNoAllocScratch(int device) {
  if (device < 0 || device >= kMaxScratchDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_scratch_ptr[device] != nullptr) return hipSuccess;
  void *ptr = nullptr;
  const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (err != hipSuccess) return err;
  g_scratch_ptr[device] = ptr;
  return hipSuccess;
}

}  // namespace sparse_conv
}  // namespace mluop

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc,
    const mluOpTensorDescriptor_t output_grad_desc,
    const mluOpTensorDescriptor_t indice_pairs_desc,
    const mluOpTensorDescriptor_t filters_grad_desc, const int64_t indice_num[],
    const int64_t inverse, const int64_t subm, size_t *size) {
  const std::string api = "[mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize]";
  (void)subm;
  PARAM_CHECK(api, size != nullptr);
  mluOpStatus_t st = baseParamCheck(api, handle, features_desc, output_grad_desc,
                                    indice_pairs_desc, filters_grad_desc, indice_num, inverse);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (anyZeroElement(features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc)) {
    return MLUOP_STATUS_SUCCESS;
  }
  const ConvProblem p =
      makeProblem(handle, features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc,
                  indice_num, inverse, nullptr);
  *size = mluop::sparse_conv::backwardFilterWorkspaceBytes(p);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpIndiceConvolutionBackwardFilter(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc, const void *features,
    const mluOpTensorDescriptor_t output_grad_desc, const void *output_grad,
    const mluOpTensorDescriptor_t indice_pairs_desc, const void *indice_pairs,
    const int64_t indice_num[], const int64_t inverse, const int64_t subm, void *workspace,
    size_t workspace_size, const mluOpTensorDescriptor_t filters_grad_desc, void *filters_grad) {
  const std::string api = "[mluOpIndiceConvolutionBackwardFilter]";
  (void)subm;
  mluOpStatus_t st = baseParamCheck(api, handle, features_desc, output_grad_desc,
                                    indice_pairs_desc, filters_grad_desc, indice_num, inverse);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (anyZeroElement(features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc)) {
    return MLUOP_STATUS_SUCCESS;
  }
  PARAM_CHECK(api, features != nullptr);
  PARAM_CHECK(api, output_grad != nullptr);
  PARAM_CHECK(api, indice_pairs != nullptr);
  PARAM_CHECK(api, filters_grad != nullptr);
  if (workspace_size > 0) {
    PARAM_CHECK(api, workspace != nullptr);
  }
  const ConvProblem p =
      makeProblem(handle, features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc,
                  indice_num, inverse, indice_pairs);
  const size_t need = mluop::sparse_conv::backwardFilterWorkspaceBytes(p);
  if (workspace_size < need || (need > 0 && workspace == nullptr)) {
    MLUOP_LOG(ERROR) << api << " workspace of " << workspace_size
                     << " bytes is smaller than the " << need
                     << " bytes mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize reports.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (mluop::gen_case::mode() != 0) {
    // (reference indice_convolution_backward_filter.cpp:82-97)
    mluop::gen_case::CaseWriter c(handle, "indice_convolution_backward_filter",
                                  "indice_convolution_backward_param");
    c.input("features", features_desc, features);
    c.input("output_grad", output_grad_desc, output_grad);
    c.input("indice_pairs", indice_pairs_desc, indice_pairs);
    c.output("filters_grad", filters_grad_desc);
    c.params("indice_num", indice_num, p.K);
    c.param("sub_m", subm);
    c.param("inverse", inverse);
    c.finish(0.003);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, filters_grad, filters_grad_desc->total_tensor_size);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, workspace, workspace_size);
  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchBackwardFilter(handle->launchCtx(), p, features,
                                                                output_grad, workspace,
                                                                filters_grad));
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtIndiceConvolutionBackwardFilterNoAlloc(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc, const void *features,
    const mluOpTensorDescriptor_t output_grad_desc, const void *output_grad,
    const mluOpTensorDescriptor_t indice_pairs_desc, const void *indice_pairs,
    const int64_t indice_num[], const int64_t inverse, const int64_t subm,
    const mluOpTensorDescriptor_t filters_grad_desc, void *filters_grad) {
  const std::string api = "[mluOpExtIndiceConvolutionBackwardFilterNoAlloc]";
  (void)subm;
  mluOpStatus_t st = baseParamCheck(api, handle, features_desc, output_grad_desc,
                                    indice_pairs_desc, filters_grad_desc, indice_num, inverse);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  if (anyZeroElement(features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc)) {
    return MLUOP_STATUS_SUCCESS;
  }
  PARAM_CHECK(api, features != nullptr);
  PARAM_CHECK(api, output_grad != nullptr);
  PARAM_CHECK(api, indice_pairs != nullptr);
  PARAM_CHECK(api, filters_grad != nullptr);
  ConvProblem p =
      makeProblem(handle, features_desc, output_grad_desc, indice_pairs_desc, filters_grad_desc,
                  indice_num, inverse, indice_pairs);
  // the pair lists are cut into as many slices as the array has room for partial tiles
  p.max_partial_tiles = (int)(((size_t)MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES - 4096) /
                              ((size_t)p.Ci * p.Co * sizeof(float)));
  if (!mluop::sparse_conv::backwardFilterLaunchesOnly(p)) {
    MLUOP_LOG(ERROR) << api << " a kernel volume of " << p.K << " offsets needs a staging copy "
                     << "and a wait for the queue; use mluOpIndiceConvolutionBackwardFilter.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  const size_t need = mluop::sparse_conv::backwardFilterWorkspaceBytes(p);
  if (need > (size_t)MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES) {
    MLUOP_LOG(ERROR) << api << " this shape needs " << need << " bytes of scratch memory, the "
                     << "library holds " << (size_t)MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES
                     << "; use mluOpIndiceConvolutionBackwardFilter with a workspace.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  DEVICE_HANDLE_CHECK(api, handle);
  void *ptr = nullptr;
  if (handle->device < kMaxScratchDevices) {
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    ptr = g_scratch_ptr[handle->device];
  }
  if (ptr == nullptr) {
    MLUOP_LOG(ERROR) << api << " the scratch memory of device " << handle->device
                     << " was not found when the handle was created.";
    return MLUOP_STATUS_NOT_INITIALIZED;
  }
  // the handle's kernel choices, but no event pairs: the per-kernel timer creates events on demand
  const mluop::LaunchCtx lc(handle->queue, nullptr, &handle->kernel_choices);
  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchBackwardFilter(lc, p, features, output_grad,
                                                                ptr, filters_grad));
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
