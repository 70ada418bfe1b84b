// mluOpGetIndicePairs / mluOpGetIndicePairsWorkspaceSize.
//
// The parameter checks come in the order, and give the status codes, of
// reference kernels/sparse_conv/get_indice_pairs/get_indice_pairs.cpp:78-277
// (the status tables of the reference's API tests are replayed against this
// file); what follows them is the HIP rulebook kernel set.
#include <string>

#include "core/core.h"
#include "core/gen_case.h"
#include "sparse_conv/rulebook.h"
#include "sparse_conv/rulebook_notes.h"

namespace {

using mluop::sparse_conv::RulebookGeom;

// The four tensors of the operator, in the order every per-tensor check visits them.
struct RulebookTensors {
  mluOpTensorDescriptor_t all[4];
  const mluOpTensorDescriptor_t &indices = all[0];
  const mluOpTensorDescriptor_t &indice_pairs = all[1];
  const mluOpTensorDescriptor_t &out_indices = all[2];
  const mluOpTensorDescriptor_t &indice_num = all[3];

  RulebookTensors(mluOpTensorDescriptor_t a, mluOpTensorDescriptor_t b, mluOpTensorDescriptor_t c,
                  mluOpTensorDescriptor_t d)
      : all{a, b, c, d} {}
  RulebookTensors(const RulebookTensors &) = delete;
  const mluOpTensorDescriptor_t *begin() const { return all; }
  const mluOpTensorDescriptor_t *end() const { return all + 4; }
  static const char *name(int i) {
    static const char *const names[] = {"indices_desc", "indice_pairs_desc", "out_indices_desc",
                                        "indice_num_desc"};
    return names[i];
  }
  bool anyEmpty() const {
    for (const mluOpTensorDescriptor_t d : *this)
      if (mluOpGetTensorElementNum(d) == 0) return true;
    return false;
  }
};

struct Volumes {
  int64_t kernel = 1, input = 1, output = 1;  // input and output include the batch
};

// Everything that can be decided from the descriptors.  `*done` is set when the
// call has nothing left to do (an empty tensor).
mluOpStatus_t checkGeometry(const std::string &api, mluOpHandle_t handle,
                            mluOpSparseConvolutionDescriptor_t conv, const RulebookTensors &t,
                            Volumes *vol, bool *done) {
  *done = false;
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, conv != NULL);
  {
    int i = 0;
    for (const mluOpTensorDescriptor_t d : t) {
      PARAM_CHECK_V2(api, d != NULL, RulebookTensors::name(i) << " is NULL.");
      ++i;
    }
  }
  if (handle->arch != 950) {
    MLUOP_LOG(ERROR) << api << " Only gfx950 devices are supported, this handle is on gfx"
                     << handle->arch << ".";
    return MLUOP_STATUS_ARCH_MISMATCH;
  }
  // a descriptor that was never set has dimNb 0
  PARAM_CHECK(api, conv->dimNb == 5);
  const int axes = conv->dimNb - 2;

  // ranks, then the fixed extents: indices [L,4], indice_pairs [K,2,L], out_indices [M,4], indice_num [K]
  const int ranks[] = {2, 3, 2, 1};
  {
    int i = 0;
    for (const mluOpTensorDescriptor_t d : t) {
      PARAM_CHECK_V2(api, d->getDim() == ranks[i], RulebookTensors::name(i) << " has the wrong rank.");
      ++i;
    }
  }
  PARAM_CHECK(api, t.indices->getDimIndex(1) == 4);
  PARAM_CHECK(api, t.out_indices->getDimIndex(1) == 4);
  PARAM_CHECK(api, t.indice_pairs->getDimIndex(1) == 2);
  const int64_t rows = t.indices->getDimIndex(0);
  PARAM_CHECK(api, t.indice_pairs->getDimIndex(2) == rows);
  PARAM_CHECK(api, t.indice_pairs->getDimIndex(0) == t.indice_num->getDimIndex(0));

  vol->input = vol->output = conv->batch;
  for (int a = 0; a < axes; ++a) {
    vol->kernel *= conv->filter_space[a];
    vol->output *= conv->output_space[a];
    vol->input *= conv->input_space[a];
  }
  PARAM_CHECK_LE(api, rows, vol->input);
  for (int a = 0; a < axes; ++a) {
    const std::string where = "i: " + std::to_string(a) + ".";
    PARAM_CHECK_V2(api, conv->pad[a] >= 0, where);
    PARAM_CHECK_V2(api, conv->dilation[a] >= 1, where);
    PARAM_CHECK_V2(api, conv->stride[a] >= 1, where);
    if (conv->dilation[a] != 1 && conv->stride[a] != 1) {
      MLUOP_LOG(ERROR) << api << " dilation[" << a << "] and stride[" << a
                       << "] cannot both be larger than 1.";
      return MLUOP_STATUS_BAD_PARAM;
    }
  }
  PARAM_CHECK(api, t.indice_pairs->getDimIndex(0) == vol->kernel);
  PARAM_CHECK_LE(api, vol->kernel, 4096);
  PARAM_CHECK_LE(api, t.out_indices->getDimIndex(0), vol->output);

  {
    int i = 0;
    for (const mluOpTensorDescriptor_t d : t) {
      STRIDE_TENSOR_CHECK(api, d, RulebookTensors::name(i) << " must be contiguous");
      ++i;
    }
  }
  PARAM_CHECK_LE(api, rows, INDICE_IN_LARGE_TENSOR_NUM);
  for (const mluOpTensorDescriptor_t d : t) {
    if (mluOpGetTensorElementNum(d) >= LARGE_TENSOR_NUM) {
      MLUOP_LOG(ERROR) << api << " Overflow max tensor num. Tensors must hold fewer than 2^31 "
                       << "elements.";
      return MLUOP_STATUS_NOT_SUPPORTED;
    }
  }
  // Linear cell indices are 32-bit: batch * volume must stay below 2^31 (the
  // reference multiplies plain ints here without a check).
  if ((uint64_t)vol->output >= LARGE_TENSOR_NUM || (uint64_t)vol->input >= LARGE_TENSOR_NUM) {
    MLUOP_LOG(ERROR) << api << " batch * spatial volume must be smaller than 2^31.";
    return MLUOP_STATUS_NOT_SUPPORTED;
  }
  {
    int i = 0;
    for (const mluOpTensorDescriptor_t d : t) {
      PARAM_CHECK_V2(api, d->getDtype() == MLUOP_DTYPE_INT32, RulebookTensors::name(i) << " must be int32.");
      ++i;
    }
  }
  if (conv->sub_m) {
    // a submanifold rulebook keeps the input's cells: same space, unit stride and dilation
    for (int a = 0; a < axes; ++a) {
      const std::string where = "i: " + std::to_string(a) + ".";
      PARAM_CHECK_V2(api, conv->input_space[a] == conv->output_space[a], where);
      PARAM_CHECK_V2(api, conv->stride[a] == 1, where);
      PARAM_CHECK_V2(api, conv->dilation[a] == 1, where);
    }
  }
  if (t.anyEmpty()) {
    conv->num_act_out = 0;
    *done = true;
  }
  return MLUOP_STATUS_SUCCESS;
}

RulebookGeom geometryOf(const mluOpSparseConvolutionStruct *conv, const RulebookTensors &t,
                        const Volumes &vol) {
  RulebookGeom g;
  g.batch = conv->batch;
  for (int a = 0; a < 3; ++a) {
    g.in_space[a] = conv->input_space[a];
    g.out_space[a] = conv->output_space[a];
    g.ksize[a] = conv->filter_space[a];
    g.pad[a] = conv->pad[a];
    g.stride[a] = conv->stride[a];
    g.dilation[a] = conv->dilation[a];
  }
  g.K = (int)vol.kernel;
  g.L = (int)t.indices->getDimIndex(0);
  g.out_rows = (int)t.out_indices->getDimIndex(0);
  g.sub_m = conv->sub_m != 0;
  return g;
}

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpGetIndicePairs(
    mluOpHandle_t handle, const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
    const mluOpTensorDescriptor_t indices_desc, const void *indices, void *workspace,
    const size_t workspace_size, const mluOpTensorDescriptor_t indice_pairs_desc,
    void *indice_pairs, const mluOpTensorDescriptor_t out_indices_desc, void *out_indices,
    const mluOpTensorDescriptor_t indice_num_desc, void *indice_num) {
  const std::string api = "[mluOpGetIndicesPairs]";
  const RulebookTensors t(indices_desc, indice_pairs_desc, out_indices_desc, indice_num_desc);
  Volumes vol;
  bool done = false;
  const mluOpStatus_t checked = checkGeometry(api, handle, sparse_conv_desc, t, &vol, &done);
  if (checked != MLUOP_STATUS_SUCCESS || done) return checked;

  PARAM_CHECK(api, indices != NULL);
  PARAM_CHECK(api, indice_pairs != NULL);
  PARAM_CHECK(api, out_indices != NULL);
  PARAM_CHECK(api, indice_num != NULL);
  if (workspace_size != 0) {
    PARAM_CHECK(api, workspace != NULL);
  }
  const RulebookGeom g = geometryOf(sparse_conv_desc, t, vol);
  const size_t need = mluop::sparse_conv::rulebookWorkspaceBytes(g);
  if (workspace_size < need || workspace == NULL) {
    MLUOP_LOG(ERROR) << api << " workspace of " << workspace_size << " bytes is smaller than the "
                     << need << " bytes mluOpGetIndicePairsWorkspaceSize reports.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  if (mluop::gen_case::mode() != 0) {
    // (reference get_indice_pairs.cpp:47-75)
    mluop::gen_case::CaseWriter c(handle, "get_indice_pairs", "get_indice_pairs_param");
    c.input("indices", indices_desc, indices);
    c.output("out_indices", out_indices_desc);
    c.output("indice_pairs", indice_pairs_desc);
    c.output("indice_num", indice_num_desc);
    c.param("dimnb", sparse_conv_desc->dimNb);
    c.param("batch", sparse_conv_desc->batch);
    c.params("pad", sparse_conv_desc->pad, 3);
    c.params("stride", sparse_conv_desc->stride, 3);
    c.params("dilation", sparse_conv_desc->dilation, 3);
    c.params("input_space", sparse_conv_desc->input_space, 3);
    c.params("filter_space", sparse_conv_desc->filter_space, 3);
    c.params("output_space", sparse_conv_desc->output_space, 3);
    c.param("sub_m", sparse_conv_desc->sub_m);
    c.param("transpose", sparse_conv_desc->transpose);
    c.param("inverse", sparse_conv_desc->inverse);
    c.finish(0.0);
  }
  DEVICE_HANDLE_CHECK(api, handle);
  if (!g.sub_m) {
    // Regular mode hands the number of output rows to the host descriptor and has to wait for
    // it: nothing a graph can record.  Refused before anything is enqueued, so that the
    // caller's capture stays valid.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    HIP_CHECK_RETURN(api, hipStreamIsCapturing(handle->queue, &capturing));
    if (capturing != hipStreamCaptureStatusNone) {
      MLUOP_LOG(ERROR) << api << " the handle's queue is being captured into a graph, and a rulebook that is not "
                       << "submanifold waits for its output row count: build it outside the capture.";
      return MLUOP_STATUS_NOT_SUPPORTED;
    }
  }

  const int32_t *in_rows = static_cast<const int32_t *>(indices);
  int32_t *pairs = static_cast<int32_t *>(indice_pairs);
  int32_t *out_rows = static_cast<int32_t *>(out_indices);
  int32_t *counts = static_cast<int32_t *>(indice_num);
  // the other outputs and the workspace are no pair tensors any more, whatever was noted there
  mluop::sparse_conv::forgetRulebookNotesIn(handle, out_indices, out_indices_desc->total_tensor_size);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, indice_num, indice_num_desc->total_tensor_size);
  mluop::sparse_conv::forgetRulebookNotesIn(handle, workspace, workspace_size);
  const mluop::sparse_conv::RulebookReportTarget report =
      mluop::sparse_conv::openRulebookNote(handle, indice_pairs, g.K, g.L);
  if (g.sub_m) {
    // Submanifold mode leaves num_act_out untouched, as the reference does
    // (normal_get_indice_pairs.cpp:848-975): the caller uses the input row count.
    HIP_CHECK_RETURN(api, mluop::sparse_conv::launchSubmRulebook(handle->launchCtx(), g, in_rows, workspace,
                                                                 pairs, out_rows, counts, report));
    return MLUOP_STATUS_SUCCESS;
  }
  HIP_CHECK_RETURN(api, mluop::sparse_conv::launchRegularRulebook(handle->launchCtx(), g, in_rows, workspace,
                                                                  pairs, out_rows, counts,
                                                                  handle->pinned_scalar, handle->readback_event,
                                                                  report));
  // The output row count travels back through the host descriptor, which needs one wait
  // (the reference waits for its queue at normal_get_indice_pairs.cpp:531-533): here for the
  // kernel that numbers the output cells; the one that writes the pair lists runs on behind
  // it, in queue order like everything the caller enqueues next.
  HIP_CHECK_RETURN(api, hipEventSynchronize(handle->readback_event));
  const int num_act_out = handle->pinned_scalar[0];
  sparse_conv_desc->num_act_out = num_act_out;
  if (num_act_out > g.out_rows) {
    MLUOP_LOG(ERROR) << api << " out_indices holds " << g.out_rows << " rows but " << num_act_out
                     << " output cells are active; rows beyond the tensor were dropped.";
    return MLUOP_STATUS_BAD_PARAM;
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetIndicePairsWorkspaceSize(
    mluOpHandle_t handle, const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
    const mluOpTensorDescriptor_t indices_desc, const mluOpTensorDescriptor_t indice_pairs_desc,
    const mluOpTensorDescriptor_t out_indices_desc, const mluOpTensorDescriptor_t indice_num_desc,
    size_t *workspace_size) {
  const std::string api = "[mluOpGetIndicePairsWorkspaceSize]";
  const RulebookTensors t(indices_desc, indice_pairs_desc, out_indices_desc, indice_num_desc);
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, sparse_conv_desc != NULL);
  {
    int i = 0;
    for (const mluOpTensorDescriptor_t d : t) {
      PARAM_CHECK_V2(api, d != NULL, RulebookTensors::name(i) << " is NULL.");
      ++i;
    }
  }
  PARAM_CHECK(api, workspace_size != NULL);
  // an empty tensor needs no workspace, whatever else the descriptors say
  if (t.anyEmpty()) {
    *workspace_size = 0;
    return MLUOP_STATUS_SUCCESS;
  }
  Volumes vol;
  bool done = false;
  const mluOpStatus_t checked = checkGeometry(api, handle, sparse_conv_desc, t, &vol, &done);
  if (checked != MLUOP_STATUS_SUCCESS) return checked;
  *workspace_size = mluop::sparse_conv::rulebookWorkspaceBytes(geometryOf(sparse_conv_desc, t, vol));
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
