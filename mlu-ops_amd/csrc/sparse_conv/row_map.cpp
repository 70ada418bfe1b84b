// Row maps kept across calls.  mluOpIndiceConvolutionForward and ...BackwardData turn the
// pair lists into a [K, rows] map of partner rows on every call, because the reference API
// hands them nothing else.  Layers that share a rulebook (every submanifold layer of a stage,
// and the forward and backward pass of each) can build that map once instead.
#include "sparse_conv/row_map.h"

#include "mlu_op_ext.h"

using mluop::sparse_conv::ConvProblem;
using mluop::sparse_conv::GatherDirection;
using mluop::sparse_conv::RowMapShape;

namespace mluop {
namespace sparse_conv {

mluOpStatus_t takeRowMap(const std::string &api, mluOpHandle_t handle, const void *map,
                         GatherDirection dir, ConvProblem *p) {
  if (map == nullptr) return MLUOP_STATUS_SUCCESS;
  const RowMapShape want = rowMapShape(*p, dir);
  for (const auto &r : handle->row_maps) {
    if (r.map != map) continue;
    if (r.pairs == p->indice_pairs && r.K == want.K && r.L == want.L && r.rows == want.rows &&
        r.source_rows == want.source_rows && r.row_column == want.row_column) {
      p->row_map = static_cast<const int32_t *>(map);
      return MLUOP_STATUS_SUCCESS;
    }
    MLUOP_LOG(ERROR) << api << " the row map announced by mluOpExtUseRowMap was built for another "
                     << "pair tensor, shape or direction (rows " << r.rows << ", column "
                     << r.row_column << "; this call needs rows " << want.rows << ", column "
                     << want.row_column << ").";
    return MLUOP_STATUS_BAD_PARAM;
  }
  MLUOP_LOG(ERROR) << api << " the row map announced by mluOpExtUseRowMap is not known.";
  return MLUOP_STATUS_BAD_PARAM;
}

}  // namespace sparse_conv
}  // namespace mluop

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpExtGetRowMapSize(const mluOpTensorDescriptor_t indice_pairs_desc,
                                                  int64_t rows, size_t *size) {
  const std::string api = "[mluOpExtGetRowMapSize]";
  PARAM_CHECK(api, indice_pairs_desc != NULL);
  PARAM_CHECK(api, size != NULL);
  PARAM_CHECK(api, indice_pairs_desc->dim == 3);
  PARAM_CHECK(api, indice_pairs_desc->dims[1] == 2);
  PARAM_CHECK(api, rows >= 0 && rows <= INT32_MAX);
  PARAM_CHECK(api, indice_pairs_desc->dims[0] >= 0 && indice_pairs_desc->dims[0] * rows <= INT32_MAX);
  *size = mluop::sparse_conv::rowMapBytes((int)indice_pairs_desc->dims[0], (int)rows);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtBuildRowMap(mluOpHandle_t handle,
                                                const mluOpTensorDescriptor_t indice_pairs_desc,
                                                const void *indice_pairs, const int64_t indice_num[],
                                                int64_t rows, int64_t source_rows, int row_column,
                                                void *row_map, size_t size, int64_t *lost_pairs) {
  const std::string api = "[mluOpExtBuildRowMap]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, indice_pairs_desc != NULL);
  PARAM_CHECK(api, indice_num != NULL);
  // without a place for the verdict the build neither counts nor waits: the caller's promise
  // of distinct pairs (mluOpExtSetDistinctPairsPromise) has to stand in for it
  PARAM_CHECK(api, lost_pairs != NULL || handle->distinct_pairs_promised);
  PARAM_CHECK(api, indice_pairs_desc->dim == 3);
  PARAM_CHECK(api, indice_pairs_desc->dims[1] == 2);
  PARAM_CHECK(api, indice_pairs_desc->dtype == MLUOP_DTYPE_INT32);
  PARAM_CHECK(api, row_column == 0 || row_column == 1);
  PARAM_CHECK(api, rows > 0 && rows <= INT32_MAX);
  PARAM_CHECK(api, source_rows > 0 && source_rows <= INT32_MAX);
  const int64_t K = indice_pairs_desc->dims[0], L = indice_pairs_desc->dims[2];
  PARAM_CHECK(api, K > 0 && L > 0 && L <= INT32_MAX && K * rows <= INT32_MAX);
  // the pair column that names the result rows indexes a tensor of `rows` rows: L for column 0
  PARAM_CHECK(api, (row_column == 0 ? rows : source_rows) == L);
  PARAM_CHECK(api, indice_pairs != NULL);
  PARAM_CHECK(api, row_map != NULL);
  size_t need = 0;
  mluOpStatus_t st = mluOpExtGetRowMapSize(indice_pairs_desc, rows, &need);
  if (st != MLUOP_STATUS_SUCCESS) return st;
  PARAM_CHECK(api, size >= need);
  int64_t expected = 0;
  for (int64_t k = 0; k < K; ++k) {
    PARAM_CHECK(api, indice_num[k] >= 0 && indice_num[k] <= L);
    expected += indice_num[k];
  }
  DEVICE_HANDLE_CHECK(api, handle);

  // forget what this buffer held before
  auto &maps = handle->row_maps;
  for (size_t i = 0; i < maps.size();) {
    if (maps[i].map == row_map) maps.erase(maps.begin() + i);
    else ++i;
  }
  const RowMapShape shape{(int)K, (int)L, (int)rows, (int)source_rows, row_column};
  HIP_CHECK_RETURN(api, mluop::sparse_conv::buildRowMap(
                            handle->launchCtx(), static_cast<const int32_t *>(indice_pairs), indice_num,
                            shape, row_map, lost_pairs != NULL ? handle->pinned_scalar : nullptr));
  if (lost_pairs != NULL) {
    HIP_CHECK_RETURN(api, hipStreamSynchronize(handle->queue));
    *lost_pairs = expected - (int64_t)handle->pinned_scalar[0];
  }
  if (lost_pairs == NULL || *lost_pairs == 0) {
    if (maps.size() >= 256) maps.erase(maps.begin());
    maps.push_back({row_map, indice_pairs, (int)K, (int)L, (int)rows, (int)source_rows, row_column});
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtUseRowMap(mluOpHandle_t handle, const void *row_map) {
  const std::string api = "[mluOpExtUseRowMap]";
  PARAM_CHECK(api, handle != NULL);
  if (row_map != NULL) {
    bool known = false;
    for (const auto &r : handle->row_maps) known = known || r.map == row_map;
    if (!known) {
      MLUOP_LOG(ERROR) << api << " no row map was built into this buffer on this handle, or pairs "
                       << "were lost when it was built.";
      return MLUOP_STATUS_BAD_PARAM;
    }
  }
  handle->pending_row_map = row_map;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtForgetRowMap(mluOpHandle_t handle, const void *row_map) {
  const std::string api = "[mluOpExtForgetRowMap]";
  PARAM_CHECK(api, handle != NULL);
  auto &maps = handle->row_maps;
  for (size_t i = 0; i < maps.size();) {
    if (row_map == NULL || maps[i].map == row_map) maps.erase(maps.begin() + i);
    else ++i;
  }
  if (row_map == NULL || handle->pending_row_map == row_map) handle->pending_row_map = nullptr;
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
