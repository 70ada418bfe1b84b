// Host-side interface of the indice-convolution kernel set (forward,
// backward data, backward filter).
#ifndef MLUOP_AMD_SPARSE_CONV_INDICE_CONV_H_
#define MLUOP_AMD_SPARSE_CONV_INDICE_CONV_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "core/launch.h"

namespace mluop {
namespace sparse_conv {

enum class ElemType { kHalf, kBFloat16, kFloat };

inline size_t elemSize(ElemType t) { return t == ElemType::kFloat ? 4 : 2; }

// A filter tensor seen as W(k, ci, co) = base[k*stride_k + ci*stride_ci + co*stride_co]
// (element strides), which covers every accepted filter layout without a
// transposed copy.
struct FilterView {
  const void *base;
  int64_t stride_k;
  int64_t stride_ci;
  int64_t stride_co;
};

// What the caller knows about the pair column that names a launch's result rows.
enum class ListTrust {
  kNone,     // nothing, or that it is out of order: the launch builds a row map
  kInOrder,  // it ascends inside every offset (checked again on the device)
  kUnknown,  // a rulebook of this handle whose report has not arrived: the kernels decide
};

struct ConvProblem {
  ElemType dtype;
  int K;          // kernel volume = indice_pairs.dim[0]
  int L;          // indice_pairs.dim[2] = rows of the tensor pair column 0 indexes
  int num_out;    // rows of the tensor pair column 1 indexes
  int Ci;
  int Co;
  const int32_t *indice_pairs;  // device [K, 2, L]
  const int64_t *indice_num;    // host [K]
  // Inverse convolution: the rulebook of the partner layer read backwards.
  // Pair column 0 then names rows of the output-side tensors (L of them) and
  // column 1 rows of the input-side tensors (num_out of them).
  bool inverse = false;
  // The caller promised that no offset names a result row twice: no check for lost pairs.
  bool distinct_pairs = false;
  // Forward and backward data: the [K, rows] row map of exactly this rulebook and direction,
  // built ahead by buildRowMap with no pair lost (so the pairs are distinct as well); the
  // launch then neither clears nor fills a map of its own.
  const int32_t *row_map = nullptr;
  // Forward and backward data: the caller has reason to believe (it is checked on the
  // device) that inside every offset the pair column naming the result rows ascends strictly
  // and all indices are in range, so the kernels read the lists cut by tile instead of
  // building a row map.  `ticket` is a value no earlier launch on this workspace used.
  ListTrust list_trust = ListTrust::kNone;
  unsigned long long ticket = 0;
  // Backward filter only: the most Ci x Co fp32 partial tiles the workspace may hold (0: as
  // many as the kernels like to use); the pair lists are cut into fewer, longer slices then.
  int max_partial_tiles = 0;
  // Backward filter only: element strides of dW(k, ci, co) in filters_grad;
  // all zero = the positional [K, Ci, Co].
  int64_t grad_stride_k = 0, grad_stride_ci = 0, grad_stride_co = 0;
};

// Which of the two gather-GEMM directions a launch computes.
//   kForward:      rows = output rows,  gathered = features,    B = W[k]
//   kBackwardData: rows = input rows,   gathered = output_grad, B = W[k]^T
enum class GatherDirection { kForward, kBackwardData };

size_t gatherConvWorkspaceBytes(const ConvProblem &p, GatherDirection dir);
hipError_t launchGatherConv(const LaunchCtx &lc, const ConvProblem &p, GatherDirection dir,
                            const void *gathered, const FilterView &filters, void *workspace,
                            void *result);

// A row map kept across calls: entry [k, r] is the partner row of result row r at offset k,
// or -1.  `row_column` is the pair column that names the result rows (1: the rows are what
// column 1 indexes, as in a forward convolution; 0: what column 0 indexes, as in backward
// data), `rows` / `source_rows` the row counts of the result and of the gathered tensor.
struct RowMapShape {
  int K, L, rows, source_rows, row_column;
};
// The shape a launch of `dir` over `p` needs.
RowMapShape rowMapShape(const ConvProblem &p, GatherDirection dir);
// Bytes of a map buffer: the entries, one counter, the per-offset counts.
size_t rowMapBytes(int K, int rows);
// Clears and fills `row_map` on the stream and, unless `filled_host` is null, counts the filled
// slots and copies the count to `*filled_host` (pinned memory); the caller waits for the stream
// before reading it.
hipError_t buildRowMap(const LaunchCtx &lc, const int32_t *indice_pairs, const int64_t *indice_num,
                       const RowMapShape &shape, void *row_map, int32_t *filled_host);

size_t backwardFilterWorkspaceBytes(const ConvProblem &p);
// True when launchBackwardFilter only enqueues kernels for this shape: no staging copy of the
// per-offset counts, no wait for the stream.
bool backwardFilterLaunchesOnly(const ConvProblem &p);
hipError_t launchBackwardFilter(const LaunchCtx &lc, const ConvProblem &p, const void *features,
                                const void *output_grad, void *workspace, void *filters_grad);

}  // namespace sparse_conv
}  // namespace mluop

#endif  // MLUOP_AMD_SPARSE_CONV_INDICE_CONV_H_
