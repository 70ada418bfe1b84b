// Host-side interface of the rulebook (indice pairs) kernel set.
#ifndef MLUOP_AMD_SPARSE_CONV_RULEBOOK_H_
#define MLUOP_AMD_SPARSE_CONV_RULEBOOK_H_

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "core/launch.h"

namespace mluop {
namespace sparse_conv {

// Geometry of one sparse convolution, axes in (d, h, w) order.
struct RulebookGeom {
  int batch;
  int in_space[3];
  int out_space[3];
  int ksize[3];
  int pad[3];
  int stride[3];
  int dilation[3];
  int K;         // kernel volume
  int L;         // active input rows
  int out_rows;  // rows of the caller's out_indices tensor (M)
  bool sub_m;
};

// Where the last kernel of a rulebook reports (pinned host memory, written from the device):
// whether the input rows were strictly ascending in (n, d, h, w) order, then the stamp that
// tells the host the report is the one it waits for.  Null words: no report.
struct RulebookReportTarget {
  unsigned long long *stamp_word = nullptr;
  unsigned int *order_word = nullptr;
  // A value no earlier rulebook of any handle used (never 0); also marks this call's words
  // in the workspace, so it is set whether or not a report is wanted.
  unsigned long long stamp = 0;
};

// Bytes of device workspace the kernel set needs for this geometry.
size_t rulebookWorkspaceBytes(const RulebookGeom &g);

// Enqueues submanifold rulebook construction on the context's stream.
hipError_t launchSubmRulebook(const LaunchCtx &lc, const RulebookGeom &g, const int32_t *indices,
                              void *workspace, int32_t *indice_pairs, int32_t *out_indices,
                              int32_t *indice_num, const RulebookReportTarget &report);

// Enqueues regular (strided / dilated) rulebook construction.  The kernel that numbers the
// output cells stores their count into `host_num_act_out` (pinned host memory) and
// `count_ready` is recorded behind it: the caller waits for that event before reading the
// count, while the kernel that writes the pair lists may still be running.
hipError_t launchRegularRulebook(const LaunchCtx &lc, const RulebookGeom &g,
                                 const int32_t *indices, void *workspace, int32_t *indice_pairs,
                                 int32_t *out_indices, int32_t *indice_num,
                                 int32_t *host_num_act_out, hipEvent_t count_ready,
                                 const RulebookReportTarget &report);

}  // namespace sparse_conv
}  // namespace mluop

#endif  // MLUOP_AMD_SPARSE_CONV_RULEBOOK_H_
