/* CPU oracle for dynamic point-to-voxel scatter, forward (TEST INFRASTRUCTURE,
 * not product code).
 *
 * Plain-C restatement of the reference gtest executor's cpuCompute
 * (test/mlu_op_gtest/pb_gtest/src/zoo/dynamic_point_to_voxel_forward/
 *  dynamic_point_to_voxel_forward.cpp:107-252):
 *   rows with a negative coordinate become (-1,-1,-1)        :135-143
 *   points sorted by coordinate triple, unique triples       :145-182
 *   voxel_num, voxel_coors (the -1 triple is not a voxel)    :184-196
 *   point2voxel_map                                          :198-209
 *   voxel_points_count                                       :211-230
 *   voxel_feats: max, or mean as sum of feats/count in point order :232-262
 * Rows of the outputs past voxel_num keep the fill the operator gives them
 * (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_forward/
 *  dynamic_point_to_voxel_forward.cpp:343-358: -inf for max, 0 for mean;
 *  coordinates and counts 0).
 *
 * Pinned by tests/test_oracle_dynamic_point_to_voxel.py against the two case
 * files the reference ships for this operator (tests/golden/
 * dynamic_point_to_voxel_forward/case_0.prototxt, case_1.prototxt) and an
 * independent numpy.unique formulation.
 *
 * oracle_dynamic_point_to_voxel_backward restates the backward executor
 * (test/mlu_op_gtest/pb_gtest/src/zoo/dynamic_point_to_voxel_backward/
 *  dynamic_point_to_voxel_backward.cpp:108-166, max reduction only) and is
 * pinned by the reference's case file for it (tests/golden/
 * dynamic_point_to_voxel_backward/case_1.prototxt) and by round trips through
 * the forward oracle.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static const int32_t *g_coors;

static int cmp_rows(const void *a, const void *b) {
  const int32_t *x = g_coors + 3 * (size_t)(*(const int32_t *)a);
  const int32_t *y = g_coors + 3 * (size_t)(*(const int32_t *)b);
  for (int k = 0; k < 3; ++k) {
    if (x[k] < y[k]) return -1;
    if (x[k] > y[k]) return 1;
  }
  /* equal triples: by point index, which makes the order total (the reference's
   * std::sort leaves it open; nothing below depends on it) */
  return (*(const int32_t *)a > *(const int32_t *)b) - (*(const int32_t *)a < *(const int32_t *)b);
}

static int same_row(const int32_t *c, int32_t i, int32_t j) {
  return c[3 * (size_t)i] == c[3 * (size_t)j] && c[3 * (size_t)i + 1] == c[3 * (size_t)j + 1] &&
         c[3 * (size_t)i + 2] == c[3 * (size_t)j + 2];
}

/* reduce_max != 0: max, else mean.  coors [n,3] is modified in place as the
 * operator does.  Outputs have `m` rows (m >= number of voxels). */
int32_t oracle_dynamic_point_to_voxel_forward(int32_t reduce_max, const float *feats, int32_t *coors,
                                              int32_t n, int32_t c, int32_t m, float *voxel_feats,
                                              int32_t *voxel_coors, int32_t *point2voxel_map,
                                              int32_t *voxel_points_count, int32_t *voxel_num) {
  const float fill = reduce_max ? -INFINITY : 0.f;
  for (size_t i = 0; i < (size_t)m * c; ++i) voxel_feats[i] = fill;
  memset(voxel_coors, 0, sizeof(int32_t) * 3 * (size_t)m);
  memset(voxel_points_count, 0, sizeof(int32_t) * (size_t)m);
  *voxel_num = 0;
  if (n == 0 || c == 0) return 0;

  for (int32_t i = 0; i < n; ++i) {
    int32_t *r = coors + 3 * (size_t)i;
    if (r[0] < 0 || r[1] < 0 || r[2] < 0) r[0] = r[1] = r[2] = -1;
  }
  int32_t *order = (int32_t *)malloc(sizeof(int32_t) * (size_t)n);
  if (!order) return -1;
  for (int32_t i = 0; i < n; ++i) order[i] = i;
  g_coors = coors;
  qsort(order, (size_t)n, sizeof(int32_t), cmp_rows);

  const int32_t flag = coors[3 * (size_t)order[0]] == -1;  /* the -1 triple sorts first */
  int32_t id = 0;                                          /* index among unique triples */
  for (int32_t p = 0; p < n; ++p) {
    if (p > 0 && !same_row(coors, order[p], order[p - 1])) ++id;
    const int32_t v = id - flag;
    point2voxel_map[order[p]] = v;
    if (v >= 0 && v < m) {
      if (voxel_points_count[v] == 0) memcpy(voxel_coors + 3 * (size_t)v, coors + 3 * (size_t)order[p], 12);
      voxel_points_count[v] += 1;
    }
  }
  *voxel_num = id + 1 - flag;
  free(order);

  for (int32_t i = 0; i < n; ++i) {
    const int32_t v = point2voxel_map[i];
    if (v == -1 || v >= m) continue;
    const float *src = feats + (size_t)i * c;
    float *dst = voxel_feats + (size_t)v * c;
    if (reduce_max) {
      for (int32_t j = 0; j < c; ++j)
        if (src[j] >= dst[j]) dst[j] = src[j];
    } else {
      const int32_t count = voxel_points_count[v];
      for (int32_t j = 0; j < c; ++j) dst[j] += src[j] / count;
    }
  }
  return 0;
}

/* The gradient of a voxel's maximum goes to the first point (lowest index) whose
 * feature equals it; everything else is zero.  A (voxel, feature) no point of
 * which matches gives its gradient to nobody: the operator's scatter drops the
 * out-of-range index it leaves there
 * (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_backward/
 *  dynamic_point_to_voxel_backward.cpp:272-330), where the gtest body would write
 * past the end of grad_feats.  voxel rows: `m` in the tensors, `voxel_num` used. */
int32_t oracle_dynamic_point_to_voxel_backward(const float *grad_voxel_feats, const float *feats,
                                               const float *voxel_feats,
                                               const int32_t *point2voxel_map, int32_t voxel_num,
                                               int32_t n, int32_t c, int32_t m, float *grad_feats) {
  memset(grad_feats, 0, sizeof(float) * (size_t)n * c);
  if (voxel_num > m) voxel_num = m;
  if (n == 0 || c == 0 || voxel_num <= 0) return 0;
  int32_t *from = (int32_t *)malloc(sizeof(int32_t) * (size_t)voxel_num * c);
  if (!from) return -1;
  for (size_t i = 0; i < (size_t)voxel_num * c; ++i) from[i] = n;
  for (int32_t x = 0; x < n; ++x) {
    const int32_t v = point2voxel_map[x];
    if (v < 0 || v >= voxel_num) continue;
    for (int32_t j = 0; j < c; ++j)
      if (feats[(size_t)x * c + j] == voxel_feats[(size_t)v * c + j] && x < from[(size_t)v * c + j])
        from[(size_t)v * c + j] = x;
  }
  for (int32_t v = 0; v < voxel_num; ++v)
    for (int32_t j = 0; j < c; ++j) {
      const int32_t x = from[(size_t)v * c + j];
      if (x < n) grad_feats[(size_t)x * c + j] = grad_voxel_feats[(size_t)v * c + j];
    }
  free(from);
  return 0;
}
