/* CPU oracle for hard voxelization (TEST INFRASTRUCTURE, not product code).
 *
 * Plain-C restatement of the reference gtest executor's cpuCompute for
 * mluOpVoxelization, deterministic mode
 * (test/mlu_op_gtest/pb_gtest/src/zoo/voxelization/voxelization.cpp):
 *   cell of every point            :121-149 (dynamicVoxelize)
 *   position of a point in its cell:151-192 (pointToVoxelidx)
 *   voxel numbering, point counts  :194-221 (determinVoxelNum)
 *   copying points and coordinates :223-256 (assignPointToVoxel, assignVoxelCoors)
 *   grid extents and the sequence  :258-320 (deterministic_hard_voxelize)
 * The outputs start from zero, as the operator fills them
 * (kernels/voxelization/voxelization.cpp:283-309).  The quadratic search for
 * earlier points of the same cell is kept as the reference has it.
 *
 * Pinned by tests/test_oracle_voxelization.py: hand-worked cases, an
 * independent sort-based numpy formulation, and invariants.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* voxelization.cpp:121-149.  coors rows are (z, y, x); a point outside the
 * range gets -1 in its first component (the reference leaves the others
 * unset there; they are set to -1 here and never read). */
/* The reference converts floorf() straight to int32_t, which is undefined in C
 * for NaN and for values outside the int range; x86 gives INT_MIN there, which
 * the range test then rejects.  That outcome is spelled out here. */
static int cell_index(float p, float lo, float size, int32_t grid, int32_t *out) {
  const float f = floorf((p - lo) / size);
  if (!(f >= -2147483648.f && f < 2147483648.f)) return 0;
  const int32_t c = (int32_t)f;
  if (c < 0 || c >= grid) return 0;
  *out = c;
  return 1;
}

static void dynamic_voxelize(const float *points, int32_t *coors, const float *voxel_size,
                             const float *range, const int32_t grid[3], int64_t num_points,
                             int64_t num_features) {
  for (int64_t i = 0; i < num_points; ++i) {
    const float *p = points + i * num_features;
    int32_t *c = coors + i * 3;
    int32_t cx, cy, cz;
    c[0] = c[1] = c[2] = -1;
    if (!cell_index(p[0], range[0], voxel_size[0], grid[0], &cx)) continue;
    if (!cell_index(p[1], range[1], voxel_size[1], grid[1], &cy)) continue;
    if (!cell_index(p[2], range[2], voxel_size[2], grid[2], &cz)) continue;
    c[0] = cz;
    c[1] = cy;
    c[2] = cx;
  }
}

/* voxelization.cpp:151-192 */
static void point_to_voxelidx(const int32_t *coors, int32_t *pt_voxelidx, int32_t *pt_pointidx,
                              int32_t max_points, int64_t num_points) {
  for (int64_t i = 0; i < num_points; ++i) {
    const int32_t *c = coors + i * 3;
    if (c[0] == -1) {
      pt_pointidx[i] = -1;
      pt_voxelidx[i] = -1;
      continue;
    }
    int32_t num = 0;
    for (int64_t j = 0; j < i; ++j) {
      const int32_t *q = coors + j * 3;
      if (q[0] == -1) continue;
      if (q[0] == c[0] && q[1] == c[1] && q[2] == c[2]) {
        ++num;
        if (num == 1) {
          pt_pointidx[i] = (int32_t)j;
        } else if (num >= max_points) {
          break;
        }
      }
    }
    if (num == 0) pt_pointidx[i] = (int32_t)i;
    pt_voxelidx[i] = num < max_points ? num : -1;
  }
}

/* voxelization.cpp:194-221 */
static void determine_voxel_num(int32_t *num_points_per_voxel, const int32_t *pt_voxelidx,
                                const int32_t *pt_pointidx, int32_t *coor_voxelidx,
                                int32_t *voxel_num, int32_t max_voxels, int64_t num_points) {
  for (int64_t i = 0; i < num_points; ++i) {
    const int32_t pos = pt_voxelidx[i];
    coor_voxelidx[i] = -1;
    if (pos == -1) {
      continue;
    } else if (pos == 0) {
      const int32_t v = *voxel_num;
      if (v >= max_voxels) continue;
      *voxel_num += 1;
      coor_voxelidx[i] = v;
      num_points_per_voxel[v] = 1;
    } else {
      const int32_t v = coor_voxelidx[pt_pointidx[i]];
      if (v != -1) {
        coor_voxelidx[i] = v;
        num_points_per_voxel[v] += 1;
      }
    }
  }
}

/* Returns 0, or -1 when memory runs out.  voxels [max_voxels, max_points, F],
 * coors [max_voxels, 3], num_points_per_voxel [max_voxels], voxel_num [1]. */
int32_t oracle_voxelization(const float *points, const float *voxel_size, const float *coors_range,
                            int64_t num_points, int64_t num_features, int32_t max_points,
                            int32_t max_voxels, float *voxels, int32_t *coors,
                            int32_t *num_points_per_voxel, int32_t *voxel_num) {
  /* voxelization.cpp:274-276: float quotient, rounded half away from zero */
  int32_t grid[3];
  for (int a = 0; a < 3; ++a)
    grid[a] = (int32_t)round((coors_range[3 + a] - coors_range[a]) / voxel_size[a]);

  memset(voxels, 0, sizeof(float) * (size_t)max_voxels * max_points * num_features);
  memset(coors, 0, sizeof(int32_t) * (size_t)max_voxels * 3);
  memset(num_points_per_voxel, 0, sizeof(int32_t) * (size_t)max_voxels);
  *voxel_num = 0;
  if (num_points == 0 || max_points == 0 || max_voxels == 0) return 0;

  int32_t *temp_coors = (int32_t *)malloc(sizeof(int32_t) * num_points * 3);
  int32_t *pt_pointidx = (int32_t *)malloc(sizeof(int32_t) * num_points);
  int32_t *pt_voxelidx = (int32_t *)malloc(sizeof(int32_t) * num_points);
  int32_t *coor_voxelidx = (int32_t *)malloc(sizeof(int32_t) * num_points);
  if (!temp_coors || !pt_pointidx || !pt_voxelidx || !coor_voxelidx) {
    free(temp_coors); free(pt_pointidx); free(pt_voxelidx); free(coor_voxelidx);
    return -1;
  }
  dynamic_voxelize(points, temp_coors, voxel_size, coors_range, grid, num_points, num_features);
  point_to_voxelidx(temp_coors, pt_voxelidx, pt_pointidx, max_points, num_points);
  determine_voxel_num(num_points_per_voxel, pt_voxelidx, pt_pointidx, coor_voxelidx, voxel_num,
                      max_voxels, num_points);
  /* voxelization.cpp:223-256 */
  for (int64_t i = 0; i < num_points; ++i) {
    const int32_t num = pt_voxelidx[i];
    const int32_t v = coor_voxelidx[i];
    if (num > -1 && v > -1) {
      memcpy(voxels + ((size_t)v * max_points + num) * num_features, points + i * num_features,
             sizeof(float) * num_features);
      if (num == 0) memcpy(coors + (size_t)v * 3, temp_coors + i * 3, sizeof(int32_t) * 3);
    }
  }
  free(temp_coors); free(pt_pointidx); free(pt_voxelidx); free(coor_voxelidx);
  return 0;
}
