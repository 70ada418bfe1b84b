/*
 * sparse_conv_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded CPU restatement of the reference's own oracle for
 * the sparse-convolution path: the `cpuCompute` bodies of the four gtest
 * executors under reference test/mlu_op_gtest/pb_gtest/src/zoo/ plus the
 * harness's dtype round trips and diff metrics.  Only tests/, the smoke check
 * and the benchmark's cpu_baseline leg may load this file's library; the
 * product library never links or calls it.
 *
 * The reference's gtest binary cannot be built here (it needs cnrt.h, cnnl.h,
 * protobuf-generated headers and googletest), so this file restates the
 * algorithm: same loop order, same dense output grid, same fp32 accumulation.
 *
 * Parity pins (tests/test_oracle_*.py): brute force over tiny grids, closed
 * forms on full blocks, subm symmetry, dense torch conv3d / autograd in fp64,
 * adjoint identities, numpy float16 for the casts, closed forms for the
 * metrics.  No function below is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------
 * Rulebook.  reference zoo/get_indice_pairs/get_indice_pairs.cpp:177-406
 * ---------------------------------------------------------------------- */

/* getValidOutPos, reference :234-286.  For one input position enumerates the
 * output positions it contributes to, with the kernel offset of each.
 * `out` holds rows of (ndim + 1) ints: the output position, then the offset. */
static int valid_out_pos(const int32_t *input_pos, const int32_t *kernel_size,
                         const int32_t *pad, const int32_t *stride, const int32_t *dilation,
                         const int32_t *out_space, int32_t *out, int ndim) {
  int32_t lowers[3], uppers[3], counter[3], counter_size[3];
  int32_t point_counter = 0, num_points = 1;
  for (int i = 0; i < ndim; ++i) {
    lowers[i] = (input_pos[i] - (kernel_size[i] - 1) * dilation[i] - 1 + stride[i] + pad[i]) /
                stride[i];
    uppers[i] = (input_pos[i] + pad[i]) / stride[i];
  }
  for (int i = 0; i < ndim; ++i) {
    counter_size[i] = (uppers[i] - lowers[i]) / dilation[i] + 1;
    num_points *= counter_size[i];
  }
  for (int i = 0; i < ndim; ++i) counter[i] = 0;
  for (int i = 0; i < num_points; ++i) {
    int valid = 1;
    int32_t m = 1, offset = 0;
    for (int j = ndim - 1; j >= 0; --j) {
      int32_t val = uppers[j] - counter[j] * dilation[j];
      out[point_counter * (ndim + 1) + j] = val;
      if (val < 0 || val > out_space[j] - 1) valid = 0;
      offset += m * (input_pos[j] - val * stride[j] + pad[j]) / dilation[j];
      m *= kernel_size[j];
    }
    out[point_counter * (ndim + 1) + ndim] = offset;
    if (valid) point_counter++;
    counter[ndim - 1] += 1;
    for (int c = ndim - 1; c >= 0; --c) {
      if (counter[c] == counter_size[c] && c > 0) {
        counter[c - 1] += 1;
        counter[c] = 0;
      }
    }
  }
  return point_counter;
}

static int32_t linear_index(const int32_t *pos, const int32_t *space, int ndim) {
  int32_t r = 0, s = 1;
  for (int k = ndim - 1; k >= 0; --k) {
    r += pos[k] * s;
    s *= space[k];
  }
  return r;
}

static int cmp_int32(const void *a, const void *b) {
  int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
  return (x > y) - (x < y);
}

/* cpuCompute + cpuGetIndicePairs, reference :177-232 and :288-406.
 *   indices      [L, 4]  (n, d, h, w)
 *   indice_pairs [K, 2, L], out_indices [out_rows, 4], indice_num [K]
 * Returns the number of active outputs (L in submanifold mode), or -1 when
 * memory runs out.  `exact_count` != 0 replaces the reference's
 * "distinct values minus one sentinel" (:380) by the true distinct count; the
 * two differ only when every (input, offset) combination is valid. */
int32_t oracle_get_indice_pairs(const int32_t *indices, int32_t L, int32_t batch,
                                const int32_t *pad, const int32_t *stride,
                                const int32_t *dilation, const int32_t *filter_space,
                                const int32_t *out_space, int32_t sub_m, int32_t out_rows,
                                int32_t exact_count, int32_t *indice_pairs,
                                int32_t *out_indices, int32_t *indice_num) {
  const int ndim = 3;
  int32_t spatial = 1, K = 1;
  for (int i = 0; i < ndim; ++i) {
    spatial *= out_space[i];
    K *= filter_space[i];
  }
  const int64_t grid_size = (int64_t)batch * spatial;
  int32_t *grid = (int32_t *)malloc(sizeof(int32_t) * (size_t)(grid_size > 0 ? grid_size : 1));
  int32_t *points = (int32_t *)malloc(sizeof(int32_t) * (size_t)K * (ndim + 1));
  int32_t *cand = (int32_t *)malloc(sizeof(int32_t) * (size_t)K * (size_t)(L > 0 ? L : 1));
  if (!grid || !points || !cand) {
    free(grid); free(points); free(cand);
    return -1;
  }
  /* initial values, reference :186-202 */
  for (int64_t i = 0; i < grid_size; ++i) grid[i] = -1;
  for (int64_t i = 0; i < (int64_t)K * 2 * L; ++i) indice_pairs[i] = -1;
  for (int32_t i = 0; i < K; ++i) indice_num[i] = 0;
  for (int64_t i = 0; i < (int64_t)out_rows * 4; ++i) out_indices[i] = -1;
  const int32_t sentinel = batch * spatial + 1; /* reference :315-318 */
  for (int64_t i = 0; i < (int64_t)K * L; ++i) cand[i] = sentinel;

  int32_t num_act_out = 0;
  if (sub_m) { /* reference :331-342 */
    for (int32_t j = 0; j < L; ++j) {
      const int32_t *row = indices + (size_t)j * 4;
      int32_t index = linear_index(row + 1, out_space, ndim) + spatial * row[0];
      grid[index] = j; /* last writer wins */
    }
    for (int64_t j = 0; j < (int64_t)L * 4 && j < (int64_t)out_rows * 4; ++j)
      out_indices[j] = indices[j];
    num_act_out = L;
  }

  for (int32_t j = 0; j < L; ++j) { /* reference :344-370 */
    const int32_t *row = indices + (size_t)j * 4;
    const int32_t batch_idx = row[0];
    const int n_valid = valid_out_pos(row + 1, filter_space, pad, stride, dilation, out_space,
                                      points, ndim);
    for (int i = 0; i < n_valid; ++i) {
      const int32_t *pt = points + i * (ndim + 1);
      const int32_t offset = pt[ndim];
      const int32_t index = linear_index(pt, out_space, ndim) + spatial * batch_idx;
      if (sub_m) {
        if (grid[index] > -1) {
          const int32_t old = indice_num[offset]++;
          indice_pairs[(size_t)offset * 2 * L + old] = j;
          indice_pairs[(size_t)offset * 2 * L + L + old] = grid[index];
        }
      } else {
        const int32_t old = indice_num[offset]++;
        indice_pairs[(size_t)offset * 2 * L + old] = j;
        indice_pairs[(size_t)offset * 2 * L + L + old] = index;
        cand[(size_t)offset * L + old] = index;
      }
    }
  }

  if (!sub_m) { /* reference :372-403 */
    const size_t n = (size_t)K * L;
    qsort(cand, n, sizeof(int32_t), cmp_int32);
    size_t uniq = 0;
    for (size_t i = 0; i < n; ++i) {
      if (i == 0 || cand[i] != cand[i - 1]) cand[uniq++] = cand[i];
    }
    if (exact_count) {
      num_act_out = (int32_t)uniq;
      if (uniq > 0 && cand[uniq - 1] == sentinel) num_act_out -= 1;
    } else {
      num_act_out = (int32_t)uniq - 1;
    }
    for (int32_t j = 0; j < num_act_out; ++j) {
      int32_t index = cand[j];
      grid[index] = j;
      if (j < out_rows) {
        int32_t *o = out_indices + (size_t)j * 4;
        o[0] = index / spatial;
        index -= o[0] * spatial;
        o[1] = index / (out_space[2] * out_space[1]);
        index -= o[1] * (out_space[2] * out_space[1]);
        o[2] = index / out_space[2];
        index -= o[2] * out_space[2];
        o[3] = index;
      }
    }
    for (int32_t j = 0; j < L; ++j) {
      for (int32_t k = 0; k < K; ++k) {
        int32_t *slot = indice_pairs + (size_t)k * 2 * L + L + j;
        if (*slot > -1) *slot = grid[*slot];
      }
    }
  }
  free(grid);
  free(points);
  free(cand);
  return num_act_out;
}

/* ------------------------------------------------------------------------
 * Forward.  reference zoo/indice_convolution_forward/
 * indice_convolution_forward.cpp:86-176.  `filters` is [K, Ci, Co] (the
 * reference transposes other layouts to this one first, :101-141).
 * ---------------------------------------------------------------------- */
void oracle_indice_conv_forward(const float *features, const float *filters,
                                const int32_t *indice_pairs, const int64_t *indice_num,
                                int64_t L, int64_t K, int64_t ci, int64_t co, int64_t num_act_out,
                                float *features_out) {
  memset(features_out, 0, sizeof(float) * (size_t)(num_act_out * co));
  for (int64_t k = 0; k < K; ++k) {
    for (int64_t p = 0; p < indice_num[k]; ++p) {
      const int64_t in = indice_pairs[k * 2 * L + p];
      const int64_t out = indice_pairs[k * 2 * L + L + p];
      if (out < 0 || in < 0) continue;
      for (int64_t c = 0; c < ci; ++c) {
        const float x = features[in * ci + c];
        const float *w = filters + k * ci * co + c * co;
        float *o = features_out + out * co;
        for (int64_t d = 0; d < co; ++d) o[d] += x * w[d];
      }
    }
  }
}

/* The layout transposes the executors apply before computing
 * (forward :119-141, backward data cpuTransposeFilter :178-252): any accepted
 * filter layout -> [K, Ci, Co].  layout: 0 NCHW, 1 NHWC, 2 HWCN, 3 NDHWC,
 * 4 ARRAY, 5 NCDHW (values of mluOpTensorLayout_t). */
void oracle_filters_to_kcico(const float *filters, int32_t layout, int64_t K, int64_t ci,
                             int64_t co, float *out) {
  int64_t sk, sci, sco;
  if (layout == 1 || layout == 3) {        /* N(D)HWC: [Co, K, Ci] */
    sk = ci; sci = 1; sco = K * ci;
  } else if (layout == 0 || layout == 5) { /* NC(D)HW: [Co, Ci, K] */
    sk = 1; sci = K; sco = ci * K;
  } else {                                 /* (D)HWCN / ARRAY: [K, Ci, Co] */
    sk = ci * co; sci = co; sco = 1;
  }
  for (int64_t k = 0; k < K; ++k)
    for (int64_t c = 0; c < ci; ++c)
      for (int64_t d = 0; d < co; ++d)
        out[k * ci * co + c * co + d] = filters[k * sk + c * sci + d * sco];
}

/* ------------------------------------------------------------------------
 * Backward data.  reference zoo/indice_convolution_backward_data/
 * indice_convolution_backward_data.cpp:254-343, float branch (:318-320).
 * `filters` is [K, Ci, Co].
 * ---------------------------------------------------------------------- */
void oracle_indice_conv_backward_data(const float *output_grad, const float *filters,
                                      const int32_t *indice_pairs, const int64_t *indice_num,
                                      int64_t L, int64_t K, int64_t ci, int64_t co,
                                      float *input_grad) {
  for (int64_t i = 0; i < L * ci; ++i) input_grad[i] = 0.f;
  for (int64_t k = 0; k < K; ++k) {
    const float *sub_filter = filters + k * ci * co;
    for (int64_t l = 0; l < indice_num[k]; ++l) {
      const int64_t in = indice_pairs[k * 2 * L + l];
      const int64_t out = indice_pairs[k * 2 * L + L + l];
      if (in < 0 || out < 0) continue;
      float *dx = input_grad + in * ci;
      const float *dy = output_grad + out * co;
      for (int64_t c = 0; c < ci; ++c) {
        float acc = 0.f;
        for (int64_t d = 0; d < co; ++d) acc += dy[d] * sub_filter[c * co + d];
        dx[c] += acc;
      }
    }
  }
}

/* ------------------------------------------------------------------------
 * Backward filter.  reference zoo/indice_convolution_backward_filter/
 * indice_convolution_backward_filter.cpp:121-178.  K comes from the pair
 * tensor, as in the device code, not from layout getters.  Output [K, Ci, Co].
 * ---------------------------------------------------------------------- */
void oracle_indice_conv_backward_filter(const float *features, const float *output_grad,
                                        const int32_t *indice_pairs, const int64_t *indice_num,
                                        int64_t L, int64_t K, int64_t ci, int64_t co,
                                        float *filters_grad) {
  for (int64_t k = 0; k < K; ++k) {
    for (int64_t c = 0; c < ci; ++c) {
      for (int64_t d = 0; d < co; ++d) {
        float s = 0.f;
        for (int64_t p = 0; p < indice_num[k]; ++p) {
          const int64_t in = indice_pairs[k * 2 * L + p];
          const int64_t out = indice_pairs[k * 2 * L + L + p];
          if (in < 0 || out < 0) continue;
          s += features[in * ci + c] * output_grad[out * co + d];
        }
        filters_grad[k * ci * co + c * co + d] = s;
      }
    }
  }
}

/* Same sums with the pair loop outermost: identical per-element summation
 * order (ascending p), far fewer cache misses.  Used as the timed CPU
 * baseline for large cases; tests check it equals the function above. */
void oracle_indice_conv_backward_filter_fast(const float *features, const float *output_grad,
                                             const int32_t *indice_pairs,
                                             const int64_t *indice_num, int64_t L, int64_t K,
                                             int64_t ci, int64_t co, float *filters_grad) {
  for (int64_t i = 0; i < K * ci * co; ++i) filters_grad[i] = 0.f;
  for (int64_t k = 0; k < K; ++k) {
    float *g = filters_grad + k * ci * co;
    for (int64_t p = 0; p < indice_num[k]; ++p) {
      const int64_t in = indice_pairs[k * 2 * L + p];
      const int64_t out = indice_pairs[k * 2 * L + L + p];
      if (in < 0 || out < 0) continue;
      const float *x = features + in * ci;
      const float *dy = output_grad + out * co;
      for (int64_t c = 0; c < ci; ++c) {
        const float xv = x[c];
        for (int64_t d = 0; d < co; ++d) g[c * co + d] += xv * dy[d];
      }
    }
  }
}

/* ------------------------------------------------------------------------
 * dtype round trips of the harness.
 * fp32 -> fp16: reference pb_gtest/src/tools.cpp:460-505 (round to nearest
 * even; finite values beyond the half range saturate to 0x7bff there).
 * fp32 -> bf16: reference pb_gtest/src/tools.cpp:691-710.
 * ---------------------------------------------------------------------- */
static uint16_t float_to_half_bits(float x) {
  int32_t in;
  memcpy(&in, &x, 4);
  int sign = (in >> 31) & 1;
  int exp = ((in >> 23) & 0xff) - 127;
  int denorm = 0, eff, g = 0;
  if (exp == 128 && (in & 0x7fffff)) {
    exp = 0x1f - 15; eff = 0x200;
  } else if (exp == 128) {
    exp = 0x1f - 15; eff = 0x000;
  } else if (exp >= 16) {
    exp = 0xf; eff = 0x3ff;
  } else if (exp >= -14) {
    int gr_last = in & 0xfff;
    int gr_first = (in >> 12) & 1;
    int g_last = (in >> 13) & 1;
    g = (gr_first && gr_last) || (gr_first && g_last);
    eff = (in >> 13) & 0x3ff;
  } else if (exp >= -24) {
    g = (((in & 0x7fffff) | 0x800000) >> (-exp - 2)) & 1;
    eff = (((in & 0x7fffff) | 0x800000) >> (-exp - 1)) & 0x3ff;
    denorm = 1; exp = 0;
  } else {
    exp = 0; denorm = 1;
    eff = (in & 0x7fffffff) ? 1 : 0;
  }
  eff += g;
  exp = denorm ? exp : exp + 15;
  return (uint16_t)((sign << 15) + (exp << 10) + eff);
}

static float half_bits_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h >> 15) << 31;
  int exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ff;
  uint32_t out;
  if (exp == 0) {
    if (man == 0) {
      out = sign;
    } else {
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400));
      out = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ff) << 13);
    }
  } else if (exp == 0x1f) {
    out = sign | 0x7f800000u | (man << 13);
  } else {
    out = sign | ((uint32_t)(exp - 15 + 127) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &out, 4);
  return f;
}

void oracle_round_through_half(const float *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = half_bits_to_float(float_to_half_bits(src[i]));
}

void oracle_float_to_half_bits(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) dst[i] = float_to_half_bits(src[i]);
}

void oracle_float_to_bf16_bits(const float *src, uint16_t *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    uint32_t u;
    memcpy(&u, &src[i], 4);
    if (isnan(src[i])) {
      dst[i] = 0x7FC0;
    } else {
      uint32_t bias = ((u >> 16) & 1u) + 0x7FFFu;
      dst[i] = (uint16_t)((u + bias) >> 16);
    }
  }
}

void oracle_round_through_bf16(const float *src, float *dst, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    uint16_t b;
    oracle_float_to_bf16_bits(&src[i], &b, 1);
    uint32_t u = (uint32_t)b << 16;
    memcpy(&dst[i], &u, 4);
  }
}

/* ------------------------------------------------------------------------
 * Diff metrics.  reference pb_gtest/include/evaluator.h:431-519.
 * a = device result, b = oracle result.  eps3 is the threshold below which
 * diff3 uses the absolute error (1e-6 for float, 1e-4 for half).
 * ---------------------------------------------------------------------- */
double oracle_diff1(const float *a, const float *b, int64_t n) {
  double num = 0.0, den = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    num += fabs((double)a[i] - (double)b[i]);
    den += fabs((double)b[i]);
  }
  return num / (den + 1e-9);
}

double oracle_diff2(const float *a, const float *b, int64_t n) {
  double num = 0.0, den = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    double d = (double)a[i] - (double)b[i];
    num += d * d;
    den += (double)b[i] * (double)b[i];
  }
  return sqrt(num / (den + 1e-9));
}

double oracle_diff3(const float *a, const float *b, int64_t n, double eps3) {
  double mx = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    double num = fabs((double)a[i] - (double)b[i]);
    double den = fabs((double)b[i]);
    double ratio = den < eps3 ? num : num / (den + 1e-9);
    if (ratio > mx) mx = ratio;
  }
  return mx;
}
