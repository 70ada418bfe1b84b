// Dynamic point-to-voxel scatter, forward: points that share a coordinate
// triple form a voxel; voxels are numbered in ascending (lexicographic) order
// of their triples; the features of a voxel's points are reduced by max or
// mean.  The reference delegates the grouping to a vendor "unique" routine
// (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_forward/
//  dynamic_point_to_voxel_forward.cpp:300-340) and reduces with atomics.
//
// Here:
//   1 dpvPrepare   rows with a negative coordinate become (-1,-1,-1) in place;
//                  the largest coordinate of every axis is collected so that
//                  the sorts run over as few bits as the data needs
//   2 one stable radix sort of (packed triple, point index) when the three
//                  coordinates (+1) fit 64 bits together, which they do up to
//                  2^21 cells per axis; otherwise three stable sorts, last
//                  axis first.  Either way the points end up in ascending
//                  triple order, equal triples in point order
//   3 dpvHeads + inclusive scan: number of the triple each sorted point has
//   4 dpvEmit      point2voxel_map, voxel_coors, first sorted position of
//                  every voxel, voxel_num
//   5 dpvReduce    one thread per (voxel, feature) walks the voxel's points in
//                  point order: max, or the sum of feats / count in exactly
//                  the order the sequential definition adds them, so the mean
//                  has the same bits on every run
#include <hip/hip_runtime.h>
#include <cstring>

#include "core/device_sort.h"

#include "dynamic_point_to_voxel/scatter_points.h"

namespace mluop {
namespace dynamic_point_to_voxel {
namespace {

constexpr int kBlock = 256;

inline int gridFor(size_t n, int cap = 1 << 20) {
  size_t b = (n + kBlock - 1) / kBlock;
  if (b < 1) b = 1;
  return (int)(b > (size_t)cap ? (size_t)cap : b);
}

size_t alignUp(size_t v) { return (v + 255) & ~(size_t)255; }

__global__ __launch_bounds__(kBlock) void dpvFill(float *voxel_feats, size_t feat_words,
                                                  float fill, int32_t *voxel_coors,
                                                  int32_t *voxel_points_count, int rows,
                                                  int32_t *axis_max) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
  for (size_t i = t; i < feat_words; i += stride) voxel_feats[i] = fill;
  for (size_t i = t; i < (size_t)rows * 3; i += stride) voxel_coors[i] = 0;
  for (size_t i = t; i < (size_t)rows; i += stride) voxel_points_count[i] = 0;
  if (t < 3) axis_max[t] = -1;
}

__global__ __launch_bounds__(kBlock) void dpvPrepare(int32_t *coors, int n, uint32_t *keys,
                                                     uint32_t *points, int32_t *axis_max) {
  // grid-stride: a few hundred blocks, so that the three atomics per block stay cheap
  int m0 = -1, m1 = -1, m2 = -1;
  for (int i = blockIdx.x * kBlock + threadIdx.x; i < n; i += gridDim.x * kBlock) {
    int c0 = coors[3 * (size_t)i];
    int c1 = coors[3 * (size_t)i + 1];
    int c2 = coors[3 * (size_t)i + 2];
    if (c0 < 0 || c1 < 0 || c2 < 0) {
      c0 = c1 = c2 = -1;
      coors[3 * (size_t)i] = -1;
      coors[3 * (size_t)i + 1] = -1;
      coors[3 * (size_t)i + 2] = -1;
    }
    keys[i] = (uint32_t)(c2 + 1);  // the last axis is sorted first (three-sort path)
    points[i] = (uint32_t)i;
    m0 = max(m0, c0);
    m1 = max(m1, c1);
    m2 = max(m2, c2);
  }
  // block maxima, then one atomic per axis and block
  __shared__ int s_max[3][kBlock / 64];
  for (int off = 32; off > 0; off >>= 1) {
    m0 = max(m0, __shfl_xor(m0, off, 64));
    m1 = max(m1, __shfl_xor(m1, off, 64));
    m2 = max(m2, __shfl_xor(m2, off, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    s_max[0][threadIdx.x >> 6] = m0;
    s_max[1][threadIdx.x >> 6] = m1;
    s_max[2][threadIdx.x >> 6] = m2;
  }
  __syncthreads();
  if (threadIdx.x < 3) {
    int m = s_max[threadIdx.x][0];
    for (int w = 1; w < kBlock / 64; ++w) m = max(m, s_max[threadIdx.x][w]);
    if (m >= 0) atomicMax(&axis_max[threadIdx.x], m);
  }
}

// key = (c0+1, c1+1, c2+1) packed most significant first; rows are already masked
template <typename KeyT>
__global__ __launch_bounds__(kBlock) void dpvPackKeys(const int32_t *__restrict__ coors, int n,
                                                      int bits1, int bits2, KeyT *keys) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const KeyT k0 = (KeyT)(uint32_t)(coors[3 * (size_t)i] + 1);
  const KeyT k1 = (KeyT)(uint32_t)(coors[3 * (size_t)i + 1] + 1);
  const KeyT k2 = (KeyT)(uint32_t)(coors[3 * (size_t)i + 2] + 1);
  keys[i] = (k0 << (bits1 + bits2)) | (k1 << bits2) | k2;
}

// The 32-bit packed key in the low half of a 64-bit word and the point index in the high
// half: sorted as one key by the low bits, the point travels with it (half the scattered
// stores of a sort of pairs).
__global__ __launch_bounds__(kBlock) void dpvPackRecords(const int32_t *__restrict__ coors, int n,
                                                         int bits1, int bits2, unsigned long long *records) {
  const int i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const uint32_t k0 = (uint32_t)(coors[3 * (size_t)i] + 1);
  const uint32_t k1 = (uint32_t)(coors[3 * (size_t)i + 1] + 1);
  const uint32_t k2 = (uint32_t)(coors[3 * (size_t)i + 2] + 1);
  const uint32_t key = (k0 << (bits1 + bits2)) | (k1 << bits2) | k2;
  records[i] = ((unsigned long long)(uint32_t)i << 32) | key;
}

// head[p] = 1 where the key half of the sorted records changes
__global__ __launch_bounds__(kBlock) void dpvHeadsFromRecords(const unsigned long long *__restrict__ sorted,
                                                              int n, uint32_t *head) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  head[p] = (p == 0 || (uint32_t)sorted[p] != (uint32_t)sorted[p - 1]) ? 1u : 0u;
}

// keys[p] = coordinate `axis` of the point at sorted position p, plus one
__global__ __launch_bounds__(kBlock) void dpvGatherKeys(const int32_t *__restrict__ coors,
                                                        const uint32_t *__restrict__ points, int n,
                                                        int axis, uint32_t *keys) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p < n) keys[p] = (uint32_t)(coors[3 * (size_t)points[p] + axis] + 1);
}

// head[p] = 1 where the sorted packed key changes
template <typename KeyT>
__global__ __launch_bounds__(kBlock) void dpvHeadsFromKeys(const KeyT *__restrict__ sorted_keys,
                                                           int n, uint32_t *head) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  head[p] = (p == 0 || sorted_keys[p] != sorted_keys[p - 1]) ? 1u : 0u;
}

__global__ __launch_bounds__(kBlock) void dpvHeads(const int32_t *__restrict__ coors,
                                                   const uint32_t *__restrict__ points, int n,
                                                   uint32_t *head) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  if (p == 0) {
    head[0] = 1;
    return;
  }
  const int32_t *a = coors + 3 * (size_t)points[p];
  const int32_t *b = coors + 3 * (size_t)points[p - 1];
  head[p] = (a[0] != b[0] || a[1] != b[1] || a[2] != b[2]) ? 1u : 0u;
}

// (`points` holds the sorted point indices `stride` words apart: 1, or 2 where they are the
// high halves of sorted records; with records, a voxel's coordinates are unpacked from the
// key half, bits1 and bits2 wide for the last two axes, instead of gathered from its first point)
__global__ __launch_bounds__(kBlock) void dpvEmit(const int32_t *__restrict__ coors,
                                                  const uint32_t *__restrict__ points, int stride,
                                                  bool keys_beside_points, int bits1, int bits2,
                                                  const uint32_t *__restrict__ head,
                                                  const uint32_t *__restrict__ triple_count, int n,
                                                  int rows, int32_t *point2voxel_map,
                                                  int32_t *voxel_coors, int32_t *first_pos,
                                                  int32_t *voxel_num) {
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  // the (-1,-1,-1) triple sorts first and is not a voxel
  const int skipped = coors[3 * (size_t)points[0]] == -1 ? 1 : 0;
  const int v = (int)triple_count[p] - 1 - skipped;
  const uint32_t i = points[(size_t)p * stride];
  point2voxel_map[i] = v;
  if (head[p] && v >= 0 && v <= rows) {
    first_pos[v] = p;  // one past the last stored voxel included: it ends that voxel
    if (v < rows) {
      if (keys_beside_points) {
        const uint32_t key = points[(size_t)p * stride - 1];  // the low half of the record
        voxel_coors[3 * (size_t)v] = (int32_t)(key >> (bits1 + bits2)) - 1;
        voxel_coors[3 * (size_t)v + 1] = (int32_t)((key >> bits2) & ((1u << bits1) - 1u)) - 1;
        voxel_coors[3 * (size_t)v + 2] = (int32_t)(key & ((1u << bits2) - 1u)) - 1;
      } else {
        voxel_coors[3 * (size_t)v] = coors[3 * (size_t)i];
        voxel_coors[3 * (size_t)v + 1] = coors[3 * (size_t)i + 1];
        voxel_coors[3 * (size_t)v + 2] = coors[3 * (size_t)i + 2];
      }
    }
  }
  if (p == n - 1) *voxel_num = v + 1;
}

__global__ __launch_bounds__(kBlock) void dpvReduce(const float *__restrict__ feats,
                                                    const uint32_t *__restrict__ points, int stride,
                                                    const int32_t *__restrict__ first_pos,
                                                    const int32_t *__restrict__ voxel_num, int n,
                                                    int num_features, int rows, bool reduce_max,
                                                    float *voxel_feats,
                                                    int32_t *voxel_points_count) {
  const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
  const int voxels = min(*voxel_num, rows);
  if (t >= (size_t)voxels * num_features) return;
  const int v = (int)(t / num_features);
  const int f = (int)(t % num_features);
  const int begin = first_pos[v];
  // dpvEmit stores the first position of voxel `rows` too, when there is one
  const int stop = v + 1 < *voxel_num ? first_pos[v + 1] : n;
  const int count = stop - begin;
  if (f == 0) voxel_points_count[v] = count;
  if (reduce_max) {
    float best = -INFINITY;
    for (int p = begin; p < stop; ++p) {
      const float x = feats[(size_t)points[(size_t)p * stride] * num_features + f];
      if (x >= best) best = x;
    }
    voxel_feats[t] = best;
  } else {
    float sum = 0.f;
    const float fcount = (float)count;
    for (int p = begin; p < stop; ++p)
      sum = __fadd_rn(sum, __fdiv_rn(feats[(size_t)points[(size_t)p * stride] * num_features + f], fcount));
    voxel_feats[t] = sum;
  }
}

// ---- backward of the max reduction ----

__global__ __launch_bounds__(kBlock) void dpvBackwardInit(float *grad_feats, size_t grad_words,
                                                          int32_t *from, size_t from_words,
                                                          int32_t none) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
  for (size_t i = t; i < grad_words; i += stride) grad_feats[i] = 0.f;
  for (size_t i = t; i < from_words; i += stride) from[i] = none;
}

// from[v, c] = lowest point index whose feature equals the voxel's maximum
__global__ __launch_bounds__(kBlock) void dpvBackwardFindSource(
    const float *__restrict__ feats, const float *__restrict__ voxel_feats,
    const int32_t *__restrict__ point2voxel_map, int n, int num_features, int rows, int32_t *from) {
  const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= (size_t)n * num_features) return;
  const int x = (int)(t / num_features);
  const int c = (int)(t % num_features);
  const int v = point2voxel_map[x];
  if (v < 0 || v >= rows) return;
  if (feats[t] == voxel_feats[(size_t)v * num_features + c])
    atomicMin(&from[(size_t)v * num_features + c], x);
}

__global__ __launch_bounds__(kBlock) void dpvBackwardScatter(
    const float *__restrict__ grad_voxel_feats, const int32_t *__restrict__ from,
    const int32_t *__restrict__ voxel_num, int n, int num_features, int rows, float *grad_feats) {
  const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
  const int voxels = min(*voxel_num, rows);
  if (t >= (size_t)voxels * num_features) return;
  const int x = from[t];
  if (x < n) grad_feats[(size_t)x * num_features + t % num_features] = grad_voxel_feats[t];
}

struct Workspace {
  uint32_t *keys_a, *keys_b, *points_a, *points_b, *head, *triple_count;
  int32_t *first_pos, *axis_max;
  void *library;
  size_t total;
};

Workspace carve(void *base, const ScatterShape &s, size_t library_bytes) {
  const size_t n = (size_t)s.num_points;
  // Blocks start at the caller's pointer rounded up to 256 bytes (64-bit keys, packed sort
  // keys and the sort's counters need their alignment whatever the caller
  // passes); the reported size includes that slack.  A null base only measures.
  char *p = base ? reinterpret_cast<char *>(alignUp(reinterpret_cast<uintptr_t>(base))) : nullptr;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *q = p ? p + off : nullptr;
    off += alignUp(bytes);
    return q;
  };
  Workspace w;
  w.keys_a = reinterpret_cast<uint32_t *>(take(8 * n));  // 64-bit packed keys at most
  w.keys_b = reinterpret_cast<uint32_t *>(take(8 * n));
  w.points_a = reinterpret_cast<uint32_t *>(take(4 * n));
  w.points_b = reinterpret_cast<uint32_t *>(take(4 * n));
  w.head = reinterpret_cast<uint32_t *>(take(4 * n));
  w.triple_count = reinterpret_cast<uint32_t *>(take(4 * n));
  w.first_pos = reinterpret_cast<int32_t *>(take(4 * (n + 1)));
  w.axis_max = reinterpret_cast<int32_t *>(take(16));
  w.library = take(library_bytes);
  w.total = off + 256;
  return w;
}

int bitsFor(int32_t max_coordinate) {  // keys are coordinate + 1, 0 for the -1 triple
  const uint32_t top = (uint32_t)(max_coordinate + 1);
  int b = 1;
  while (b < 32 && (top >> b) != 0) ++b;
  return b;
}

}  // namespace

size_t scatterWorkspaceBytes(const ScatterShape &s, size_t library_bytes) {
  return carve(nullptr, s, library_bytes).total;
}

hipError_t libraryWorkspaceBytes(const ScatterShape &s, hipStream_t stream, size_t *bytes) {
  (void)stream;
  *bytes = device_sort::workspaceBytes((size_t)s.num_points);
  return hipSuccess;
}

hipError_t launchScatterPoints(const LaunchCtx &lc, const ScatterShape &s, const float *feats,
                               int32_t *coors, void *workspace, size_t workspace_bytes,
                               int32_t *pinned_host, float *voxel_feats, int32_t *voxel_coors,
                               int32_t *point2voxel_map, int32_t *voxel_points_count,
                               int32_t *voxel_num) {
  const int n = s.num_points;
  size_t library_bytes = 0;
  hipError_t e = libraryWorkspaceBytes(s, lc.stream, &library_bytes);
  if (e != hipSuccess) return e;
  const Workspace w = carve(workspace, s, library_bytes);
  if (w.total > workspace_bytes) return hipErrorInvalidValue;
  const int blocks = gridFor((size_t)n);

  const size_t feat_words = (size_t)s.voxel_rows * s.num_features;
  lc.begin("dpvFill");
  dpvFill<<<gridFor(feat_words > (size_t)n ? feat_words : (size_t)n, 4096), kBlock, 0, lc.stream>>>(
      voxel_feats, feat_words, s.reduce_max ? -INFINITY : 0.f, voxel_coors, voxel_points_count,
      s.voxel_rows, w.axis_max);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;

  lc.begin("dpvPrepare");
  dpvPrepare<<<gridFor((size_t)n, 512), kBlock, 0, lc.stream>>>(coors, n, w.keys_a, w.points_a,
                                                                w.axis_max);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;
  e = hipMemcpyAsync(pinned_host, w.axis_max, 3 * sizeof(int32_t), hipMemcpyDeviceToHost,
                     lc.stream);
  if (e != hipSuccess) return e;
  if ((e = hipStreamSynchronize(lc.stream)) != hipSuccess) return e;
  const int bits[3] = {bitsFor(pinned_host[0]), bitsFor(pinned_host[1]), bitsFor(pinned_host[2])};

  uint32_t *pts_in = w.points_a, *pts_out = w.points_b;
  bool packed = false;
  const int total_bits = bits[0] + bits[1] + bits[2];
  bool in_b = false;  // which pair of arrays a sort left its result in
  const uint32_t *record_points = nullptr;  // sorted point indices inside 64-bit records
  if (total_bits <= 64) {
    if (total_bits <= 32) {
      unsigned long long *ra = reinterpret_cast<unsigned long long *>(w.keys_a);
      unsigned long long *rb = reinterpret_cast<unsigned long long *>(w.keys_b);
      lc.begin("dpvPackKeys");
      dpvPackRecords<<<blocks, kBlock, 0, lc.stream>>>(coors, n, bits[1], bits[2], ra);
      lc.end();
      if ((e = hipGetLastError()) != hipSuccess) return e;
      lc.begin("radixSortPairs");
      e = device_sort::sortKeys<unsigned long long>(lc.stream, w.library, ra, rb, (size_t)n, total_bits, &in_b);
      lc.end();
      if (e != hipSuccess) return e;
      const unsigned long long *sorted = in_b ? rb : ra;
      lc.begin("dpvHeads");
      dpvHeadsFromRecords<<<blocks, kBlock, 0, lc.stream>>>(sorted, n, w.head);
      lc.end();
      record_points = reinterpret_cast<const uint32_t *>(sorted) + 1;  // the high halves
    } else {
      unsigned long long *ka = reinterpret_cast<unsigned long long *>(w.keys_a);
      unsigned long long *kb = reinterpret_cast<unsigned long long *>(w.keys_b);
      lc.begin("dpvPackKeys");
      dpvPackKeys<unsigned long long><<<blocks, kBlock, 0, lc.stream>>>(coors, n, bits[1], bits[2], ka);
      lc.end();
      if ((e = hipGetLastError()) != hipSuccess) return e;
      lc.begin("radixSortPairs");
      e = device_sort::sortPairs<unsigned long long>(lc.stream, w.library, ka, kb, pts_in, pts_out,
                                                     (size_t)n, total_bits, &in_b);
      lc.end();
      if (e != hipSuccess) return e;
      lc.begin("dpvHeads");
      dpvHeadsFromKeys<unsigned long long><<<blocks, kBlock, 0, lc.stream>>>(in_b ? kb : ka, n, w.head);
      lc.end();
    }
    if ((e = hipGetLastError()) != hipSuccess) return e;
    if (in_b && record_points == nullptr) pts_in = pts_out;
    packed = true;
  } else {
    // last axis first; every pass is stable, so the final order is lexicographic
    // with equal triples in point order
    for (int axis = 2; axis >= 0; --axis) {
      if (axis != 2) {
        lc.begin("dpvGatherKeys");
        dpvGatherKeys<<<blocks, kBlock, 0, lc.stream>>>(coors, pts_in, n, axis, w.keys_a);
        lc.end();
        if ((e = hipGetLastError()) != hipSuccess) return e;
      }
      lc.begin("radixSortPairs");
      e = device_sort::sortPairs<uint32_t>(lc.stream, w.library, w.keys_a, w.keys_b, pts_in, pts_out,
                                           (size_t)n, bits[axis], &in_b);
      lc.end();
      if (e != hipSuccess) return e;
      if (in_b) {
        uint32_t *t = pts_in;
        pts_in = pts_out;
        pts_out = t;
      }
    }
  }
  const uint32_t *sorted_points = record_points != nullptr ? record_points : pts_in;
  const int point_stride = record_points != nullptr ? 2 : 1;

  if (!packed) {
    lc.begin("dpvHeads");
    dpvHeads<<<blocks, kBlock, 0, lc.stream>>>(coors, sorted_points, n, w.head);
    lc.end();
    if ((e = hipGetLastError()) != hipSuccess) return e;
  }
  lc.begin("inclusiveScan");
  e = device_sort::prefixSums(lc.stream, w.library, w.head, w.triple_count, (size_t)n, true);
  lc.end();
  if (e != hipSuccess) return e;

  lc.begin("dpvEmit");
  dpvEmit<<<blocks, kBlock, 0, lc.stream>>>(coors, sorted_points, point_stride, record_points != nullptr,
                                             bits[1], bits[2], w.head, w.triple_count, n,
                                             s.voxel_rows, point2voxel_map, voxel_coors,
                                             w.first_pos, voxel_num);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;

  lc.begin("dpvReduce");
  dpvReduce<<<gridFor(feat_words), kBlock, 0, lc.stream>>>(
      feats, sorted_points, point_stride, w.first_pos, voxel_num, n, s.num_features, s.voxel_rows, s.reduce_max,
      voxel_feats, voxel_points_count);
  lc.end();
  return hipGetLastError();
}

hipError_t launchScatterPointsBackward(const LaunchCtx &lc, int num_points, int num_features,
                                       int voxel_rows, const float *grad_voxel_feats,
                                       const float *feats, const float *voxel_feats,
                                       const int32_t *point2voxel_map, const int32_t *voxel_num,
                                       int32_t *from, float *grad_feats) {
  const size_t grad_words = (size_t)num_points * num_features;
  const size_t from_words = (size_t)voxel_rows * num_features;
  lc.begin("dpvBackwardInit");
  dpvBackwardInit<<<gridFor(grad_words, 4096), kBlock, 0, lc.stream>>>(grad_feats, grad_words, from,
                                                                       from_words, num_points);
  lc.end();
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || from_words == 0) return e;
  lc.begin("dpvBackwardFindSource");
  dpvBackwardFindSource<<<gridFor(grad_words), kBlock, 0, lc.stream>>>(
      feats, voxel_feats, point2voxel_map, num_points, num_features, voxel_rows, from);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;
  lc.begin("dpvBackwardScatter");
  dpvBackwardScatter<<<gridFor(from_words), kBlock, 0, lc.stream>>>(
      grad_voxel_feats, from, voxel_num, num_points, num_features, voxel_rows, grad_feats);
  lc.end();
  return hipGetLastError();
}

}  // namespace dynamic_point_to_voxel
}  // namespace mluop
