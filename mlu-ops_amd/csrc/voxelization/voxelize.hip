// Hard voxelization (deterministic): every point is assigned to the cell of a
// regular grid it falls in; cells are numbered in the order of their first
// point, keep their first max_points points in point order, and only the
// first max_voxels cells are kept.
//
// The reference searches, for every point, all earlier points for the same
// cell (kernels/voxelization/voxelization_kernel.mlu, KernelPoint2Voxel), then
// numbers the voxels with a single core
// (kernels/voxelization/voxelization.cpp:45-53).  Here the same result comes
// from grouping instead of searching:
//   1 voxCellSlots   cell of every point; the 64-bit cell id is entered into an
//                    open-addressing table, whose slot number names the cell
//   2 radix sort     (slot, point index) pairs, packed into 64-bit words, by slot, least significant
//                    digit first and therefore stable: every cell's points end
//                    up adjacent and in point order
//   3 voxMarkFirst   the first point of every cell (the point at the head of the cell's
//                    run) raises its flag in an array over the points
//   4 prefix sums over the flags: the voxel number of a cell is the number of first
//                    points in front of its own, which is the sequential numbering of the
//                    reference
//   5 voxAssign      in sorted order: position in the cell = sorted position - head of the
//                    run, voxel number from the bitmap; copies points and coordinates,
//                    counts points per voxel
// Integer atomics only (table insertion, per-voxel counts): the outputs are
// the same bits on every run.
#include <hip/hip_runtime.h>
#include <cstring>

#include "core/device_sort.h"

#include "voxelization/voxelize.h"

namespace mluop {
namespace voxelization {
namespace {

constexpr unsigned long long kEmptyKey = ~0ull;
constexpr int kBlock = 256;

inline int gridFor(size_t n, int cap = 1 << 20) {
  size_t b = (n + kBlock - 1) / kBlock;
  if (b < 1) b = 1;
  return (int)(b > (size_t)cap ? (size_t)cap : b);
}

size_t alignUp(size_t v) { return (v + 255) & ~(size_t)255; }

uint32_t tableSlots(int64_t num_points) {
  uint32_t cap = 1024;
  while ((int64_t)cap < 2 * num_points) cap <<= 1;
  return cap;
}

int bitsFor(uint32_t cap) {  // slot numbers 0..cap (cap itself marks "no cell")
  int b = 1;
  while ((1ull << b) <= cap) ++b;
  return b;
}

// Up to five regions of 32-bit words filled by one launch.
constexpr int kFillRegions = 5;
struct FillRegions {
  uint32_t *base[kFillRegions];
  size_t words[kFillRegions];
  uint32_t value[kFillRegions];
};

__global__ __launch_bounds__(kBlock) void voxFillRegions(FillRegions r) {
#pragma unroll
  for (int g = 0; g < kFillRegions; ++g) {
    // words in front of the first 16-byte boundary, 16-byte stores, words behind the last
    size_t head = ((16 - (reinterpret_cast<uintptr_t>(r.base[g]) & 15)) & 15) / 4;
    head = head < r.words[g] ? head : r.words[g];
    uint32_t *body = r.base[g] + head;
    const size_t body_words = r.words[g] - head;
    const size_t quads = body_words / 4;
    const uint32_t value = r.value[g];
    const uint4 v = make_uint4(value, value, value, value);
    uint4 *dst = reinterpret_cast<uint4 *>(body);
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < quads;
         i += (size_t)gridDim.x * kBlock)
      dst[i] = v;
    if (blockIdx.x == 0) {
      if (threadIdx.x < head) r.base[g][threadIdx.x] = value;
      if (threadIdx.x < (body_words & 3)) body[quads * 4 + threadIdx.x] = value;
    }
  }
}

// Cells along one axis: the float quotient rounded half away from zero.
__device__ inline int axisCells(float lo, float hi, float size) {
  const float g = roundf((hi - lo) / size);
  return (g >= 1.f && g < 2147483648.f) ? (int)g : 0;
}

// Cell index of a coordinate, or -1 outside [0, cells) (NaN included).
__device__ inline int cellIndex(float p, float lo, float size, int cells) {
  const float f = floorf((p - lo) / size);
  if (!(f >= 0.f && f < 2147483648.f)) return -1;
  const int c = (int)f;
  return c < cells ? c : -1;
}

__device__ inline uint32_t mix64(unsigned long long k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return (uint32_t)k;
}

// The cell (z, y, x) of a point, or cz < 0 outside the grid.
struct Cell {
  int cz, cy, cx, gy, gx;
  unsigned long long cells;
};
__device__ inline Cell cellOfPoint(const float *__restrict__ p, const float *__restrict__ voxel_size,
                                   const float *__restrict__ range) {
  const float sx = voxel_size[0], sy = voxel_size[1], sz = voxel_size[2];
  const float x0 = range[0], y0 = range[1], z0 = range[2];
  const int gx = axisCells(x0, range[3], sx);
  const int gy = axisCells(y0, range[4], sy);
  const int gz = axisCells(z0, range[5], sz);
  Cell c;
  c.gx = gx;
  c.gy = gy;
  c.cells = (unsigned long long)gz * (unsigned long long)gy * gx;
  c.cx = cellIndex(p[0], x0, sx, gx);
  c.cy = c.cx < 0 ? -1 : cellIndex(p[1], y0, sy, gy);
  c.cz = c.cy < 0 ? -1 : cellIndex(p[2], z0, sz, gz);
  return c;
}

__global__ __launch_bounds__(kBlock) void voxCellSlots(
    const float *__restrict__ points, const float *__restrict__ voxel_size,
    const float *__restrict__ range, int64_t n, int num_features, unsigned long long *keys,
    uint32_t cap, unsigned long long *slot_and_point) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  const Cell c = cellOfPoint(points + i * num_features, voxel_size, range);
  const int cz = c.cz, cy = c.cy, cx = c.cx, gy = c.gy, gx = c.gx;
  // (table slot in the low half, point index in the high half: sorted as one 64-bit key by
  // the slot's bits, the point travels with it)
  const unsigned long long point_half = (unsigned long long)i << 32;
  if (cz < 0) {
    slot_and_point[i] = point_half | cap;
    return;
  }
  const unsigned long long key =
      ((unsigned long long)cz * (unsigned long long)gy + cy) * (unsigned long long)gx + cx;
  uint32_t slot = mix64(key) & (cap - 1);
  // At most half of the slots are ever taken, so an empty one is always reached.
  // A grid of fewer than 2^32 - 1 cells (the same for every thread) keeps 32-bit
  // keys in the first half of the table: 32-bit compare-and-swap is several times
  // faster than the 64-bit one.
  if (c.cells < 0xffffffffull) {
    uint32_t *keys32 = reinterpret_cast<uint32_t *>(keys);
    const uint32_t key32 = (uint32_t)key;
    while (true) {
      const uint32_t seen = atomicCAS(&keys32[slot], 0xffffffffu, key32);
      if (seen == 0xffffffffu || seen == key32) break;
      slot = (slot + 1) & (cap - 1);
    }
  } else {
    while (true) {
      const unsigned long long seen = atomicCAS(&keys[slot], kEmptyKey, key);
      if (seen == kEmptyKey || seen == key) break;
      slot = (slot + 1) & (cap - 1);
    }
  }
  slot_and_point[i] = point_half | slot;
}

// is_first[f] = 1 <=> point f is the first of its cell (the array was cleared by the fill; a
// plain store per cell: a bitmap would take an atomic per cell, four times as long).
__global__ __launch_bounds__(kBlock) void voxMarkFirst(const unsigned long long *__restrict__ sorted,
                                                       int64_t n, uint32_t cap, uint32_t *is_first) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  const unsigned long long mine = sorted[p];
  const uint32_t s = (uint32_t)mine;
  if (s == cap) return;
  if (p == 0 || (uint32_t)sorted[p - 1] != s) is_first[(uint32_t)(mine >> 32)] = 1u;
}

// First sorted position whose slot is `s`, which lies in front of position `from` (whose slot
// is `s` as well): doubling steps backwards, then a binary search.
__device__ inline int64_t headBefore(const unsigned long long *__restrict__ sorted, int64_t from, uint32_t s) {
  int64_t hi = from;  // sorted[hi] holds slot s
  int64_t step = 1;
  int64_t lo = hi - step;
  while (lo >= 0 && (uint32_t)sorted[lo] == s) {
    hi = lo;
    step *= 2;
    lo = hi - step;
  }
  if (lo < 0) {
    if ((uint32_t)sorted[0] == s) return 0;
    lo = 0;
  }
  // sorted[lo] is another slot's, sorted[hi] this one's, the run starts in (lo, hi]
  while (hi - lo > 1) {
    const int64_t mid = lo + (hi - lo) / 2;
    if ((uint32_t)sorted[mid] == s)
      hi = mid;
    else
      lo = mid;
  }
  return hi;
}

// Thread p takes the point at sorted position p.  The head of its cell's run is the nearest
// position at or in front of p where the slot changes: found among the lanes of the wave by a
// running maximum, and looked up behind the wave only by the lanes of a run that began earlier.
__global__ __launch_bounds__(kBlock) void voxAssign(
    const float *__restrict__ points, const float *__restrict__ voxel_size,
    const float *__restrict__ range, const unsigned long long *__restrict__ sorted,
    const uint32_t *__restrict__ is_first,
    const uint32_t *__restrict__ voxel_of_first, int64_t n, uint32_t cap, int num_features, int max_points,
    int max_voxels, float *voxels, int32_t *coors, int32_t *num_points_per_voxel, int32_t *voxel_num) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int lane = threadIdx.x & 63;
  if (p == 0) {
    uint32_t cells = 0;
    if (n > 0) cells = voxel_of_first[n - 1] + is_first[n - 1];
    *voxel_num = cells < (uint32_t)max_voxels ? (int32_t)cells : max_voxels;
  }
  const bool live = p < n;
  const unsigned long long mine = live ? sorted[p] : (unsigned long long)cap;
  const uint32_t s = (uint32_t)mine;
  const uint32_t before = (live && p > 0) ? (uint32_t)sorted[p - 1] : cap;
  const bool starts = live && s != cap && (p == 0 || before != s);
  // nearest run start at or below this lane, inside the wave (-1: none)
  long long head = starts ? (long long)p : -1;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const long long up = __shfl_up(head, d, 64);
    if (lane >= d && up > head) head = up;
  }
  if (!live || s == cap) return;
  if (head < 0) head = headBefore(sorted, p - lane, s);  // (position p - lane holds slot s too)
  const int64_t r = p - head;
  if (r >= max_points) return;
  const uint32_t f = (uint32_t)(sorted[head] >> 32);
  const uint32_t v = voxel_of_first[f];  // first points in front of f
  if (v >= (uint32_t)max_voxels) return;
  const uint32_t i = (uint32_t)(mine >> 32);
  const float *src = points + (size_t)i * num_features;
  float *dst = voxels + ((size_t)v * max_points + r) * num_features;
  for (int k = 0; k < num_features; ++k) dst[k] = src[k];
  atomicAdd(&num_points_per_voxel[v], 1);
  if (r == 0) {
    const Cell c = cellOfPoint(src, voxel_size, range);
    coors[3 * (size_t)v] = c.cz;
    coors[3 * (size_t)v + 1] = c.cy;
    coors[3 * (size_t)v + 2] = c.cx;
  }
}

struct Workspace {
  unsigned long long *pairs_a, *pairs_b;  // table slot | point index << 32
  uint32_t *is_first, *voxel_of_first;
  unsigned long long *keys;
  void *library;
  size_t total;
};

Workspace carve(void *base, const VoxelizeShape &s, size_t library_bytes) {
  const size_t n = (size_t)s.num_points;
  const uint32_t cap = tableSlots(s.num_points);
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
  w.pairs_a = reinterpret_cast<unsigned long long *>(take(8 * n));
  w.pairs_b = reinterpret_cast<unsigned long long *>(take(8 * n));
  w.is_first = reinterpret_cast<uint32_t *>(take(4 * n));
  w.voxel_of_first = reinterpret_cast<uint32_t *>(take(4 * n));
  w.keys = reinterpret_cast<unsigned long long *>(take(8 * (size_t)cap));
  w.library = take(library_bytes);
  w.total = off + 256;
  return w;
}


}  // namespace

size_t voxelizeWorkspaceBytes(const VoxelizeShape &s, size_t library_bytes) {
  return carve(nullptr, s, library_bytes).total;
}

hipError_t libraryWorkspaceBytes(const VoxelizeShape &s, hipStream_t stream, size_t *bytes) {
  (void)stream;
  *bytes = device_sort::workspaceBytes((size_t)s.num_points);
  return hipSuccess;
}

hipError_t launchVoxelize(const LaunchCtx &lc, const VoxelizeShape &s, const float *points,
                          const float *voxel_size, const float *coors_range, void *workspace,
                          size_t workspace_bytes, float *voxels, int32_t *coors,
                          int32_t *num_points_per_voxel, int32_t *voxel_num) {
  const int64_t n = s.num_points;
  const uint32_t cap = tableSlots(n);
  size_t library_bytes = 0;
  hipError_t e = libraryWorkspaceBytes(s, lc.stream, &library_bytes);
  if (e != hipSuccess) return e;
  const Workspace w = carve(workspace, s, library_bytes);
  if (w.total > workspace_bytes) return hipErrorInvalidValue;

  // outputs start from zero (reference kernels/voxelization/voxelization.cpp:283-309),
  // the cell table from "empty" and the flags of first points from none raised
  FillRegions fr;
  fr.base[0] = reinterpret_cast<uint32_t *>(voxels);
  fr.words[0] = (size_t)s.max_voxels * s.max_points * s.num_features;
  fr.base[1] = reinterpret_cast<uint32_t *>(coors);
  fr.words[1] = (size_t)s.max_voxels * 3;
  fr.base[2] = reinterpret_cast<uint32_t *>(num_points_per_voxel);
  fr.words[2] = (size_t)s.max_voxels;
  fr.base[3] = reinterpret_cast<uint32_t *>(w.keys);
  fr.words[3] = (size_t)cap * 2;
  fr.base[4] = w.is_first;
  fr.words[4] = (size_t)n;
  size_t most = 0;
  for (int g = 0; g < kFillRegions; ++g) {
    fr.value[g] = g == 3 ? 0xffffffffu : 0u;
    most = fr.words[g] > most ? fr.words[g] : most;
  }
  lc.begin("voxFillRegions");
  voxFillRegions<<<gridFor(most / 4 + 1, 4096), kBlock, 0, lc.stream>>>(fr);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;

  const int blocks = gridFor((size_t)n);
  lc.begin("voxCellSlots");
  voxCellSlots<<<blocks, kBlock, 0, lc.stream>>>(points, voxel_size, coors_range, n,
                                                  s.num_features, w.keys, cap, w.pairs_a);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;

  // points grouped by table slot, the points of a slot in their input order
  lc.begin("radixSortPairs");
  bool in_b = false;
  e = device_sort::sortKeys<unsigned long long>(lc.stream, w.library, w.pairs_a, w.pairs_b, (size_t)n,
                                                bitsFor(cap), &in_b);
  lc.end();
  if (e != hipSuccess) return e;
  const unsigned long long *sorted = in_b ? w.pairs_b : w.pairs_a;

  lc.begin("voxMarkFirst");
  voxMarkFirst<<<blocks, kBlock, 0, lc.stream>>>(sorted, n, cap, w.is_first);
  lc.end();
  if ((e = hipGetLastError()) != hipSuccess) return e;

  // first points in front of every point
  lc.begin("exclusiveScan");
  e = device_sort::prefixSums(lc.stream, w.library, w.is_first, w.voxel_of_first, (size_t)n, false);
  lc.end();
  if (e != hipSuccess) return e;

  lc.begin("voxAssign");
  voxAssign<<<blocks, kBlock, 0, lc.stream>>>(points, voxel_size, coors_range, sorted, w.is_first, w.voxel_of_first, n, cap, s.num_features,
                                               s.max_points, s.max_voxels, voxels, coors,
                                               num_points_per_voxel, voxel_num);
  lc.end();
  return hipGetLastError();
}

}  // namespace voxelization
}  // namespace mluop
