// Rulebook (indice pairs) construction for 3-D sparse convolution on gfx950.
//
// Contract (reference test/mlu_op_gtest/pb_gtest/src/zoo/get_indice_pairs/
// get_indice_pairs.cpp:234-406): for input row j = (n, d, h, w) and kernel
// offset k = (kd*KH + kh)*KW + kw the output coordinate along each axis is
// o = (i + pad - k_axis*dilation) / stride, valid when the division is exact
// and 0 <= o < O_axis.  Submanifold mode keeps a pair when some input row sits
// at the output coordinate (output row = that input row, the highest row index
// wins for duplicated coordinates); regular mode keeps every valid pair and
// numbers the distinct output cells in ascending linear order.  Inside one
// offset, pairs are listed by ascending input row; unused tails are -1.
//
// Kernel set
//   submanifold:  prepare (copy out_indices, clear the hash table, write the sorted-cell
//                 arrays and decide whether the rows are in strict cell order) -> insert
//                 rows into the hash table (returns at once for rows in order) -> probe
//                 (rows in order: search the sorted cells, offsets below the centre only
//                 where the kernel is centred; otherwise: the hash table), every wave of
//                 64 rows staging the pairs it found -> place: sums the staged counts in
//                 front of each wave and moves the pairs to their final positions
//   regular:      clear bitmap -> mark output cells + stage (output cell in place of the
//                 output row) -> bitmap popcount scan (ranks, out_indices) -> place, cells
//                 to ranks
// The stable order needs no sort: rows are visited in ascending order by
// construction (lane = row) and positions come from exclusive prefix sums.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "core/wave_scan.h"
#include "sparse_conv/rulebook.h"

namespace mluop {
namespace sparse_conv {
namespace {

constexpr int kBlock = 256;
constexpr int kWave = 64;
constexpr uint32_t kEmptyKey = 0xffffffffu;  // no cell index reaches 2^31
constexpr int kGroup = 8;                    // offsets resolved together per lane
constexpr int kMaxInlineOffsets = 128;       // kernel volumes with an in-argument offset table
constexpr int kWordsPerBlock = 256;  // bitmap words (64 cells each) per block, one a thread
constexpr int kSelfScanBlocks = 4096;  // up to here every workgroup sums the block counts in front of it

// Division of a non-negative int by a divisor fixed for the launch:
// n / d = (n * mul) >> (31 + shift) for every 0 <= n < 2^31, with shift = ceil(log2 d)
// and mul = ceil(2^(31 + shift) / d) < 2^32.  (n * mul exceeds n / d * 2^(31+shift)
// by less than 2^(31+shift) / d, too little to reach the next quotient.)
struct FastDiv {
  uint32_t mul;
  int shift;
};

inline FastDiv makeFastDiv(int d) {
  FastDiv f;
  f.shift = 0;
  while ((1ll << f.shift) < (long long)d) ++f.shift;
  const unsigned long long p = 1ull << (31 + f.shift);
  f.mul = (uint32_t)((p + (unsigned long long)d - 1) / (unsigned long long)d);
  return f;
}

__device__ __forceinline__ int fastDiv(int n, FastDiv f) {
  return (int)(((unsigned long long)(uint32_t)n * f.mul) >> (31 + f.shift));
}

struct GeomDev {
  int batch;
  int out[3];
  int ks[3];
  int pad[3];
  int stride[3];
  int dil[3];
  int K;
  int L;
  FastDiv by_stride[3];
  FastDiv by_out_volume;  // out[0] * out[1] * out[2]
  FastDiv by_out_plane;   // out[1] * out[2]
  FastDiv by_out_width;   // out[2]
};

// Home slot of a cell (before masking): the run of 16 cells along W it belongs
// to is hashed, the position inside the run is kept.  Neighbours along W have
// neighbouring home slots, so one window of consecutive keys answers the
// probes of all kernel positions along W.
__device__ __forceinline__ uint32_t hashCell(uint32_t key) {
  uint32_t h = (key >> 4) * 0x9E3779B1u;
  h ^= h >> 15;
  return (h << 4) | (key & 15u);
}

__device__ __forceinline__ int4 loadCoord(const int32_t *indices, int j, bool aligned) {
  if (aligned) return reinterpret_cast<const int4 *>(indices)[j];
  const int32_t *p = indices + 4 * (size_t)j;
  return make_int4(p[0], p[1], p[2], p[3]);
}

__device__ __forceinline__ void storeCoord(int32_t *dst, int j, int4 v, bool aligned) {
  if (aligned) {
    reinterpret_cast<int4 *>(dst)[j] = v;
  } else {
    int32_t *p = dst + 4 * (size_t)j;
    p[0] = v.x; p[1] = v.y; p[2] = v.z; p[3] = v.w;
  }
}

// Output coordinate along one axis; -1 when this (input, offset) has none.
__device__ __forceinline__ int axisOut(int i, int pad, int kk, int dil, int stride, FastDiv by_stride,
                                       int osize) {
  int num = i + pad - kk * dil;
  if (num < 0) return -1;
  int o = num;
  if (stride != 1) {
    o = fastDiv(num, by_stride);
    if (o * stride != num) return -1;
  }
  return o < osize ? o : -1;
}

// Strictly below in (n, d, h, w) order, which is the order of linear cell indices.
__device__ __forceinline__ bool coordBelow(int4 a, int4 b) {
  if (a.x != b.x) return a.x < b.x;
  if (a.y != b.y) return a.y < b.y;
  if (a.z != b.z) return a.z < b.z;
  return a.w < b.w;
}

// Row j and the row before it are out of cell order (or equal): the rulebook's report
// will say so.  *rows_in_order was set to 1 by the first launch.
__device__ __forceinline__ void noteRowOrder(const int32_t *indices, int j, int4 c, bool aligned,
                                             int32_t *rows_in_order) {
  if (j > 0 && !coordBelow(loadCoord(indices, j - 1, aligned), c)) *rows_in_order = 0;
}

// The rulebook's report to the host: the flag first, then the stamp the host looks for.
__device__ __forceinline__ void fileReport(bool rows_in_order, const RulebookReportTarget &report) {
  if (report.stamp_word == nullptr) return;
  *report.order_word = rows_in_order ? 1u : 0u;
  __threadfence_system();
  __hip_atomic_store(report.stamp_word, report.stamp, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Up to three ranges of 32-bit words, each set to its own value (16-byte stores: every
// count is a multiple of 4 and every range 16-byte aligned, as workspace blocks are; a
// caller's tensor that is not goes word by word).  Also raises the rows-in-order flag.
struct FillRanges {
  uint32_t *dst[3];
  size_t n[3];
  uint32_t value[3];
};

__global__ __launch_bounds__(kBlock) void rbFill(FillRanges r, int32_t *rows_in_order) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *rows_in_order = 1;
  const size_t stride = (size_t)gridDim.x * kBlock;
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    if (r.n[i] == 0) continue;
    const uint32_t v = r.value[i];
    if ((reinterpret_cast<uintptr_t>(r.dst[i]) & 15u) == 0 && (r.n[i] & 3u) == 0) {
      uint4 *d4 = reinterpret_cast<uint4 *>(r.dst[i]);
      const size_t n4 = r.n[i] / 4;
      for (size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x; t < n4; t += stride)
        d4[t] = make_uint4(v, v, v, v);
    } else {
      for (size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x; t < r.n[i]; t += stride) r.dst[i][t] = v;
    }
  }
}

// Rows that arrive in strict cell order (every coordinate inside the space, every row's
// linear cell above its predecessor's) need no table: the array of their cells is sorted, a
// cell's place in it is the row that sits there, and looking a neighbour up is a search.
// What the searching kernel reads:
//   cells[i]    the linear cell of row i, then 0xffffffff up to the array's capacity
//   samples[s]  cells[s << shift], then 0xffffffff up to n_pad (a power of two that the
//               searching workgroup keeps in LDS: the search's first steps cost no memory
//               round trip, the last `shift` steps walk 2^shift consecutive cells)
//   unordered   a 64-bit word that holds this call's stamp (a value no earlier call wrote)
//               when the rows are NOT in strict cell order: nothing needs clearing first
struct SortedCells {
  uint32_t *cells;
  uint32_t *samples;
  unsigned long long *unordered;
  unsigned long long stamp;
  int capacity;  // entries of cells[]
  int shift;
  int n_pad;     // entries of samples[]
  // kernel edges odd and padding = dilation * (edge - 1) / 2: offset K - 1 - k mirrors k
  bool mirror;
  int mirror_groups_per_slice;  // groups of offsets a blockIdx.y slice of the probe takes then
};
constexpr int kMaxSamples = 4096;

__device__ __forceinline__ bool rowsUnordered(const SortedCells &sc) { return *sc.unordered == sc.stamp; }

// First launch of a submanifold rulebook: clears the hash table (needed only when the rows
// turn out unordered, which no launch knows before this one has finished), copies the
// coordinates to out_indices, writes the sorted-cell arrays and decides whether they may be
// used.
__global__ __launch_bounds__(kBlock) void rbSubmPrepare(GeomDev g, const int32_t *indices, bool aligned,
                                                        int32_t *out_indices, int out_rows,
                                                        FillRanges table, SortedCells sc,
                                                        bool never_sorted) {
  const size_t n_threads = (size_t)gridDim.x * kBlock;
  const size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x;
  {
    uint4 *d4 = reinterpret_cast<uint4 *>(table.dst[0]);  // capacity is a multiple of 64
    const size_t n4 = table.n[0] / 4;
    const uint32_t v = table.value[0];
    for (size_t t = tid; t < n4; t += n_threads) d4[t] = make_uint4(v, v, v, v);
  }
  if (never_sorted) {
    if (tid == 0) *sc.unordered = sc.stamp;
  } else {
    const int n_real = (g.L + (1 << sc.shift) - 1) >> sc.shift;
    for (size_t t = tid; t < (size_t)sc.n_pad; t += n_threads)
      if ((int)t >= n_real) sc.samples[t] = kEmptyKey;
  }
  const int j = (int)tid;
  if (j < g.L) {
    const int4 c = loadCoord(indices, j, aligned);
    if (j < out_rows) storeCoord(out_indices, j, c, aligned);
    if (!never_sorted) {
      const bool in_range = (unsigned)c.x < (unsigned)g.batch && (unsigned)c.y < (unsigned)g.out[0] &&
                            (unsigned)c.z < (unsigned)g.out[1] && (unsigned)c.w < (unsigned)g.out[2];
      const uint32_t cell =
          in_range ? (uint32_t)(((c.x * g.out[0] + c.y) * g.out[1] + c.z) * g.out[2] + c.w) : kEmptyKey;
      bool bad = !in_range;
      if (j > 0 && !coordBelow(loadCoord(indices, j - 1, aligned), c)) bad = true;
      if (bad) *sc.unordered = sc.stamp;
      sc.cells[j] = cell;
      if ((j & ((1 << sc.shift) - 1)) == 0) sc.samples[j >> sc.shift] = cell;
    }
  } else {
    if (j < out_rows) storeCoord(out_indices, j, make_int4(-1, -1, -1, -1), aligned);
    if (!never_sorted && j < sc.capacity) sc.cells[j] = kEmptyKey;
  }
}

// Open-addressing table over linear cell indices, for rows in any order: keys[] holds the
// cell (or kEmptyKey), vals[] the highest row index stored for that cell.  32-bit atomics
// only: a 64-bit compare-and-swap costs several times more here.  Returns at once when the
// rows are in cell order.
__global__ __launch_bounds__(kBlock) void rbSubmInsert(GeomDev g, const int32_t *indices,
                                                       bool aligned, uint32_t *keys,
                                                       int32_t *vals, uint32_t mask,
                                                       SortedCells sc, int32_t *pairs) {
  if (!rowsUnordered(sc)) return;
  int j = blockIdx.x * kBlock + threadIdx.x;
  if (j < g.L) {
    // Every pair slot starts as -1; the kernel that places the pairs overwrites the slots in
    // front of each offset's pair count.  Plain stores that nobody waits for, under the
    // table's atomics.
    for (int k = 0; k < g.K; ++k) {
      pairs[(size_t)k * 2 * g.L + j] = -1;
      pairs[((size_t)k * 2 + 1) * g.L + j] = -1;
    }
    int4 c = loadCoord(indices, j, aligned);
    bool in_range = (unsigned)c.x < (unsigned)g.batch && (unsigned)c.y < (unsigned)g.out[0] &&
                    (unsigned)c.z < (unsigned)g.out[1] && (unsigned)c.w < (unsigned)g.out[2];
    if (in_range) {
      const uint32_t cell =
          (uint32_t)(((c.x * g.out[0] + c.y) * g.out[1] + c.z) * g.out[2] + c.w);
      uint32_t slot = hashCell(cell) & mask;
      while (true) {
        const uint32_t old = atomicCAS(&keys[slot], kEmptyKey, cell);
        if (old == kEmptyKey || old == cell) {
          atomicMax(&vals[slot], j);
          break;
        }
        slot = (slot + 1) & mask;
      }
    }
  }
}

// ---- pairs to their final positions -----------------------------------------------
//
// A pair's position inside its offset is the number of pairs earlier rows hold there.
// The probe kernels do not know it yet.  A wave (64 consecutive rows) resolving a slice of
// the offsets (blockIdx.y) owns one block of the staging buffer and stages the pairs it
// found there back to back, offset after offset, each offset's pairs in lane order:
// what crosses the kernel boundary is the pairs (a few per wave and offset) and not a slot
// for every (row, offset), and the block's lines are written whole (a slot array per
// offset with a few words used per wave left every line partly written, which the memory
// behind the cache turns into read-modify-write; that layout spent as long on staging as
// on probing).  counts[k][wave] gets the number of pairs of (offset, wave) in its low 8
// bits and their start inside the block above them.  rbPlacePairs then moves them: a
// workgroup adds up the counts in front of its 64 waves, scans its own, and copies the
// staged pairs to their final positions.
// (Looking back over earlier workgroups inside the probe kernel instead, single-pass-scan
// style, was built and measured: all workgroups finish probing at the same moment, so
// the look-back degenerates into a chain over hundreds of workgroups per offset; 400 us.)
struct Staging {
  int32_t *stage;       // blocks of block_ints: submanifold: output row << 6 | lane; regular: output cell
  uint8_t *stage_lane;  // same blocks, regular mode only: lane of the staged pair
  int32_t *counts;      // [K, n_wave]: pairs | start in the block << 8
  int n_wave;
  int k_per_slice;      // offsets per blockIdx.y slice
  int block_ints;       // k_per_slice * 64
  int mirror_k_per_slice;  // offsets per slice where only the offsets below the centre are probed
};

__device__ __forceinline__ size_t stageBlock(const Staging &st, int slice, int wave) {
  return ((size_t)slice * st.n_wave + wave) * (size_t)st.block_ints;
}

// Stages the pairs of offsets k_first .. k_first + N - 1 (those below k_end); `run` is the
// number of pairs the wave has staged in its block so far (the same in every lane).
template <bool SUBM, int N>
__device__ __forceinline__ void stagePairs(const int (&res)[N], int k_first, int k_end, int j,
                                           const Staging &st, int *run) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wt = j >> 6;
  const unsigned long long lt_mask = (1ull << lane) - 1ull;
  const size_t block = stageBlock(st, blockIdx.y, wt);
  int my_entry = 0;  // lane u keeps the count word of offset k_first + u
#pragma unroll
  for (int u = 0; u < N; ++u) {
    const int k = k_first + u;
    if (k < k_end) {
      const unsigned long long b = __ballot(res[u] >= 0);
      if (res[u] >= 0) {
        const size_t at = block + (size_t)(*run + __popcll(b & lt_mask));
        if (SUBM) {
          st.stage[at] = (res[u] << 6) | lane;
        } else {
          st.stage[at] = res[u];
          st.stage_lane[at] = (uint8_t)lane;
        }
      }
      const int n = __popcll(b);
      if (lane == u) my_entry = n | (*run << 8);
      *run += n;
    }
  }
  if (lane < N && k_first + lane < k_end) st.counts[(size_t)(k_first + lane) * st.n_wave + wt] = my_entry;
}

// Marks the output cells cell[0..N) of the 64 lanes (kEmptyKey: none) in the bitmap.
// Rows in cell order walk along w, so the lanes of a wavefront mark runs of cells
// in the same bitmap word: a run's bits are gathered at its last lane, which alone
// goes to memory (atomics on the bitmap are what a marking kernel would wait for).  Lanes
// with no output cell join the run in front of them; a lane whose word is below one
// in front of it (rows out of order) marks its cell by itself.
template <int N>
__device__ __forceinline__ void markCells(const uint32_t (&cell)[N], unsigned long long *bitmap) {
  const int lane = threadIdx.x & (kWave - 1);
  uint32_t word_at[N];
  unsigned long long bits[N];
  uint32_t alone = 0;
#pragma unroll
  for (int u = 0; u < N; ++u) {
    const bool valid = cell[u] != kEmptyKey;
    const uint32_t mine = cell[u] >> 6;
    const uint32_t run = waveInclusiveMax(valid ? mine : 0u);
    const bool joins = valid && run == mine;
    if (valid && !joins) alone |= 1u << u;
    uint32_t lo = 0, hi = 0;
    if (joins) {
      lo = (cell[u] & 32u) ? 0u : 1u << (cell[u] & 31u);
      hi = (cell[u] & 32u) ? 1u << (cell[u] & 31u) : 0u;
    }
    waveRunInclusiveOr(run, &lo, &hi);
    const uint32_t run_next = __shfl_down(run, 1, kWave);
    const bool last = lane == kWave - 1 || run_next != run;
    word_at[u] = run;
    bits[u] = last ? ((unsigned long long)hi << 32) | lo : 0ull;
  }
  // (a stale word from the cache only costs an atomic that changes nothing)
  unsigned long long seen[N];
#pragma unroll
  for (int u = 0; u < N; ++u) seen[u] = bits[u] ? bitmap[word_at[u]] : ~0ull;
#pragma unroll
  for (int u = 0; u < N; ++u)
    if ((seen[u] & bits[u]) != bits[u]) atomicOr(bitmap + word_at[u], bits[u]);
  if (__any(alone != 0)) {
#pragma unroll
    for (int u = 0; u < N; ++u) {
      if (alone & (1u << u)) {
        const unsigned long long bit = 1ull << (cell[u] & 63);
        unsigned long long *word = bitmap + (cell[u] >> 6);
        if ((*word & bit) == 0) atomicOr(word, bit);
      }
    }
  }
}

// One wavefront per 64 consecutive rows, offsets in groups of kGroup so that a
// lane keeps kGroup independent table probes in flight.  For every offset:
// resolve the pair (submanifold: table lookup -> output row; regular: output
// cell, marked in the bitmap), store it as a candidate at [k][row] and record
// how many lanes of the wave produced one.
template <bool SUBM>
__global__ __launch_bounds__(kBlock) void rbProbeCount(GeomDev g,
                                                       const int32_t *indices, bool aligned,
                                                       const uint32_t *keys, const int32_t *vals,
                                                       uint32_t mask, unsigned long long *bitmap,
                                                       Staging staging, int k_per_slice,
                                                       int32_t *rows_in_order, int32_t *pairs) {
  const int j = blockIdx.x * kBlock + threadIdx.x;
  // blockIdx.y selects a slice of the offsets: more waves in flight than rows alone give
  const int k_lo = blockIdx.y * k_per_slice;
  const int k_hi = k_lo + k_per_slice < g.K ? k_lo + k_per_slice : g.K;
  if ((j >> 6) >= staging.n_wave) return;  // whole wave beyond the last row
  const bool active = j < g.L;
  int4 c = make_int4(-1, 0, 0, 0);
  if (active) c = loadCoord(indices, j, aligned);
  if (!SUBM && active && blockIdx.y == 0) noteRowOrder(indices, j, c, aligned, rows_in_order);
  const bool n_ok = active && (unsigned)c.x < (unsigned)g.batch;
  // (kd, kh, kw) of the slice's first offset, advanced by one offset a step: all of it
  // the same for every lane
  int kd = k_lo / (g.ks[1] * g.ks[2]);
  int kh = (k_lo - kd * g.ks[1] * g.ks[2]) / g.ks[2];
  int kw = k_lo - (kd * g.ks[1] + kh) * g.ks[2];
  // The cell of (row, offset) is plane + ow: `plane` (the cell of w = 0 in the output line,
  // or -1 when (kd, kh) has no output line for this row) is computed again only when kh or
  // kd changes, once in ks[2] offsets.
  int base_d = 0, plane = -1;
  bool new_d = true, new_h = true;
  int staged = 0;
  for (int k0 = k_lo; k0 < k_hi; k0 += kGroup) {
    uint32_t cell[kGroup];
    int res[kGroup];
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      cell[u] = kEmptyKey;
      res[u] = -1;
      const int k = k0 + u;
      if (k < k_hi) {
        if (new_d) {
          const int od = axisOut(c.y, g.pad[0], kd, g.dil[0], g.stride[0], g.by_stride[0], g.out[0]);
          base_d = n_ok && od >= 0 ? (c.x * g.out[0] + od) * g.out[1] : -1;
        }
        if (new_h) {
          const int oh = axisOut(c.z, g.pad[1], kh, g.dil[1], g.stride[1], g.by_stride[1], g.out[1]);
          plane = base_d >= 0 && oh >= 0 ? (base_d + oh) * g.out[2] : -1;
        }
        const int ow = axisOut(c.w, g.pad[2], kw, g.dil[2], g.stride[2], g.by_stride[2], g.out[2]);
        if ((plane | ow) >= 0) cell[u] = (uint32_t)(plane + ow);
        new_d = false;
        new_h = false;
        if (++kw == g.ks[2]) {
          kw = 0;
          new_h = true;
          if (++kh == g.ks[1]) {
            kh = 0;
            ++kd;
            new_d = true;
          }
        }
      }
    }
    if (SUBM) {
      uint32_t slot[kGroup];
      uint32_t pending = 0, hit = 0;
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        slot[u] = hashCell(cell[u]) & mask;
        if (cell[u] != kEmptyKey) pending |= 1u << u;
      }
      // Every round issues one load per unresolved probe of the lane, all
      // independent; the wave leaves when its longest probe sequence ends.
      while (__any(pending != 0)) {
        uint32_t key[kGroup];
#pragma unroll
        for (int u = 0; u < kGroup; ++u) {
          key[u] = kEmptyKey;
          if (pending & (1u << u)) key[u] = keys[slot[u]];
        }
#pragma unroll
        for (int u = 0; u < kGroup; ++u) {
          if (pending & (1u << u)) {
            if (key[u] == kEmptyKey) {
              pending &= ~(1u << u);
            } else if (key[u] == cell[u]) {
              pending &= ~(1u << u);
              hit |= 1u << u;
            } else {
              slot[u] = (slot[u] + 1) & mask;
            }
          }
        }
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        if (hit & (1u << u)) res[u] = vals[slot[u]];
      }
    } else {
#pragma unroll
      for (int u = 0; u < kGroup; ++u)
        if (cell[u] != kEmptyKey) res[u] = (int)cell[u];
      markCells<kGroup>(cell, bitmap);
      // every pair slot of this row and these offsets starts out as -1; the kernel that
      // places the pairs overwrites the front of each list afterwards
      if (active) {
        for (int k = k0; k < k0 + kGroup && k < k_hi; ++k) {
          pairs[(size_t)(2 * k) * g.L + j] = -1;
          pairs[(size_t)(2 * k + 1) * g.L + j] = -1;
        }
      }
    }
    stagePairs<SUBM, kGroup>(res, k0, k_hi, j, staging, &staged);
  }
}

// Regular mode with a stride above 1 and a small kernel (KD x KH x KW known at compile
// time).  Of the K offsets of a row only those whose kernel position has the right
// remainder on every axis give an output cell: one in eight at stride 2.  Marking cells is
// the expensive part (a dozen cross-lane steps per marked cell), so it runs over the
// candidates of a row, the m-th valid kernel position of every axis (mark_n[a] of them at
// most: 2 x 2 x 2 for a 3 x 3 x 3 kernel at stride 2, one for 2 x 2 x 2), and not over the
// offsets; staging, which must go offset by offset, is a bit test and an addition per
// offset once the output coordinate of every kernel position is known.  blockIdx.y
// slices both: the candidates along d for marking, the offsets for staging.
template <int KD, int KH, int KW>
__global__ __launch_bounds__(kBlock) void rbProbeStrided(GeomDev g, const int32_t *indices, bool aligned,
                                                          unsigned long long *bitmap, Staging staging,
                                                          int k_per_slice, int mark_d, int mark_h,
                                                          int32_t *rows_in_order, int32_t *pairs) {
  constexpr int K = KD * KH * KW;
  const int j = blockIdx.x * kBlock + threadIdx.x;
  const int k_lo = blockIdx.y * k_per_slice;
  const int k_hi = k_lo + k_per_slice < K ? k_lo + k_per_slice : K;
  if ((j >> 6) >= staging.n_wave) return;  // whole wave beyond the last row
  const bool active = j < g.L;
  int4 c = make_int4(-1, 0, 0, 0);
  if (active) {
    c = loadCoord(indices, j, aligned);
    if (blockIdx.y == 0) noteRowOrder(indices, j, c, aligned, rows_in_order);
    // every pair slot of this row starts out as -1 for the slice's offsets; the kernel that
    // places the pairs overwrites the front of each list afterwards
    for (int k = k_lo; k < k_hi; ++k) {
      pairs[(size_t)(2 * k) * g.L + j] = -1;
      pairs[(size_t)(2 * k + 1) * g.L + j] = -1;
    }
  }
  const bool n_ok = active && (unsigned)c.x < (unsigned)g.batch;
  // output coordinate of every kernel position, or -1
  int od[KD], oh[KH], ow[KW];
#pragma unroll
  for (int t = 0; t < KD; ++t)
    od[t] = n_ok ? axisOut(c.y, g.pad[0], t, g.dil[0], g.stride[0], g.by_stride[0], g.out[0]) : -1;
#pragma unroll
  for (int t = 0; t < KH; ++t) oh[t] = axisOut(c.z, g.pad[1], t, g.dil[1], g.stride[1], g.by_stride[1], g.out[1]);
#pragma unroll
  for (int t = 0; t < KW; ++t) ow[t] = axisOut(c.w, g.pad[2], t, g.dil[2], g.stride[2], g.by_stride[2], g.out[2]);
  // the valid ones in ascending kernel position: the candidates
  int cd[KD], ch[KH], cw[KW];
  {
    int n = 0;
#pragma unroll
    for (int t = 0; t < KD; ++t) cd[t] = -1;
#pragma unroll
    for (int t = 0; t < KD; ++t) {
#pragma unroll
      for (int m = 0; m < KD; ++m)
        if (od[t] >= 0 && n == m) cd[m] = od[t];
      n += od[t] >= 0 ? 1 : 0;
    }
    n = 0;
#pragma unroll
    for (int t = 0; t < KH; ++t) ch[t] = -1;
#pragma unroll
    for (int t = 0; t < KH; ++t) {
#pragma unroll
      for (int m = 0; m < KH; ++m)
        if (oh[t] >= 0 && n == m) ch[m] = oh[t];
      n += oh[t] >= 0 ? 1 : 0;
    }
    n = 0;
#pragma unroll
    for (int t = 0; t < KW; ++t) cw[t] = -1;
#pragma unroll
    for (int t = 0; t < KW; ++t) {
#pragma unroll
      for (int m = 0; m < KW; ++m)
        if (ow[t] >= 0 && n == m) cw[m] = ow[t];
      n += ow[t] >= 0 ? 1 : 0;
    }
  }
  // marking: candidate m_d along d goes to slice m_d % gridDim.y
#pragma unroll
  for (int md = 0; md < KD; ++md) {
    if (md >= mark_d || md % (int)gridDim.y != (int)blockIdx.y) continue;
#pragma unroll
    for (int mh = 0; mh < KH; ++mh) {
      if (mh >= mark_h) continue;
      uint32_t cell[KW];
      const int line = (cd[md] | ch[mh]) >= 0 ? ((c.x * g.out[0] + cd[md]) * g.out[1] + ch[mh]) * g.out[2] : -1;
#pragma unroll
      for (int mw = 0; mw < KW; ++mw) cell[mw] = (line | cw[mw]) >= 0 ? (uint32_t)(line + cw[mw]) : kEmptyKey;
      markCells<KW>(cell, bitmap);
    }
  }
  // staging: offset by offset, KW at a time
  int staged = 0;
#pragma unroll
  for (int kd = 0; kd < KD; ++kd) {
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) {
      const int k_first = (kd * KH + kh) * KW;
      if (k_first < k_lo || k_first >= k_hi) continue;
      int res[KW];
      const int line = (od[kd] | oh[kh]) >= 0 ? ((c.x * g.out[0] + od[kd]) * g.out[1] + oh[kh]) * g.out[2] : -1;
#pragma unroll
      for (int kw = 0; kw < KW; ++kw) res[kw] = (line | ow[kw]) >= 0 ? line + ow[kw] : -1;
      stagePairs<false, KW>(res, k_first, k_hi, j, staging, &staged);
    }
  }
}

// Offsets of a unit-stride kernel volume (at most kMaxInlineOffsets of them, kernel edges
// <= 32).  With stride 1 the output cell of (row, offset) is the row's own padded cell
// minus a per-offset constant, and whether it lies inside the output space is one bit per
// axis and kernel position, computed once per row.
struct UnitStrideOffsets {
  uint32_t packed[kMaxInlineOffsets];  // kd | kh << 8 | kw << 16
  uint32_t delta[kMaxInlineOffsets];   // linear distance from the padded cell
};

// Number of elements below t in a sorted array of n elements (n a power of two >= 4),
// three pivots a step; at(i) reads element i.
template <typename F>
__device__ __forceinline__ int countBelow(F at, int n, uint32_t t) {
  int base = 0;
  int len = n;
  while (len >= 4) {
    const int q = len >> 2;
    const uint32_t p1 = at(base + q - 1);
    const uint32_t p2 = at(base + 2 * q - 1);
    const uint32_t p3 = at(base + 3 * q - 1);
    base += ((p1 < t ? 1 : 0) + (p2 < t ? 1 : 0) + (p3 < t ? 1 : 0)) * q;
    len = q;
  }
  if (len == 2) base += at(base) < t ? 1 : 0;
  return base + (at(base) < t ? 1 : 0);
}

// Probe over the sorted cell array (rows in strict cell order, unit strides).  Offsets are
// taken in groups of KW consecutive ones that look at KW consecutive cells (KW = the kernel's
// width along W at dilation 1, or 1: every offset its own group), G groups a pass.
//
// The lowest cells that the 64 rows of a wave look for in one group ascend with the rows, so
// everything the wave can find lies between the places of its first and its last row's
// cell.  Two lanes per group search these two among the samples in LDS (one search for all
// groups of the pass), the wave copies the kSpan cells from there on to LDS with a few
// coalesced loads, and every lane finishes its own search inside that copy: no memory
// round trip per search step and a tenth of the instructions of a search per lane over the
// whole array.  A wave whose rows are spread so thin that its span is longer falls back to
// exactly that: per lane over the samples, then with three pivots a step over the 2^shift
// cells between two samples down to a stretch of kChunk cells, which is read in one go.
// Either way the cells found that belong to the group are the neighbours that exist, and
// their places are their rows.
//
// With `mirror` (kernel edges odd, padding = dilation * (edge - 1) / 2) only the offsets
// below the centre are probed: row o found from row i at offset k finds i at offset
// K - 1 - k, and since o ascends with i the list of K - 1 - k is the list of k with its
// columns exchanged; the centre offset pairs every row with itself.
//
// The wave also sets the pair slots of its rows to -1 for the offsets it resolves (and
// their mirror images), stores that nobody waits for; the kernel that places the pairs
// overwrites the front of each list afterwards.
constexpr int kChunk = 8;
constexpr int kSpan = 256;
constexpr int kSpanPad = 8;
struct CellQuad {
  uint32_t v[4];
};

template <int KW, int G>
__device__ __forceinline__ void sortedProbe(const GeomDev &g, const UnitStrideOffsets &tab,
                                            const int32_t *indices, bool aligned, const SortedCells &sc,
                                            const Staging &staging, int groups_per_slice, int32_t *pairs) {
  constexpr int N = G * KW;
  constexpr int QUADS = (kChunk + KW + 3) / 4;
  static_assert(N <= 32 && 2 * G <= kWave && KW <= kSpanPad, "bit masks, lanes, padding");
  __shared__ uint32_t s_samples[kMaxSamples];
  __shared__ uint32_t s_span[kBlock / kWave][G][kSpan + kSpanPad];
  if ((sc.n_pad & 1023) == 0) {
    for (int i = threadIdx.x; i < sc.n_pad / 4; i += kBlock)
      reinterpret_cast<uint4 *>(s_samples)[i] = reinterpret_cast<const uint4 *>(sc.samples)[i];
  } else {
    for (int i = threadIdx.x; i < sc.n_pad; i += kBlock) s_samples[i] = sc.samples[i];
  }
  const int j = blockIdx.x * kBlock + threadIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x >> 6;
  // offsets below k_all are probed, in groups [t_lo, t_hi) by this slice
  const int k_all = sc.mirror ? g.K / 2 : g.K;
  const int n_groups = (k_all + KW - 1) / KW;
  const int per_slice = sc.mirror ? sc.mirror_groups_per_slice : groups_per_slice;
  const int t_lo = blockIdx.y * per_slice;
  const int t_hi = t_lo + per_slice < n_groups ? t_lo + per_slice : n_groups;
  const int k_end = KW * t_hi < k_all ? KW * t_hi : k_all;
  const bool active = j < g.L;
  int4 c = make_int4(0, 0, 0, 0);
  if (active) {
    c = loadCoord(indices, j, aligned);
    for (int k = KW * t_lo; k < k_end; ++k) {
      pairs[(size_t)(2 * k) * g.L + j] = -1;
      pairs[(size_t)(2 * k + 1) * g.L + j] = -1;
      if (sc.mirror) {
        pairs[(size_t)(2 * (g.K - 1 - k)) * g.L + j] = -1;
        pairs[(size_t)(2 * (g.K - 1 - k) + 1) * g.L + j] = -1;
      }
    }
  }
  __syncthreads();
  if ((j >> 6) >= staging.n_wave || t_lo >= t_hi) return;  // nothing for this wave
  uint32_t ok_d = 0, ok_h = 0, ok_w = 0;
  for (int t = 0; t < g.ks[0]; ++t)
    ok_d |= (uint32_t)((unsigned)(c.y + g.pad[0] - t * g.dil[0]) < (unsigned)g.out[0]) << t;
  for (int t = 0; t < g.ks[1]; ++t)
    ok_h |= (uint32_t)((unsigned)(c.z + g.pad[1] - t * g.dil[1]) < (unsigned)g.out[1]) << t;
  for (int t = 0; t < g.ks[2]; ++t)
    ok_w |= (uint32_t)((unsigned)(c.w + g.pad[2] - t * g.dil[2]) < (unsigned)g.out[2]) << t;
  if (!active) ok_d = 0;
  const uint32_t padded = (((uint32_t)c.x * g.out[0] + (uint32_t)(c.y + g.pad[0])) * g.out[1] +
                           (uint32_t)(c.z + g.pad[1])) * g.out[2] + (uint32_t)(c.w + g.pad[2]);
  const uint32_t *cells = sc.cells;
  auto sample = [&](int i) { return s_samples[i]; };
  int staged = 0;
  for (int t0 = t_lo; t0 < t_hi; t0 += G) {
    uint32_t low[G];     // lowest cell of the group (modulo 2^32: it may lie below cell 0)
    uint32_t target[G];  // what is searched for: the lowest cell, or cell 0
    uint32_t want = 0;
    int res[N];
    unsigned long long wanting[G];  // lanes that look for something in the group
#pragma unroll
    for (int a = 0; a < G; ++a) {
      const int t = t0 + a < t_hi ? t0 + a : t_hi - 1;  // clamped: a valid table entry
      low[a] = padded - tab.delta[KW * t + KW - 1];
#pragma unroll
      for (int d = 0; d < KW; ++d) {
        const int u = KW * a + (KW - 1 - d);
        const int k = KW * t + (KW - 1 - d);
        const uint32_t pk = tab.packed[k];
        res[u] = -1;
        if (t0 + a < t_hi && k < k_end &&
            ((ok_d >> (pk & 0xff)) & (ok_h >> ((pk >> 8) & 0xff)) & (ok_w >> (pk >> 16)) & 1u))
          want |= 1u << u;
      }
      const bool any = ((want >> (KW * a)) & ((1u << KW) - 1u)) != 0;
      target[a] = any && (int32_t)low[a] >= 0 ? low[a] : 0u;
      wanting[a] = __ballot(any);
    }
    // where the wave's span of every group starts, and whether kSpan cells cover it
    int start[G];
    bool fits = true;
    {
      uint32_t bound = 0;
#pragma unroll
      for (int a = 0; a < G; ++a) {
        const int l_first = wanting[a] ? __ffsll((long long)wanting[a]) - 1 : 0;
        const int l_last = wanting[a] ? 63 - __clzll((long long)wanting[a]) : 0;
        const uint32_t t_first = (uint32_t)__builtin_amdgcn_readlane((int)target[a], l_first);
        const uint32_t t_last = (uint32_t)__builtin_amdgcn_readlane((int)target[a], l_last);
        if (lane == 2 * a) bound = t_first;
        if (lane == 2 * a + 1) bound = t_last;
      }
      const int below = countBelow(sample, sc.n_pad, bound);
      // the first cell >= bound lies in (sample below - 1 .. sample below] << shift
      const int from = (below - 1) * (1 << sc.shift) + 1;
      const int edge = (lane & 1) ? below << sc.shift : (from > 0 ? from : 0);
#pragma unroll
      for (int a = 0; a < G; ++a) {
        start[a] = __builtin_amdgcn_readlane(edge, 2 * a);
        const int last = __builtin_amdgcn_readlane(edge, 2 * a + 1);
        if (wanting[a] != 0 && last - start[a] > kSpan) fits = false;
      }
    }
    if (fits) {
#pragma unroll
      for (int a = 0; a < G; ++a) {
        if (wanting[a] == 0) continue;
        uint32_t piece[kSpan / kWave], extra = 0;
#pragma unroll
        for (int i = 0; i < kSpan / kWave; ++i) piece[i] = cells[start[a] + i * kWave + lane];
        if (lane < kSpanPad) extra = cells[start[a] + kSpan + lane];
#pragma unroll
        for (int i = 0; i < kSpan / kWave; ++i) s_span[wv][a][i * kWave + lane] = piece[i];
        if (lane < kSpanPad) s_span[wv][a][kSpan + lane] = extra;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int a = 0; a < G; ++a) {
        if (wanting[a] == 0) continue;
        const uint32_t *span = s_span[wv][a];
        const int at = countBelow([&](int i) { return span[i]; }, kSpan, target[a]);
#pragma unroll
        for (int i = 0; i < KW; ++i) {
          const uint32_t rel = span[at + i] - low[a];
#pragma unroll
          for (int d = 0; d < KW; ++d) {
            const int u = KW * a + (KW - 1 - d);
            if (rel == (uint32_t)d && (want & (1u << u))) res[u] = start[a] + at + i;
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    } else {
#pragma unroll
      for (int a = 0; a < G; ++a) {
        if (wanting[a] == 0) continue;
        const int below = countBelow(sample, sc.n_pad, target[a]);
        const int from = (below - 1) * (1 << sc.shift) + 1;
        int first = from > 0 ? from : 0;
        int len = 1 << sc.shift;
        while (len > kChunk) {
          if (len >= 4 * kChunk) {
            const int q = len >> 2;
            const uint32_t p1 = cells[first + q - 1];
            const uint32_t p2 = cells[first + 2 * q - 1];
            const uint32_t p3 = cells[first + 3 * q - 1];
            first += ((p1 < target[a] ? 1 : 0) + (p2 < target[a] ? 1 : 0) + (p3 < target[a] ? 1 : 0)) * q;
            len = q;
          } else {
            const int half = len >> 1;
            first += cells[first + half - 1] < target[a] ? half : 0;
            len = half;
          }
        }
        // the first cell >= target is one of first .. first + kChunk
        CellQuad found[QUADS];
#pragma unroll
        for (int i = 0; i < QUADS; ++i) found[i] = *reinterpret_cast<const CellQuad *>(cells + first + 4 * i);
#pragma unroll
        for (int i = 0; i < 4 * QUADS; ++i) {
          const uint32_t rel = found[i >> 2].v[i & 3] - low[a];
#pragma unroll
          for (int d = 0; d < KW; ++d) {
            const int u = KW * a + (KW - 1 - d);
            if (rel == (uint32_t)d && (want & (1u << u))) res[u] = first + i;
          }
        }
      }
    }
    stagePairs<true, N>(res, KW * t0, k_end, j, staging, &staged);
  }
}

// Submanifold probe for unit strides (the usual case), kernel edges <= 32 and
// K <= kMaxInlineOffsets: over the sorted cells when the rows came in cell order, through
// the hash table otherwise (the per-offset work is a few integer instructions around the
// probe itself).
__global__ __launch_bounds__(kBlock) void rbSubmProbeUnitStride(
    GeomDev g, UnitStrideOffsets tab, const int32_t *indices, bool aligned, const uint32_t *keys,
    const int32_t *vals, uint32_t mask, Staging staging, int k_per_slice, SortedCells sc,
    int32_t *pairs) {
  if (!rowsUnordered(sc)) {
    sortedProbe<1, 4>(g, tab, indices, aligned, sc, staging, k_per_slice, pairs);
    return;
  }
  const int j = blockIdx.x * kBlock + threadIdx.x;
  const int k_lo = blockIdx.y * k_per_slice;
  const int k_hi = k_lo + k_per_slice < g.K ? k_lo + k_per_slice : g.K;
  if ((j >> 6) >= staging.n_wave) return;  // whole wave beyond the last row
  const bool active = j < g.L;
  int4 c = make_int4(-1, 0, 0, 0);
  if (active) c = loadCoord(indices, j, aligned);
  const bool n_ok = active && (unsigned)c.x < (unsigned)g.batch;
  // bit t of an axis mask: kernel position t lands inside the output space
  uint32_t ok_d = 0, ok_h = 0, ok_w = 0;
  for (int t = 0; t < g.ks[0]; ++t)
    ok_d |= (uint32_t)((unsigned)(c.y + g.pad[0] - t * g.dil[0]) < (unsigned)g.out[0]) << t;
  for (int t = 0; t < g.ks[1]; ++t)
    ok_h |= (uint32_t)((unsigned)(c.z + g.pad[1] - t * g.dil[1]) < (unsigned)g.out[1]) << t;
  for (int t = 0; t < g.ks[2]; ++t)
    ok_w |= (uint32_t)((unsigned)(c.w + g.pad[2] - t * g.dil[2]) < (unsigned)g.out[2]) << t;
  if (!n_ok) ok_d = 0;
  // modulo 2^32; exact for every cell inside the output space
  const uint32_t padded = (((uint32_t)c.x * g.out[0] + (uint32_t)(c.y + g.pad[0])) * g.out[1] +
                           (uint32_t)(c.z + g.pad[1])) * g.out[2] + (uint32_t)(c.w + g.pad[2]);
  int staged = 0;
  for (int k0 = k_lo; k0 < k_hi; k0 += kGroup) {
    uint32_t cell[kGroup], slot[kGroup];
    int res[kGroup];
    uint32_t pending = 0, hit = 0;
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      const int k = k0 + u < k_hi ? k0 + u : k_hi - 1;  // clamped: a valid table entry
      const uint32_t pk = tab.packed[k];
      const bool ok = k0 + u < k_hi &&
                      ((ok_d >> (pk & 0xff)) & (ok_h >> ((pk >> 8) & 0xff)) & (ok_w >> (pk >> 16)) & 1u);
      cell[u] = padded - tab.delta[k];
      slot[u] = hashCell(cell[u]) & mask;
      res[u] = -1;
      if (ok) pending |= 1u << u;
    }
    // Every round issues one load per unresolved probe of the lane, all
    // independent; the wave leaves when its longest probe sequence ends.
    while (__any(pending != 0)) {
      uint32_t key[kGroup];
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        key[u] = kEmptyKey;
        if (pending & (1u << u)) key[u] = keys[slot[u]];
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        if (pending & (1u << u)) {
          if (key[u] == cell[u]) {
            hit |= 1u << u;
            pending &= ~(1u << u);
          } else if (key[u] == kEmptyKey) {
            pending &= ~(1u << u);
          } else {
            slot[u] = (slot[u] + 1) & mask;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kGroup; ++u) {
      if (hit & (1u << u)) res[u] = vals[slot[u]];
    }
    stagePairs<true, kGroup>(res, k0, k_hi, j, staging, &staged);
  }
}

// Unit strides with a kernel KW (3 or 5) wide along W at dilation 1.  The KW
// offsets that differ only in kw look at KW consecutive cells; when those lie
// in one run of 16 their home slots are consecutive, and one load of the eight
// keys from the first home slot on holds the home slots plus the next steps of
// every probe sequence: walking it (a key equal to the cell is a hit, an empty
// slot a definite miss) settles nearly every probe of the wave in one memory
// round trip, where probing slot by slot costs one dependent round trip per
// step of the longest sequence among the wave's hundreds of probes.  Cells
// beyond a run boundary are served by a second window from the next run's
// first home slot.  Sequences that leave their window continue slot by slot.
constexpr int kWindow = 8;
struct KeyWindow {
  uint32_t k[kWindow];
};
constexpr int kGroupsPerPass = 3;  // (kd, kh) pairs resolved together per lane

template <int KW>
__global__ __launch_bounds__(kBlock) void rbSubmProbeRuns(
    GeomDev g, UnitStrideOffsets tab, const int32_t *indices, bool aligned, const uint32_t *keys,
    const int32_t *vals, uint32_t mask, Staging staging, int groups_per_slice, SortedCells sc,
    int32_t *pairs) {
  constexpr int N = kGroupsPerPass * KW;
  static_assert(KW <= kWindow && N <= 32, "window and bit masks");
  if (!rowsUnordered(sc)) {
    sortedProbe<KW, KW == 3 ? 2 : 3>(g, tab, indices, aligned, sc, staging, groups_per_slice, pairs);
    return;
  }
  const int j = blockIdx.x * kBlock + threadIdx.x;
  const int n_groups = g.K / KW;
  const int t_lo = blockIdx.y * groups_per_slice;
  const int t_hi = t_lo + groups_per_slice < n_groups ? t_lo + groups_per_slice : n_groups;
  if ((j >> 6) >= staging.n_wave) return;  // whole wave beyond the last row
  const bool active = j < g.L;
  int4 c = make_int4(-1, 0, 0, 0);
  if (active) c = loadCoord(indices, j, aligned);
  const bool n_ok = active && (unsigned)c.x < (unsigned)g.batch;
  uint32_t ok_d = 0, ok_h = 0, ok_w = 0;
  for (int t = 0; t < g.ks[0]; ++t)
    ok_d |= (uint32_t)((unsigned)(c.y + g.pad[0] - t * g.dil[0]) < (unsigned)g.out[0]) << t;
  for (int t = 0; t < g.ks[1]; ++t)
    ok_h |= (uint32_t)((unsigned)(c.z + g.pad[1] - t * g.dil[1]) < (unsigned)g.out[1]) << t;
#pragma unroll
  for (int t = 0; t < KW; ++t)
    ok_w |= (uint32_t)((unsigned)(c.w + g.pad[2] - t) < (unsigned)g.out[2]) << t;
  if (!n_ok) ok_d = 0;
  const uint32_t padded = (((uint32_t)c.x * g.out[0] + (uint32_t)(c.y + g.pad[0])) * g.out[1] +
                           (uint32_t)(c.z + g.pad[1])) * g.out[2] + (uint32_t)(c.w + g.pad[2]);
  int staged = 0;
  for (int t0 = t_lo; t0 < t_hi; t0 += kGroupsPerPass) {
    uint32_t cell[N], slot[N];
    int res[N];
    uint32_t want = 0, pending = 0, hit = 0;
#pragma unroll
    for (int a = 0; a < kGroupsPerPass; ++a) {
      const int t = t0 + a < t_hi ? t0 + a : t_hi - 1;  // clamped: a valid table entry
      const uint32_t pk = tab.packed[KW * t];
      const bool ok_t = t0 + a < t_hi && ((ok_d >> (pk & 0xff)) & (ok_h >> ((pk >> 8) & 0xff)) & 1u);
      const uint32_t c0 = padded - tab.delta[KW * t + KW - 1];  // kw = KW-1 is the lowest cell
      const int r = (int)(c0 & 15u);                            // position of c0 in its run
      // cell c0 + d belongs to kw = KW-1-d; it lies beyond c0's run when r + d > 15
      uint32_t want_a = 0, want_b = 0;
#pragma unroll
      for (int d = 0; d < KW; ++d) {
        const int u = KW * a + (KW - 1 - d);
        cell[u] = c0 + (uint32_t)d;
        res[u] = -1;
        if (ok_t && ((ok_w >> (KW - 1 - d)) & 1u)) {
          want |= 1u << u;
          if (r + d > 15) want_b |= 1u << d; else want_a |= 1u << d;
        }
      }
      // Window A starts at c0's home slot, window B at the home slot of the
      // next run's first cell; a window must end inside the table.
      const uint32_t sa = hashCell(c0) & mask;
      const uint32_t sb = hashCell(c0 + (uint32_t)(16 - r)) & mask;
      const bool load_a = want_a != 0 && sa + kWindow <= mask + 1u;
      const bool load_b = want_b != 0 && sb + kWindow <= mask + 1u;
      // A window is looked at once for all KW cells: where[d] becomes the place of the key
      // c0 + d (0..7 in window A, 8..15 in window B, -1 if it is in neither), empty_x gets
      // bit i set when slot i of the window is empty.  A cell whose key is in a window is a
      // hit wherever it sits (keys are unique in the table, and a key lies at or behind its
      // home slot); a cell without one is a miss for sure when its window has an empty slot
      // at or behind the cell's home slot, and goes on slot by slot behind the window
      // otherwise.
      int where[KW];
#pragma unroll
      for (int d = 0; d < KW; ++d) where[d] = -1;
      uint32_t empty_a = 0, empty_b = 0;
      KeyWindow win_a;
#pragma unroll
      for (int i = 0; i < kWindow; ++i) win_a.k[i] = kEmptyKey;
      if (load_a) win_a = *reinterpret_cast<const KeyWindow *>(keys + sa);
      if (__any(load_b)) {  // few waves have a lane whose cells cross a run boundary
        KeyWindow win_b;
#pragma unroll
        for (int i = 0; i < kWindow; ++i) win_b.k[i] = kEmptyKey;
        if (load_b) win_b = *reinterpret_cast<const KeyWindow *>(keys + sb);
#pragma unroll
        for (int i = 0; i < kWindow; ++i) {
          const uint32_t rel = win_b.k[i] - c0;
          if (win_b.k[i] == kEmptyKey) empty_b |= 1u << i;
#pragma unroll
          for (int d = 0; d < KW; ++d) where[d] = rel == (uint32_t)d ? kWindow + i : where[d];
        }
      }
#pragma unroll
      for (int i = 0; i < kWindow; ++i) {
        const uint32_t rel = win_a.k[i] - c0;
        if (win_a.k[i] == kEmptyKey) empty_a |= 1u << i;
#pragma unroll
        for (int d = 0; d < KW; ++d) where[d] = rel == (uint32_t)d ? i : where[d];
      }
#pragma unroll
      for (int d = 0; d < KW; ++d) {
        const int u = KW * a + (KW - 1 - d);
        if (!(want & (1u << u))) continue;
        const bool beyond = r + d > 15;
        const bool loaded = beyond ? load_b : load_a;
        if (!loaded) {  // window would leave the table: slot by slot from the home slot
          slot[u] = hashCell(cell[u]) & mask;
          pending |= 1u << u;
        } else if (where[d] >= 0) {
          hit |= 1u << u;
          slot[u] = (where[d] >= kWindow ? sb : sa) + (uint32_t)(where[d] & (kWindow - 1));
        } else if (((beyond ? empty_b : empty_a) >> (beyond ? r + d - 16 : d)) == 0) {
          slot[u] = ((beyond ? sb : sa) + (uint32_t)kWindow) & mask;
          pending |= 1u << u;
        }
      }
    }
    while (__any(pending != 0)) {
      uint32_t key[N];
#pragma unroll
      for (int u = 0; u < N; ++u) {
        key[u] = kEmptyKey;
        if (pending & (1u << u)) key[u] = keys[slot[u]];
      }
#pragma unroll
      for (int u = 0; u < N; ++u) {
        if (pending & (1u << u)) {
          if (key[u] == cell[u]) {
            hit |= 1u << u;
            pending &= ~(1u << u);
          } else if (key[u] == kEmptyKey) {
            pending &= ~(1u << u);
          } else {
            slot[u] = (slot[u] + 1) & mask;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < N; ++u) {
      if (hit & (1u << u)) res[u] = vals[slot[u]];
    }
    stagePairs<true, N>(res, KW * t0, KW * t_hi, j, staging, &staged);
  }
}

// ---- regular mode: ranks of marked cells -----------------------------------

// Exclusive prefix sum over `n` ints per row of `data` (one block of 1024
// threads per row, four consecutive elements per thread and pass), the row
// total goes to totals[row].
constexpr int kScanBlock = 1024;
constexpr int kScanItems = 4;
__global__ __launch_bounds__(kScanBlock) void rbScanRows(int32_t *data, int n, int32_t *totals) {
  constexpr int WAVES = kScanBlock / kWave;
  __shared__ int s_wsum[WAVES];
  __shared__ int s_total;
  int32_t *row = data + (size_t)blockIdx.x * n;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  int carry = 0;
  for (int base = 0; base < n; base += kScanBlock * kScanItems) {
    const int i0 = base + threadIdx.x * kScanItems;
    int v[kScanItems];
    int mine = 0;
#pragma unroll
    for (int e = 0; e < kScanItems; ++e) {
      v[e] = i0 + e < n ? row[i0 + e] : 0;
      mine += v[e];
    }
    const int incl = waveInclusiveScan(mine);
    if (lane == kWave - 1) s_wsum[wave] = incl;
    __syncthreads();
    if (wave == 0) {
      const int w = lane < WAVES ? s_wsum[lane] : 0;
      const int wi = waveInclusiveScan(w);
      if (lane < WAVES) s_wsum[lane] = wi - w;
      if (lane == kWave - 1) s_total = wi;
    }
    __syncthreads();
    int run = carry + s_wsum[wave] + incl - mine;
#pragma unroll
    for (int e = 0; e < kScanItems; ++e) {
      if (i0 + e < n) row[i0 + e] = run;
      run += v[e];
    }
    carry += s_total;
    __syncthreads();
  }
  if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

// Marked cells per block of kWordsPerBlock bitmap words, one word a thread.
__global__ __launch_bounds__(kBlock) void rbBitmapBlockSum(const unsigned long long *bitmap,
                                                           size_t n_words, int32_t *block_sum) {
  __shared__ int s_wsum[kBlock / kWave];
  const size_t w = (size_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
  int cnt = w < n_words ? __popcll(bitmap[w]) : 0;
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) s_wsum[threadIdx.x >> 6] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
    for (int x = 0; x < kBlock / kWave; ++x) t += s_wsum[x];
    block_sum[blockIdx.x] = t;
  }
}

// Per bitmap word: number of marked cells before it (word_rank).  Every marked
// cell is decoded to (n, d, h, w) and written at its rank.  A thread owns one word; where
// a wavefront's 64 words hold many cells (a small dense grid) the wavefront decodes them
// word by word, a lane per cell, instead of each lane walking its own word's bits.  Rows
// of out_indices from the number of marked cells on are left as the caller passed them,
// as the reference's decode kernel leaves them (normal_get_indice_pairs.cpp:1143-1150).
// block_count holds the marked cells of every block of kWordsPerBlock words: either as
// counted, then each workgroup sums the counts in front of its block itself and the last
// one writes the total to num_act_out, or, for bitmaps of more blocks than that is worth,
// already scanned (`scanned`, total already in num_act_out).
__global__ __launch_bounds__(kBlock) void rbRankAndDecode(GeomDev g,
                                                          const unsigned long long *bitmap,
                                                          size_t n_words,
                                                          const int32_t *block_count,
                                                          bool scanned, int32_t *num_act_out,
                                                          int32_t *host_num_act_out,
                                                          uint32_t *word_rank,
                                                          int32_t *out_indices, bool aligned,
                                                          int out_rows) {
  __shared__ int s_wsum[kBlock / kWave];
  static_assert(kWordsPerBlock == kBlock, "one bitmap word per thread");
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  __shared__ int s_front[kBlock / kWave];
  int front = 0;  // marked cells in the blocks before this one
  if (scanned) {
    front = block_count[blockIdx.x];
  } else {
    int part = 0;
    for (int i = threadIdx.x; i < (int)blockIdx.x; i += kBlock) part += block_count[i];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
    if (lane == 0) s_front[wave] = part;
  }
  const size_t w = (size_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
  const int hw = g.out[1] * g.out[2];
  const int vol = g.out[0] * hw;
  const unsigned long long bits = w < n_words ? bitmap[w] : 0ull;
  const int mine = __popcll(bits);
  const int incl = waveInclusiveScan(mine);
  if (lane == kWave - 1) s_wsum[wave] = incl;
  __syncthreads();
  if (!scanned) {
#pragma unroll
    for (int x = 0; x < kBlock / kWave; ++x) front += s_front[x];
  }
  int rank = front + incl - mine;
#pragma unroll
  for (int x = 0; x < kBlock / kWave; ++x)
    if (x < wave) rank += s_wsum[x];
  // the count of output cells, for the device and (pinned memory) for the host
  if (!scanned && blockIdx.x == gridDim.x - 1 && threadIdx.x == kBlock - 1) {
    *num_act_out = rank + mine;
    __hip_atomic_store(host_num_act_out, rank + mine, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
  if (scanned && blockIdx.x == 0 && threadIdx.x == 0)
    __hip_atomic_store(host_num_act_out, *num_act_out, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  if (w < n_words) word_rank[w] = (uint32_t)rank;
  auto put = [&](size_t cell64, int r) {
    if (r >= out_rows) return;
    int cell = (int)cell64;
    int4 o;
    o.x = fastDiv(cell, g.by_out_volume);
    cell -= o.x * vol;
    o.y = fastDiv(cell, g.by_out_plane);
    cell -= o.y * hw;
    o.z = fastDiv(cell, g.by_out_width);
    o.w = cell - o.z * g.out[2];
    storeCoord(out_indices, r, o, aligned);
  };
  const int wave_cells = __shfl(incl, kWave - 1, kWave);
  if (wave_cells > 4 * kWave) {
    unsigned long long todo = __ballot(bits != 0ull);
    const size_t w_first = w - lane;
    while (todo) {
      const int src = __ffsll((long long)todo) - 1;
      todo &= todo - 1;
      const unsigned long long b = __shfl(bits, src, kWave);
      const int r0 = __shfl(rank, src, kWave);
      if ((b >> lane) & 1ull) put((w_first + src) * 64 + lane, r0 + __popcll(b & ((1ull << lane) - 1ull)));
    }
  } else {
    unsigned long long b = bits;
    while (b) {
      const int bit = __ffsll((long long)b) - 1;
      b &= b - 1;
      put(w * 64 + bit, rank++);
    }
  }
}

// Moves the staged pairs of kPlaceWaves waves of one offset (workgroup (x, k)) to their
// final positions: the pairs in front of the chunk are the sum of the earlier waves'
// counts (a few kilobytes, read by every workgroup of the offset rather than scanned in a
// launch of its own), wave 0 scans the chunk's own counts, and the threads then take the
// chunk's pairs in their final order, up to eight each with the loads in flight together.
// In regular mode the staged output cell becomes the output row, its rank among the
// marked cells.  One thread files the rulebook's report.
constexpr int kPlaceWaves = 64;
constexpr int kPlaceBlock = 512;
constexpr int kPlacePer = 8;  // pairs a thread moves per pass, their loads in flight together
constexpr int kPlaceMaxChunks = 8;
// chunks of kPlaceWaves waves one workgroup moves in turn: one while the grid stays within a few
// rounds of workgroups per CU
static int placeChunksPerGroup(int n_wave, int K) {
  const long chunks = (n_wave + kPlaceWaves - 1) / kPlaceWaves;
  int m = 1;
  while (m < kPlaceMaxChunks && chunks * K / m > 8192) m *= 2;
  return m;
}
// A thread takes the t-th staged pair of the chunk, whichever wave of rows staged it (most
// waves stage a handful of pairs per offset, so a lane per (wave, slot) would idle): the wave is
// the last one whose pairs start at or before t.
__device__ __forceinline__ int placeSegment(const int *s_first, int t) {
  int seg = 0;
#pragma unroll
  for (int step = kPlaceWaves / 2; step > 0; step >>= 1)
    if (s_first[seg + step] <= t) seg += step;
  return seg;
}
template <bool SUBM>
__global__ __launch_bounds__(kPlaceBlock) void rbPlacePairs(int L, Staging st,
                                                             const unsigned long long *bitmap,
                                                             const uint32_t *word_rank, int32_t *pairs,
                                                             int32_t *indice_num,
                                                             const int32_t *rows_in_order,
                                                             const unsigned long long *unordered,
                                                             bool mirror_geometry, int chunks_per_group,
                                                             RulebookReportTarget report) {
  static_assert(kPlaceWaves == kWave, "one lane per wave count in the scan");
  constexpr int kWaves = kPlaceBlock / kWave;
  __shared__ int s_first[kPlaceWaves];  // staged pairs in front of each wave of the chunk
  __shared__ int s_start[kPlaceWaves];  // where the wave's pairs start in its staging block
  __shared__ int s_total;
  __shared__ int s_wave_sum[kWaves];
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    // submanifold: the rows were in cell order unless the word holds the call's stamp
    fileReport(SUBM ? *unordered != report.stamp : *rows_in_order != 0, report);
  }
  const int k = blockIdx.y;
  const int w_first = blockIdx.x * chunks_per_group * kPlaceWaves;
  const int w_end = min(w_first + chunks_per_group * kPlaceWaves, st.n_wave);
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  // Submanifold rows in cell order with a centred kernel: the probe resolved the offsets
  // below the centre only; offset K - 1 - k gets k's pairs with the columns exchanged and
  // the centre pairs every row with itself.
  const bool mirror = SUBM && mirror_geometry && *unordered != report.stamp;
  int32_t *mirror_in = nullptr, *mirror_out = nullptr;
  if (mirror) {
    const int K = gridDim.y;
    if (k > K / 2) return;
    if (k == K / 2) {
      int32_t *in_col = pairs + (size_t)k * 2 * L;
      const int hi = w_end * kWave < L ? w_end * kWave : L;
      for (int r = w_first * kWave + tid; r < hi; r += kPlaceBlock) {
        in_col[r] = r;
        in_col[L + r] = r;
      }
      if (blockIdx.x == 0 && tid == 0) indice_num[k] = L;
      return;
    }
    mirror_in = pairs + (size_t)(K - 1 - k) * 2 * L;
    mirror_out = mirror_in + L;
  }
  const int slice = k / (mirror ? st.mirror_k_per_slice : st.k_per_slice);
  const int32_t *counts = st.counts + (size_t)k * st.n_wave;
  // (wave 0's share of the first chunk's counts, requested together with the sum's loads)
  int entry = wave == 0 && w_first + lane < st.n_wave ? counts[w_first + lane] : 0;
  // pairs of the waves in front of the group's chunks
  int part = 0;
  for (int i0 = tid; i0 < w_first; i0 += kPlaceBlock * 8) {
    int c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = i0 + j * kPlaceBlock;
      c[j] = i < w_first ? counts[i] : 0;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) part += c[j] & 0xff;
  }
  part = waveInclusiveScan(part);
  if (lane == kWave - 1) s_wave_sum[wave] = part;
  __syncthreads();
  int before = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) before += s_wave_sum[w];
  int32_t *in_col = pairs + (size_t)k * 2 * L;
  int32_t *out_col = in_col + L;
  for (int w0 = w_first; w0 < w_end; w0 += kPlaceWaves) {
    if (w0 != w_first) __syncthreads();  // the chunk before has been moved
    if (wave == 0) {
      if (w0 != w_first) entry = w0 + lane < st.n_wave ? counts[w0 + lane] : 0;
      const int mine = entry & 0xff;
      const int incl = waveInclusiveScan(mine);
      s_start[lane] = entry >> 8;
      s_first[lane] = incl - mine;
      if (lane == kWave - 1) s_total = incl;
    }
    __syncthreads();
    const int total = s_total;
    for (int t0 = tid; t0 < total; t0 += kPlaceBlock * kPlacePer) {
      int v[kPlacePer], from_lane[kPlacePer], first_row[kPlacePer];
#pragma unroll
      for (int i = 0; i < kPlacePer; ++i) {
        const int t = t0 + i * kPlaceBlock;
        v[i] = from_lane[i] = first_row[i] = 0;
        if (t < total) {
          const int seg = placeSegment(s_first, t);
          const size_t at = stageBlock(st, slice, w0 + seg) + (size_t)(s_start[seg] + t - s_first[seg]);
          first_row[i] = (w0 + seg) * kWave;
          v[i] = st.stage[at];
          if (!SUBM) from_lane[i] = (int)st.stage_lane[at];
        }
      }
      int out[kPlacePer];
      if (!SUBM) {
        unsigned long long word[kPlacePer];
        uint32_t rank[kPlacePer];
#pragma unroll
        for (int i = 0; i < kPlacePer; ++i) {
          const bool live = t0 + i * kPlaceBlock < total;
          word[i] = live ? bitmap[v[i] >> 6] : 0ull;
          rank[i] = live ? word_rank[v[i] >> 6] : 0u;
        }
#pragma unroll
        for (int i = 0; i < kPlacePer; ++i)
          out[i] = (int)(rank[i] + (uint32_t)__popcll(word[i] & ((1ull << (v[i] & 63)) - 1ull)));
      }
#pragma unroll
      for (int i = 0; i < kPlacePer; ++i) {
        const int t = t0 + i * kPlaceBlock;
        if (t < total) {
          const int to = before + t;
          const int row = first_row[i] + (SUBM ? (v[i] & 63) : from_lane[i]);
          const int partner = SUBM ? v[i] >> 6 : out[i];
          in_col[to] = row;
          out_col[to] = partner;
          if (mirror) {
            mirror_in[to] = partner;
            mirror_out[to] = row;
          }
        }
      }
    }
    before += total;
  }
  if (blockIdx.x == gridDim.x - 1 && tid == 0) {
    indice_num[k] = before;
    if (mirror) indice_num[gridDim.y - 1 - k] = before;
  }
}

// ---- host side ---------------------------------------------------------------

inline size_t alignUp(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// Load factor between 1/16 and 1/8.  Home slots keep runs of cells together, so
// occupied stretches grow with the load and a probe sequence that leaves the
// first window costs the whole wave another memory round trip; 8 L measured
// best against 4 L (longer sequences) and 16 L (more lines to clear and fetch).
inline uint32_t tableCapacity(int L) {
  uint32_t cap = 64;
  while (cap < 8u * (uint32_t)L) cap <<= 1;
  return cap;
}


struct Workspace {
  // submanifold
  uint32_t *keys = nullptr;  // keys[table_cap] immediately followed by vals[table_cap]
  int32_t *vals = nullptr;
  uint32_t table_cap = 0;
  // regular
  unsigned long long *bitmap = nullptr;
  uint32_t *word_rank = nullptr;
  int32_t *block_sum = nullptr;
  int32_t *num_act_out = nullptr;
  size_t n_words = 0;
  size_t bitmap_fill_words = 0;  // 32-bit words to clear, rounded up to a multiple of 4
  int n_bitmap_blocks = 0;
  // both
  int32_t *stage = nullptr;          // [K, L] staged pairs (see Staging)
  uint8_t *stage_lane = nullptr;     // [K, L], regular mode only
  int32_t *counts = nullptr;         // [K, n_wave]
  int n_wave = 0;
  int32_t *rows_in_order = nullptr;  // regular: 1 until a kernel finds two rows out of cell order
  // submanifold: the sorted-cell arrays and the word that says they cannot be used
  uint32_t *cells = nullptr;
  uint32_t *samples = nullptr;
  unsigned long long *unordered = nullptr;
  int cells_capacity = 0;
  int sample_shift = 0;
  int n_samples_pad = 0;
  size_t bytes = 0;
};

Workspace carve(const RulebookGeom &g, void *base) {
  Workspace ws;
  // Blocks are carved from the caller's pointer rounded up to 256 bytes; the
  // reported size includes that slack.
  char *p = base ? reinterpret_cast<char *>(alignUp(reinterpret_cast<uintptr_t>(base))) : nullptr;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *r = p ? p + off : nullptr;
    off += alignUp(bytes);
    return r;
  };
  ws.n_wave = (g.L + kWave - 1) / kWave;
  if (g.sub_m) {
    ws.table_cap = tableCapacity(g.L);
    ws.keys = reinterpret_cast<uint32_t *>(take((size_t)ws.table_cap * 8));
    ws.vals = ws.keys ? reinterpret_cast<int32_t *>(ws.keys + ws.table_cap) : nullptr;
    // one sample every 2^shift rows, at most kMaxSamples of them
    while (((g.L + (1 << ws.sample_shift) - 1) >> ws.sample_shift) > kMaxSamples) ++ws.sample_shift;
    const int n_real = (g.L + (1 << ws.sample_shift) - 1) >> ws.sample_shift;
    ws.n_samples_pad = 64;
    while (ws.n_samples_pad < n_real) ws.n_samples_pad <<= 1;
    // a wave's span starts at (n_real << shift) + 1 at most and is read kSpan + kSpanPad cells far
    ws.cells_capacity = ((n_real << ws.sample_shift) + kSpan + kSpanPad + 4 + 3) / 4 * 4;
    ws.cells = reinterpret_cast<uint32_t *>(take((size_t)ws.cells_capacity * 4));
    ws.samples = reinterpret_cast<uint32_t *>(take((size_t)ws.n_samples_pad * 4));
    ws.unordered = reinterpret_cast<unsigned long long *>(take(8));
  } else {
    const size_t cells = (size_t)g.batch * g.out_space[0] * g.out_space[1] * g.out_space[2];
    ws.n_words = (cells + 63) / 64;
    ws.n_bitmap_blocks = (int)((ws.n_words + kWordsPerBlock - 1) / kWordsPerBlock);
    ws.bitmap_fill_words = (ws.n_words * 2 + 3) / 4 * 4;
    ws.bitmap = reinterpret_cast<unsigned long long *>(take(ws.bitmap_fill_words * 4));
    ws.word_rank = reinterpret_cast<uint32_t *>(take(ws.n_words * 4));
    ws.block_sum = reinterpret_cast<int32_t *>(take((size_t)ws.n_bitmap_blocks * 4));
    ws.num_act_out = reinterpret_cast<int32_t *>(take(4));

  }
  // one block of 64 slots per (offset, wave); slices of the offsets round the offsets up
  const size_t stage_slots = (size_t)(g.K + 32) * ws.n_wave * kWave;
  ws.stage = reinterpret_cast<int32_t *>(take(stage_slots * 4));
  if (!g.sub_m) ws.stage_lane = reinterpret_cast<uint8_t *>(take(stage_slots));
  ws.counts = reinterpret_cast<int32_t *>(take((size_t)g.K * ws.n_wave * 4));
  ws.rows_in_order = reinterpret_cast<int32_t *>(take(4));
  ws.bytes = off + 256;
  return ws;
}

GeomDev toDev(const RulebookGeom &g) {
  GeomDev d;
  d.batch = g.batch;
  for (int a = 0; a < 3; ++a) {
    d.out[a] = g.out_space[a];
    d.ks[a] = g.ksize[a];
    d.pad[a] = g.pad[a];
    d.stride[a] = g.stride[a];
    d.dil[a] = g.dilation[a];
    d.by_stride[a] = makeFastDiv(g.stride[a]);
  }
  d.by_out_volume = makeFastDiv(g.out_space[0] * g.out_space[1] * g.out_space[2]);
  d.by_out_plane = makeFastDiv(g.out_space[1] * g.out_space[2]);
  d.by_out_width = makeFastDiv(g.out_space[2]);
  d.K = g.K;
  d.L = g.L;
  return d;
}

inline bool aligned16(const void *a, const void *b) {
  return (((uintptr_t)a | (uintptr_t)b) & 15u) == 0;
}

inline int fillBlocks(size_t n) {
  size_t b = (n + kBlock - 1) / kBlock;
  return (int)(b < 1 ? 1 : (b > 4096 ? 4096 : b));
}

// Offsets per blockIdx.y slice of the probe and emit kernels: one group of
// kGroup where the kernel volume allows, at most 16 slices.
int offsetsPerSlice(int K) {
  int slices = (K + kGroup - 1) / kGroup;
  if (slices > 16) slices = 16;
  if (slices < 1) slices = 1;
  return (K + slices - 1) / slices;
}

}  // namespace

size_t rulebookWorkspaceBytes(const RulebookGeom &g) { return carve(g, nullptr).bytes; }

hipError_t launchSubmRulebook(const LaunchCtx &lc, const RulebookGeom &g, const int32_t *indices,
                              void *workspace, int32_t *indice_pairs, int32_t *out_indices,
                              int32_t *indice_num, const RulebookReportTarget &report) {
  const Workspace ws = carve(g, workspace);
  const GeomDev d = toDev(g);
  const bool al = aligned16(indices, out_indices);
  const uint32_t mask = ws.table_cap - 1;
  const int l_blocks = (g.L + kBlock - 1) / kBlock;
  const bool unit_stride = g.stride[0] == 1 && g.stride[1] == 1 && g.stride[2] == 1 &&
                           g.ksize[0] <= 32 && g.ksize[1] <= 32 && g.ksize[2] <= 32 &&
                           g.K <= kMaxInlineOffsets;
  bool mirror = unit_stride;
  for (int a = 0; a < 3; ++a)
    if (g.ksize[a] % 2 == 0 || 2 * g.pad[a] != g.dilation[a] * (g.ksize[a] - 1)) mirror = false;
  SortedCells sc = {ws.cells, ws.samples, ws.unordered, report.stamp,
                    ws.cells_capacity, ws.sample_shift, ws.n_samples_pad, mirror, 0};

  // cells become kEmptyKey and rows -1 with the same all-ones pattern
  FillRanges fill = {};
  fill.dst[0] = ws.keys;
  fill.n[0] = (size_t)ws.table_cap * 2;
  fill.value[0] = kEmptyKey;
  int rows = g.L > g.out_rows ? g.L : g.out_rows;
  if (ws.cells_capacity > rows) rows = ws.cells_capacity;
  lc.begin("rbSubmPrepare");
  rbSubmPrepare<<<(rows + kBlock - 1) / kBlock, kBlock, 0, lc.stream>>>(
      d, indices, al, out_indices, g.out_rows, fill, sc, !unit_stride);
  lc.end();
  lc.begin("rbSubmInsert");
  rbSubmInsert<<<l_blocks, kBlock, 0, lc.stream>>>(d, indices, al, ws.keys, ws.vals, mask, sc, indice_pairs);
  lc.end();
  const int k_per = offsetsPerSlice(g.K);
  Staging staging = {ws.stage, nullptr, ws.counts, ws.n_wave, k_per, k_per * kWave, 0};
  // groups of `width` offsets below the centre, spread over `slices` slices
  auto mirrorSlices = [&](int width, int slices) {
    const int groups = (g.K / 2 + width - 1) / width;
    sc.mirror_groups_per_slice = (groups + slices - 1) / slices;
    staging.mirror_k_per_slice = sc.mirror_groups_per_slice * width;
  };
  const dim3 slice_grid(l_blocks, (g.K + k_per - 1) / k_per);
  if (unit_stride) {
    UnitStrideOffsets ut;
    int k = 0;
    for (int kd = 0; kd < g.ksize[0]; ++kd)
      for (int kh = 0; kh < g.ksize[1]; ++kh)
        for (int kw = 0; kw < g.ksize[2]; ++kw, ++k) {
          ut.packed[k] = (uint32_t)kd | ((uint32_t)kh << 8) | ((uint32_t)kw << 16);
          ut.delta[k] = ((uint32_t)(kd * g.dilation[0]) * (uint32_t)g.out_space[1] +
                         (uint32_t)(kh * g.dilation[1])) * (uint32_t)g.out_space[2] +
                        (uint32_t)(kw * g.dilation[2]);
        }
    for (; k < kMaxInlineOffsets; ++k) ut.packed[k] = ut.delta[k] = 0;
    if ((g.ksize[2] == 3 || g.ksize[2] == 5) && g.dilation[2] == 1) {
      // one pass of kGroupsPerPass (kd, kh) pairs per wave while that leaves enough waves
      const int n_groups = g.K / g.ksize[2];
      const int t_per = n_groups > 4 * kGroupsPerPass ? 2 * kGroupsPerPass : kGroupsPerPass;
      const dim3 grid(l_blocks, (n_groups + t_per - 1) / t_per);
      staging.k_per_slice = t_per * g.ksize[2];
      staging.block_ints = staging.k_per_slice * kWave;
      mirrorSlices(g.ksize[2], (int)grid.y);
      lc.begin("rbSubmProbeRuns");
      if (g.ksize[2] == 3)
        rbSubmProbeRuns<3><<<grid, kBlock, 0, lc.stream>>>(d, ut, indices, al, ws.keys, ws.vals, mask,
                                                           staging, t_per, sc, indice_pairs);
      else
        rbSubmProbeRuns<5><<<grid, kBlock, 0, lc.stream>>>(d, ut, indices, al, ws.keys, ws.vals, mask,
                                                           staging, t_per, sc, indice_pairs);
      lc.end();
    } else {
      mirrorSlices(1, (int)slice_grid.y);
      lc.begin("rbSubmProbeUnitStride");
      rbSubmProbeUnitStride<<<slice_grid, kBlock, 0, lc.stream>>>(d, ut, indices, al, ws.keys, ws.vals,
                                                                  mask, staging, k_per, sc, indice_pairs);
      lc.end();
    }
  } else {
    lc.begin("rbProbeCount");
    rbProbeCount<true><<<slice_grid, kBlock, 0, lc.stream>>>(d, indices, al, ws.keys, ws.vals,
                                                             mask, nullptr, staging, k_per,
                                                             nullptr, nullptr);
    lc.end();
  }
  lc.begin("rbPlacePairs");
  const int per_group = placeChunksPerGroup(ws.n_wave, g.K);
  const int place_groups = (ws.n_wave + kPlaceWaves * per_group - 1) / (kPlaceWaves * per_group);
  rbPlacePairs<true><<<dim3(place_groups, g.K), kPlaceBlock, 0, lc.stream>>>(
      g.L, staging, nullptr, nullptr, indice_pairs, indice_num, nullptr, ws.unordered, mirror, per_group, report);
  lc.end();
  return hipGetLastError();
}

hipError_t launchRegularRulebook(const LaunchCtx &lc, const RulebookGeom &g,
                                 const int32_t *indices, void *workspace, int32_t *indice_pairs,
                                 int32_t *out_indices, int32_t *indice_num,
                                 int32_t *host_num_act_out, hipEvent_t count_ready,
                                 const RulebookReportTarget &report) {
  const Workspace ws = carve(g, workspace);
  const GeomDev d = toDev(g);
  const bool al_in = aligned16(indices, indices);
  const bool al_out = aligned16(out_indices, out_indices);
  const int l_blocks = (g.L + kBlock - 1) / kBlock;

  // bitmap 0
  FillRanges fill = {};
  fill.dst[0] = reinterpret_cast<uint32_t *>(ws.bitmap);
  fill.n[0] = ws.bitmap_fill_words;
  fill.value[0] = 0u;
  lc.begin("rbFill");
  rbFill<<<fillBlocks((ws.bitmap_fill_words + fill.n[1]) / 4 + 1), kBlock, 0, lc.stream>>>(
      fill, ws.rows_in_order);
  lc.end();
  const int k_per = offsetsPerSlice(g.K);
  Staging staging = {ws.stage, ws.stage_lane, ws.counts, ws.n_wave, k_per, k_per * kWave, 0};
  const dim3 slice_grid(l_blocks, (g.K + k_per - 1) / k_per);
  // most kernel positions of one axis that can have an output cell for one input coordinate:
  // those that share a remainder of position * dilation modulo the stride
  auto candidates = [&](int a) {
    int most = 0;
    for (int r = 0; r < g.stride[a]; ++r) {
      int n = 0;
      for (int t = 0; t < g.ksize[a]; ++t) n += (t * g.dilation[a]) % g.stride[a] == r ? 1 : 0;
      most = n > most ? n : most;
    }
    return most;
  };
  const bool strided = g.stride[0] > 1 || g.stride[1] > 1 || g.stride[2] > 1;
  const bool cube3 = g.ksize[0] == 3 && g.ksize[1] == 3 && g.ksize[2] == 3;
  const bool cube2 = g.ksize[0] == 2 && g.ksize[1] == 2 && g.ksize[2] == 2;
  if (strided && (cube3 || cube2)) {
    // slices of whole (kd, kh) groups of offsets
    const int per = cube3 ? 9 : 4;
    staging.k_per_slice = per;
    staging.block_ints = per * kWave;
    const dim3 grid(l_blocks, (g.K + per - 1) / per);
    lc.begin("rbProbeStrided");
    if (cube3)
      rbProbeStrided<3, 3, 3><<<grid, kBlock, 0, lc.stream>>>(d, indices, al_in, ws.bitmap, staging, per,
                                                              candidates(0), candidates(1),
                                                              ws.rows_in_order, indice_pairs);
    else
      rbProbeStrided<2, 2, 2><<<grid, kBlock, 0, lc.stream>>>(d, indices, al_in, ws.bitmap, staging, per,
                                                              candidates(0), candidates(1),
                                                              ws.rows_in_order, indice_pairs);
    lc.end();
  } else {
    lc.begin("rbProbeCount");
    rbProbeCount<false><<<slice_grid, kBlock, 0, lc.stream>>>(d, indices, al_in, nullptr,
                                                              nullptr, 0, ws.bitmap, staging, k_per,
                                                              ws.rows_in_order, indice_pairs);
    lc.end();
  }
  lc.begin("rbBitmapBlockSum");
  rbBitmapBlockSum<<<ws.n_bitmap_blocks, kBlock, 0, lc.stream>>>(ws.bitmap, ws.n_words, ws.block_sum);
  lc.end();
  const bool scanned = ws.n_bitmap_blocks > kSelfScanBlocks;
  if (scanned) {
    lc.begin("rbScanRows");
    rbScanRows<<<1, kScanBlock, 0, lc.stream>>>(ws.block_sum, ws.n_bitmap_blocks, ws.num_act_out);
    lc.end();
  }
  lc.begin("rbRankAndDecode");
  rbRankAndDecode<<<ws.n_bitmap_blocks, kBlock, 0, lc.stream>>>(d, ws.bitmap, ws.n_words, ws.block_sum,
                                                             scanned, ws.num_act_out, host_num_act_out,
                                                             ws.word_rank, out_indices, al_out, g.out_rows);
  lc.end();
  hipError_t err = hipEventRecord(count_ready, lc.stream);
  if (err != hipSuccess) return err;
  lc.begin("rbPlacePairs");
  const int per_group = placeChunksPerGroup(ws.n_wave, g.K);
  const int place_groups = (ws.n_wave + kPlaceWaves * per_group - 1) / (kPlaceWaves * per_group);
  rbPlacePairs<false><<<dim3(place_groups, g.K), kPlaceBlock, 0, lc.stream>>>(
      g.L, staging, ws.bitmap, ws.word_rank, indice_pairs, indice_num, ws.rows_in_order, nullptr, false, per_group,
      report);
  lc.end();
  return hipGetLastError();
}

}  // namespace sparse_conv
}  // namespace mluop
