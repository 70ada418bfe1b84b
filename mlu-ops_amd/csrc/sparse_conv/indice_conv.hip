// Indice convolution kernels for gfx950: forward, backward data, backward filter.
//
// Semantics (reference test/mlu_op_gtest/pb_gtest/src/zoo/
// indice_convolution_forward/indice_convolution_forward.cpp:86-176,
// indice_convolution_backward_data/indice_convolution_backward_data.cpp:254-343,
// indice_convolution_backward_filter/indice_convolution_backward_filter.cpp:121-178):
//   forward   out[o, :]  = sum_k sum_{(i,o) in pairs[k]} feat[i, :] . W[k]
//   bwd data  dX[i, :]   = sum_k sum_{(i,o) in pairs[k]} dY[o, :] . W[k]^T
//   bwd filt  dW[k]      = sum_{(i,o) in pairs[k]} X[i, :]^T . dY[o, :]
// with fp32 accumulation and one rounding to the tensor type at the end.
//
// Forward and backward data are the same "gather convolution": every result row
// is owned by exactly one workgroup, which walks the K offsets in order and adds
// the contribution of the (at most one) gathered row per offset.  No atomics,
// no inter-workgroup reduction, so results are reproducible run to run.  The
// owner of a row finds its gathered rows through a dense row map
// map[k][row] -> gathered row or -1, rebuilt from indice_pairs on every call.
//
// Two implementations of the gather convolution:
//  * gatherConvMfma  fp16/bf16, channel counts that tile into 16x16x32 MFMA
//    blocks.  A workgroup owns up to 256 result rows; per offset the rows that
//    have a partner are compacted with wave ballots into blocks of 16, so MFMA
//    work follows the number of pairs, not K x rows.  Each wave owns a column
//    slice of the fp32 accumulator tile in LDS.
//  * gatherConvSimt  any type and channel count (fp32 always), LDS-tiled FMA.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "core/wave_scan.h"
#include "sparse_conv/indice_conv.h"

namespace mluop {
namespace sparse_conv {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned short u16;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// A workgroup barrier for LDS traffic only: what the wave wrote to or read from LDS is done,
// loads from global memory stay in flight across it (__syncthreads() would wait for them).
__device__ __forceinline__ void ldsBarrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 16 bytes per lane from global memory straight into LDS: lane l of the wave writes bytes
// [16 l, 16 l + 16) behind `lds_address` (the same in all lanes).  Written as the instruction
// itself: the compiler then does not know of an LDS write in flight, and does not hold every
// later LDS read of the wave back until all loads have returned; the caller waits (vmcnt)
// before anybody reads what was requested.
__device__ __forceinline__ void requestToLds(const void *global, uint32_t lds_address) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :: "s"(lds_address), "v"(global) : "memory", "m0");
}
constexpr int kMaxInlineK = 128;

// Pair counts per offset, passed by value for the common small kernel volumes.
struct OffsetCounts {
  int n[kMaxInlineK];
};

__device__ __forceinline__ int offsetCount(const OffsetCounts &inl, const int32_t *dev, int k) {
  return dev != nullptr ? dev[k] : inl.n[k];
}

// ---- element types ---------------------------------------------------------

// MFMA traits: an operand fragment is 16 bytes per lane (vec8: kVec elements),
// kChunk reduction channels per fragment.
struct HalfElem {
  typedef _Float16 storage;
  typedef half8 vec8;
  static constexpr int kVec = 8, kChunk = 32;
  static __device__ __forceinline__ float load(const storage *p) { return (float)*p; }
  static __device__ __forceinline__ void store(storage *p, float v) { *p = (_Float16)v; }
  static __device__ __forceinline__ float4v mfma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct BFloat16Elem {
  typedef u16 storage;
  typedef bf16x8 vec8;
  static constexpr int kVec = 8, kChunk = 32;
  static __device__ __forceinline__ float load(const storage *p) {
    return __uint_as_float((uint32_t)*p << 16);
  }
  static __device__ __forceinline__ void store(storage *p, float v) {
    uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) {  // NaN stays NaN
      *p = (u16)((u >> 16) | 0x40u);
      return;
    }
    u += 0x7fffu + ((u >> 16) & 1u);  // round to nearest even
    *p = (u16)(u >> 16);
  }
  static __device__ __forceinline__ float4v mfma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

struct FloatElem {
  typedef float storage;
  typedef float4v vec8;  // four floats: lane (m, kq) holds reduction channels 4*kq + (0..3) of a 16-chunk
  static constexpr int kVec = 4, kChunk = 16;
  static __device__ __forceinline__ float load(const storage *p) { return *p; }
  static __device__ __forceinline__ void store(storage *p, float v) { *p = v; }
  // Four 16x16x4 steps; step s pairs element s of both fragments, i.e. channel
  // 4*kq + s in MFMA reduction slot kq: a permutation of the chunk's 16 channels.
  static __device__ __forceinline__ float4v mfma(vec8 a, vec8 b, float4v c) {
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[3], b[3], c, 0, 0, 0);
    return c;
  }
};

// ---- row map ---------------------------------------------------------------

// A launch that is enqueued before anyone knows whether it is needed: it runs when `word` is
// null or holds `value`, and returns at once otherwise.  The row-map kernels of a forward
// call that started on the pair lists without knowing whether they are in order carry the
// verdict word and the call's ticket here.
struct RunIf {
  const unsigned long long *word;
  unsigned long long value;
};
__device__ __forceinline__ bool notWanted(const RunIf &r) { return r.word != nullptr && *r.word != r.value; }

__global__ __launch_bounds__(256) void fillInt32(int32_t *dst, size_t n, int32_t value) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) dst[i] = value;
}

// map[k][row - row_base] = partner row, for the first indice_num[k] pairs of every offset
// whose row lies in [row_base, row_base + n_rows): the map of one chunk of result rows.
// row_col / src_col select which pair column owns the result row (1 for
// forward, 0 for backward data).  Pairs that name a row outside their tensors are ignored.
// Every workgroup leaves the number of pairs it put into the map in accepted[its index]
// (unless accepted is null).
// A map slot holds one partner.  Rulebooks built from distinct coordinates name a
// result row once per offset at most; when coordinates repeat (or the pairs are
// made up, as in test case files) several pairs of one offset can name the same
// row, and the reference adds them all.  Plain stores keep whichever of them was
// written last; every workgroup of a gather kernel records how many slots of its
// tile it found filled, and repairLostPairs adds what the other pairs would have
// contributed when those counts fall short of the number of accepted pairs.
__global__ __launch_bounds__(256) void scatterRowMap(const int32_t *pairs, int L,
                                                     OffsetCounts inl, const int32_t *dev_counts,
                                                     int row_col, int src_col, int row_base,
                                                     int n_rows, int n_src, int32_t *map,
                                                     int32_t *accepted, RunIf run_if) {
  if (notWanted(run_if)) return;
  const int k = blockIdx.y;
  const int n = offsetCount(inl, dev_counts, k);
  const int32_t *base = pairs + (size_t)k * 2 * L;
  int mine = 0;
  for (int p = blockIdx.x * 256 + threadIdx.x; p < n; p += gridDim.x * 256) {
    const int r = base[(size_t)row_col * L + p] - row_base;
    const int s = base[(size_t)src_col * L + p];
    if ((unsigned)r < (unsigned)n_rows && (unsigned)s < (unsigned)n_src) {
      map[(size_t)k * n_rows + r] = s;
      ++mine;
    }
  }
  __shared__ int s_accepted;
  if (threadIdx.x == 0) s_accepted = 0;
  __syncthreads();
  mine = waveInclusiveScan(mine);
  if ((threadIdx.x & 63) == 63 && mine != 0) atomicAdd(&s_accepted, mine);
  __syncthreads();
  if (threadIdx.x == 0 && accepted != nullptr) accepted[blockIdx.y * gridDim.x + blockIdx.x] = s_accepted;
}

// The same on a flat grid: an offset gets the workgroups its pairs need and no
// more.  The (pairs, offset) grid above is sized by the fullest offset; at 125
// offsets of which one holds a quarter of all pairs, nine in ten of its workgroups
// exit at once and their dispatch is what the kernel costs.
struct OffsetBlocks {
  int first[kMaxInlineK];  // workgroups in front of the offset's first one
};

__global__ __launch_bounds__(256) void scatterRowMapFlat(const int32_t *pairs, int L,
                                                         OffsetCounts inl, OffsetBlocks blocks,
                                                         int K, int row_col, int src_col,
                                                         int row_base, int n_rows, int n_src,
                                                         int32_t *map, int32_t *accepted, RunIf run_if) {
  if (notWanted(run_if)) return;
  // last offset whose first workgroup is not behind this one (an offset without
  // pairs shares its prefix with the next one and is never chosen)
  int lo = 0, hi = K - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (blocks.first[mid] <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const int k = lo;
  const int p = ((int)blockIdx.x - blocks.first[k]) * 256 + threadIdx.x;
  bool ok = false;
  if (p < inl.n[k]) {
    const int32_t *base = pairs + (size_t)k * 2 * L;
    const int r = base[(size_t)row_col * L + p] - row_base;
    const int s = base[(size_t)src_col * L + p];
    ok = (unsigned)r < (unsigned)n_rows && (unsigned)s < (unsigned)n_src;
    if (ok) map[(size_t)k * n_rows + r] = s;
  }
  const int total = __syncthreads_count(ok);
  if (threadIdx.x == 0 && accepted != nullptr) accepted[blockIdx.x] = total;
}

// ---- SIMT gather convolution -------------------------------------------------
// result[r, c] = sum_k sum_q A[map[k][r], q] * B(k, q, c),
// B(k, q, c) = W[k*sK + q*sQ + c*sC].  32 x 64 result tile per block.
template <typename E>
__global__ __launch_bounds__(256) void gatherConvSimt(const typename E::storage *A, int Q,
                                                      const typename E::storage *W, int64_t sK,
                                                      int64_t sQ, int64_t sC, const int32_t *map,
                                                      int R, int K, OffsetCounts inl,
                                                      const int32_t *dev_counts, int C,
                                                      int32_t *filled,
                                                      typename E::storage *result) {
  constexpr int TR = 32, TC = 64, QC = 32;
  int slots = 0;  // filled map slots of this tile (first wave, uniform)
  __shared__ float As[TR][QC + 1];
  __shared__ float Bs[QC][TC];
  __shared__ int s_src[TR];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int r0 = blockIdx.x * TR, c0 = blockIdx.y * TC;
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int k = 0; k < K; ++k) {
    if (offsetCount(inl, dev_counts, k) <= 0) continue;
    int v = -1;
    if (tid < TR && r0 + tid < R) v = map[(size_t)k * R + r0 + tid];
    if (tid < TR) s_src[tid] = v;
    if (tid < 64) slots += __popcll(__ballot(v >= 0));
    if (!__syncthreads_or(v >= 0)) continue;
    for (int q0 = 0; q0 < Q; q0 += QC) {
#pragma unroll
      for (int i = 0; i < TR * QC / 256; ++i) {
        const int e = tid + i * 256;
        const int r = e / QC, q = e % QC;
        const int src = s_src[r];
        As[r][q] = (src >= 0 && q0 + q < Q) ? E::load(A + (size_t)src * Q + q0 + q) : 0.f;
      }
#pragma unroll
      for (int i = 0; i < QC * TC / 256; ++i) {
        const int e = tid + i * 256;
        const int q = e / TC, c = e % TC;
        Bs[q][c] = (q0 + q < Q && c0 + c < C)
                       ? E::load(W + (size_t)k * sK + (size_t)(q0 + q) * sQ + (size_t)(c0 + c) * sC)
                       : 0.f;
      }
      __syncthreads();
#pragma unroll 8
      for (int q = 0; q < QC; ++q) {
        const float a0 = As[ty * 2][q], a1 = As[ty * 2 + 1][q];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float b = Bs[q][tx * 4 + j];
          acc[0][j] += a0 * b;
          acc[1][j] += a1 * b;
        }
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = r0 + ty * 2 + i;
    if (r >= R) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = c0 + tx * 4 + j;
      if (c < C) E::store(result + (size_t)r * C + c, acc[i][j]);
    }
  }
  if (tid == 0 && blockIdx.y == 0) filled[blockIdx.x] = slots;
}

// ---- MFMA gather convolution ---------------------------------------------------

// Filter repacked into MFMA operand fragments of 16 bytes per lane (VEC elements,
// CHUNK reduction channels per fragment; 8 and 32 for the 2-byte types, 4 and 16
// for float):
// packed[(((k*(C/16) + nb)*(Q/CHUNK) + kb)*64 + lane)*VEC + e]
//   = B(k, q = kb*CHUNK + VEC*(lane/16) + e, c = nb*16 + lane%16), zero for q >= Q
// (16 reduction channels of a 2-byte type fill half a fragment).
// One launch for the two independent preparations of the MFMA path: blocks
// below fill_blocks set the row map to -1 (16-byte stores), the others repack
// the filter.
template <typename E>
__global__ __launch_bounds__(256) void fillMapPackFilter(int32_t *map, size_t map_elems,
                                                         int fill_blocks,
                                                         const typename E::storage *W, int64_t sK,
                                                         int64_t sQ, int64_t sC, int K, int Q,
                                                         int C, typename E::storage *packed,
                                                         RunIf run_if) {
  if (notWanted(run_if)) return;
  if ((int)blockIdx.x < fill_blocks) {
    const size_t quads = map_elems / 4;
    int4 *dst = reinterpret_cast<int4 *>(map);
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < quads;
         i += (size_t)fill_blocks * 256)
      dst[i] = make_int4(-1, -1, -1, -1);
    if (blockIdx.x == 0 && threadIdx.x < (map_elems & 3)) map[quads * 4 + threadIdx.x] = -1;
    return;
  }
  const int pack_blocks = gridDim.x - fill_blocks;
  constexpr int VEC = E::kVec, CHUNK = E::kChunk;
  const int chunks = (Q + CHUNK - 1) / CHUNK;  // Q below one fragment is padded with zeros
  const size_t total = (size_t)K * (C / 16) * chunks * 64;
  for (size_t t = (size_t)(blockIdx.x - fill_blocks) * 256 + threadIdx.x; t < total;
       t += (size_t)pack_blocks * 256) {
    const int lane = (int)(t & 63);
    size_t rest = t >> 6;
    const int kb = (int)(rest % chunks);
    rest /= chunks;
    const int nb = (int)(rest % (C / 16));
    const int k = (int)(rest / (C / 16));
    const int c = nb * 16 + (lane & 15);
    const int qb = kb * CHUNK + VEC * (lane >> 4);
#pragma unroll
    for (int e = 0; e < VEC; ++e)
      packed[t * VEC + e] =
          qb + e < Q ? W[(size_t)k * sK + (size_t)(qb + e) * sQ + (size_t)c * sC] : typename E::storage(0);
  }
}

// ---- where a gather kernel finds the pairs of its tile -------------------------------
//
// Either a dense row map (above), or the pair lists themselves, cut by tile.  The
// second needs the column of the pairs that names the result rows to ascend strictly
// inside every offset, which is how mluOpGetIndicePairs lists them: its input-row
// column always does (backward data), its output-row column does when the input rows
// are ordered by cell (forward).  The pairs of one offset that fall into a tile of
// result rows are then one contiguous piece of the list, and a [K, tiles + 1] table
// of cut positions replaces the [K, rows] map: nothing to clear, no slot a second pair
// could lose, a few kilobytes instead of K * rows * 4 bytes.
struct MapSource {
  static constexpr bool kSegments = false;
  const int32_t *map;
  int32_t *filled;
  RunIf run_if;
};

struct SegmentSource {
  static constexpr bool kSegments = true;
  const int32_t *pairs;               // [K, 2, L]
  const int32_t *cuts;                // [K, cut_stride]: first pair of every tile, then the count
  const unsigned long long *verdict;  // holds `ticket` when some list is not in order
  unsigned long long ticket;
  // Lists out of order: true = the kernel returns at once (row-map kernels enqueued behind
  // it do the call's work), false = every tile collects its pairs by reading all of them.
  bool leave_if_unordered;
  int L, row_col, src_col, n_src, cut_stride;
  const void *W;                      // the filter as the caller passed it, for lists out of order
  int64_t sK, sQ, sC;
  OffsetCounts counts;
};

// The pairs of one tile of result rows [r_begin, r_end) when the lists cannot be cut:
// every workgroup reads all pairs of all offsets, and each pair that names one of its
// rows is multiplied by one wave, a lane per result column, and added to the tile's
// fp32 rows in LDS (`acc`, cleared by the caller).  Offsets are taken in order with a
// barrier between them, so a row sees its offsets in the order the list kernels use;
// only rows that several pairs of one offset name depend on timing in their last
// bits.  It is slow and runs only when a pair tensor was changed
// after the library had seen it in order.
template <typename E, int NT>
__device__ __forceinline__ void scanAllPairsForTile(const typename E::storage *A, int Q,
                                                    const SegmentSource &src, int K, int r_begin,
                                                    int r_end, int C, int col0, float *acc,
                                                    int acc_stride) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const typename E::storage *W = static_cast<const typename E::storage *>(src.W);
  for (int k = 0; k < K; ++k) {
    const int n = src.counts.n[k];
    const int32_t *row_list = src.pairs + ((size_t)k * 2 + src.row_col) * src.L;
    const int32_t *src_list = src.pairs + ((size_t)k * 2 + src.src_col) * src.L;
    for (int p0 = 0; p0 < n; p0 += NT) {
      const int p = p0 + tid;
      int r = -1, g = -1;
      if (p < n) {
        r = row_list[p];
        g = src_list[p];
      }
      const bool hit = r >= r_begin && r < r_end && (unsigned)g < (unsigned)src.n_src;
      unsigned long long m = __ballot(hit);
      while (m) {
        const int from = __ffsll((long long)m) - 1;
        m &= m - 1;
        const int rr = __shfl(r, from, kWave) - r_begin;
        const typename E::storage *a = A + (size_t)__shfl(g, from, kWave) * Q;
        for (int c = lane; c < C; c += kWave) {
          const typename E::storage *w = W + (size_t)k * src.sK + (size_t)(col0 + c) * src.sC;
          float dot = 0.f;
          for (int q = 0; q < Q; ++q) dot += E::load(a + q) * E::load(w + (size_t)q * src.sQ);
          atomicAdd(&acc[rr * acc_stride + c], dot);
        }
      }
    }
    __syncthreads();
  }
}

// One launch in front of a gather kernel that reads pair lists: the first
// `pack_blocks` workgroups repack the filter into operand fragments (as
// fillMapPackFilter does), the others walk the pair lists, one pair per lane, and
//  * check what the gather kernel relies on: result rows in range and strictly
//    ascending inside the offset, gathered rows in range.  A violation stores `ticket`
//    in *verdict (a value no earlier call used, so the word needs no clearing);
//  * write the cut table: pair p is the first pair of every tile after its
//    predecessor's tile up to its own, and the last pair of an offset closes the
//    remaining tiles with the pair count (an offset without pairs gets one workgroup
//    that closes all its tiles with 0).  A lane with more than a few tiles to close
//    hands them to the whole wave.
constexpr int kCutPairsPerThread = 4;

template <typename E>
__global__ __launch_bounds__(256) void packFilterCutPairLists(
    const typename E::storage *W, int64_t sK, int64_t sQ, int64_t sC, int K, int Q, int C,
    typename E::storage *packed, int pack_blocks, const int32_t *pairs, int L, OffsetCounts inl,
    OffsetBlocks blocks, int row_col, int src_col, int R, int n_src, int tile_shift, int n_tiles,
    int32_t *cuts, unsigned long long *verdict, unsigned long long ticket) {
  if ((int)blockIdx.x < pack_blocks) {
    constexpr int VEC = E::kVec, CHUNK = E::kChunk;
    const int chunks = (Q + CHUNK - 1) / CHUNK;
    const size_t total = (size_t)K * (C / 16) * chunks * 64;
    for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < total;
         t += (size_t)pack_blocks * 256) {
      const int lane = (int)(t & 63);
      size_t rest = t >> 6;
      const int kb = (int)(rest % chunks);
      rest /= chunks;
      const int nb = (int)(rest % (C / 16));
      const int k = (int)(rest / (C / 16));
      const int c = nb * 16 + (lane & 15);
      const int qb = kb * CHUNK + VEC * (lane >> 4);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        packed[t * VEC + e] =
            qb + e < Q ? W[(size_t)k * sK + (size_t)(qb + e) * sQ + (size_t)c * sC] : typename E::storage(0);
    }
    return;
  }
  const int b = (int)blockIdx.x - pack_blocks;
  int lo = 0, hi = K - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (blocks.first[mid] <= b) lo = mid; else hi = mid - 1;
  }
  const int k = lo;
  const int n = inl.n[k];
  const int lane = threadIdx.x & 63;
  const int32_t *row_list = pairs + ((size_t)k * 2 + row_col) * L;
  const int32_t *src_list = pairs + ((size_t)k * 2 + src_col) * L;
  int32_t *row_cuts = cuts + (size_t)k * (n_tiles + 1);
  // kCutPairsPerThread pairs a thread, 256 apart: all their loads are requested first
  const int p0 = (b - blocks.first[k]) * (256 * kCutPairsPerThread) + (int)threadIdx.x;
  int rs[kCutPairsPerThread], prevs[kCutPairsPerThread], ss[kCutPairsPerThread];
#pragma unroll
  for (int j = 0; j < kCutPairsPerThread; ++j) {
    const int p = p0 + j * 256;
    rs[j] = 0;
    prevs[j] = -1;
    ss[j] = 0;
    if (p < n) {
      rs[j] = row_list[p];
      ss[j] = src_list[p];
      if (p > 0) prevs[j] = row_list[p - 1];
    }
  }
#pragma unroll
  for (int j = 0; j < kCutPairsPerThread; ++j) {
    const int p = p0 + j * 256;
    const bool live = p < n;
    const int r = rs[j], prev = prevs[j], s = ss[j];
    const bool ok = (unsigned)r < (unsigned)R && (unsigned)s < (unsigned)n_src && r > prev;
    if (live && !ok) *verdict = ticket;
    // tiles (t_lo .. t_mid] open at p, tiles (t_mid .. n_tiles] close with n; clamped so
    // that a list out of order, whose table nobody reads, still writes inside the table
    int t_mid = r >> tile_shift;
    t_mid = t_mid < 0 ? 0 : (t_mid > n_tiles - 1 ? n_tiles - 1 : t_mid);
    int t_lo = p == 0 ? -1 : (prev >> tile_shift);
    t_lo = t_lo < -1 ? -1 : (t_lo > t_mid ? t_mid : t_lo);
    // job 0: value p over (t_lo, t_mid]; job 1 (last pair only): value n over (t_mid, n_tiles]
#pragma unroll
    for (int job = 0; job < 2; ++job) {
      // (an offset without pairs has one workgroup, whose first lane closes all tiles with 0)
      const bool empty_offset = n == 0 && threadIdx.x == 0 && j == 0;
      const int first = empty_offset ? 0 : (job == 0 ? t_lo + 1 : t_mid + 1);
      const int last = job == 0 ? t_mid : n_tiles;
      const int value = job == 0 ? p : n;
      const bool mine = ((live && (job == 0 || p == n - 1)) || (empty_offset && job == 1)) && first <= last;
      const bool wide = mine && last - first >= 4;
      if (mine && !wide)
        for (int t = first; t <= last; ++t) row_cuts[t] = value;
      unsigned long long m = __ballot(wide);
      while (m) {
        const int from = __ffsll((long long)m) - 1;
        m &= m - 1;
        const int f = __shfl(first, from, kWave), l = __shfl(last, from, kWave);
        const int v = __shfl(value, from, kWave);
        for (int t = f + lane; t <= l; t += kWave) row_cuts[t] = v;
      }
    }
  }
}

constexpr int mfmaTileRows(int C) {
  // fp32 accumulator tile of about 34 KiB
  return C <= 64 ? 128 : 64;
}
constexpr int mfmaColBlocksPerWave(int C) { return C >= 128 ? 2 : 1; }
// as many fetching waves as multiplying waves (five-wave workgroups place badly on the CU)
constexpr int mfmaThreads(int C) { return 128 * (C / 16 / mfmaColBlocksPerWave(C)); }
// Register budget: two eight-wave workgroups per CU need four waves per SIMD
// (128 registers a lane); the fp32 128x128 instance holds 128 registers of
// filter fragments alone and stays at one workgroup per CU.
constexpr int mfmaWavesPerSimd(int elem_bytes, int Q, int C) {
  return (elem_bytes == 4 && Q == 128 && C == 128) ? 2 : (C >= 64 ? 4 : (C == 32 ? 3 : 2));
}
constexpr int kOffsetChunk = 28;  // offsets whose pair lists are resident in LDS at once
// Gathered rows staged in LDS per round: about 25 KiB, which one wave can hold
// in registers while they travel (at most 24 16-byte pieces per lane).
constexpr int mfmaStageRows(int row_bytes) {
  return row_bytes <= 64 ? 256 : (row_bytes <= 128 ? 192 : (row_bytes <= 256 ? 96 : 48));
}
// 16-pair blocks multiplied together; bounded by the registers the W fragments of two batches
// take (16 bytes per lane for every 16-byte piece of a row and every 16 result columns).
constexpr int mfmaBatchBlocks(int elem_bytes, int Q, int C) {
  const int regs_per_block = ((Q * elem_bytes + 63) / 64) * mfmaColBlocksPerWave(C) * 4;
  const int g = 32 / regs_per_block;
  return g < 1 ? 1 : (g > 4 ? 4 : g);
}

// Workgroup = TR result rows x C columns (column group blockIdx.y of the ldc
// result columns), WAVES multiplying waves and as many fetching waves.
// Multiplying wave w owns columns [w*16*NB, (w+1)*16*NB) of the
// fp32 accumulator tile in LDS, so no two waves ever touch the same accumulator
// element and every element sees its contributions in ascending offset order.
//
// Per chunk of kOffsetChunk offsets:
//   A   wave w (of all waves) loads map[k][row] for the offsets k = w (mod all
//       waves) of the chunk and all rows of the tile, ballots which rows have a
//       partner and, after the per-offset counts have been exchanged, compacts
//       one entry per pair (partner row << 8 | result row) into a flat list
//       ordered by offset.  The list is cut into blocks of up to 16 entries of
//       one offset, and the block list is padded to a whole batch.
//   B   the flat list is walked in rounds of STEP entries.  The partner rows of
//       a round are fetched by the fetching waves alone, with row-contiguous
//       16-byte loads (fetching them in the MFMA operand's own lane order
//       touches 16 rows per load and runs at a third of the L1 rate, once per
//       column wave), and written to the LDS stage between two barriers when
//       the multiplying waves have finished the round before.  Waves of their
//       own keep these loads out of the multiplying waves' in-order load
//       counter, where waiting for the next W fragments would also wait for
//       them.  Every multiplying wave reads its operand fragments from the
//       staged rows, multiplies W[k]^T (16 result columns x Q, fetched one
//       batch ahead) by the block's rows (Q x 16 pairs), which leaves four
//       consecutive result columns of one pair in every lane, and adds them to
//       the accumulator row of that pair with one 16-byte read-modify-write.
//       Lanes past the end of a short block repeat its first entry and
//       accumulate into a spare row.
template <typename E, int Q, int C, typename SRC>
__global__ __launch_bounds__(mfmaThreads(C)) __attribute__((amdgpu_waves_per_eu(mfmaWavesPerSimd((int)sizeof(typename E::storage), Q, C),
                                   mfmaWavesPerSimd((int)sizeof(typename E::storage), Q, C))))
void gatherConvMfma(const typename E::storage *A, const typename E::storage *packedW,
                    SRC source, int R, int K, int ldc, typename E::storage *result) {
  typedef typename E::vec8 vec8;
  typedef typename E::storage S;
  constexpr int NB = mfmaColBlocksPerWave(C);
  constexpr int WAVES = C / 16 / NB;            // multiplying waves
  constexpr int NT = mfmaThreads(C);
  constexpr int TR = mfmaTileRows(C);
  constexpr int NSEG = TR / 64;
  constexpr int KB = (Q + E::kChunk - 1) / E::kChunk;  // operand fragments per row
  constexpr bool kPartialFragment = Q < E::kChunk;     // 16 channels of a 2-byte type: upper lanes are zero
  constexpr int KC = kOffsetChunk;
  constexpr int ALLW = NT / 64;                 // multiplying + fetching waves
  constexpr int FW = ALLW - WAVES;              // fetching waves
  constexpr int KPW = (KC + ALLW - 1) / ALLW;   // offsets a wave scans per chunk
  constexpr int G = mfmaBatchBlocks((int)sizeof(S), Q, C);
  constexpr int GROUPS = C / 16;
  constexpr int MAX_ENT = KC * TR;
  constexpr int MAX_BLK = KC * (TR / 16) + G;
  constexpr int ACC_STRIDE = C + 4;             // floats; rows 16 apart fall into distinct banks
  constexpr int ROW_BYTES = Q * (int)sizeof(S);  // one gathered row
  constexpr int STAGE_STRIDE = ROW_BYTES + 16;  // padded: 16 rows x 16 bytes hit 64 distinct banks
  constexpr int PPR = ROW_BYTES / 16;           // 16-byte pieces per row
  constexpr int SROWS = mfmaStageRows(ROW_BYTES);
  constexpr int STEP = SROWS - G * 16;          // a batch starting inside a round ends inside its stage
  constexpr int PT = SROWS * PPR / (64 * FW);   // pieces per lane of a fetching wave
  static_assert(SROWS * PPR % (64 * FW) == 0 && PT <= 24, "stage must split evenly over the fetching waves");
  static_assert(KC <= 64 && MAX_ENT <= 65536 && TR <= 256, "descriptor packing");

  __shared__ __attribute__((aligned(16))) float s_acc[(TR + 1) * ACC_STRIDE];
  __shared__ __attribute__((aligned(16))) char s_stage[SROWS * STAGE_STRIDE];
  __shared__ uint32_t s_ent[MAX_ENT];   // partner row << 8 | result row in the tile
  __shared__ uint32_t s_blk[MAX_BLK];   // offset in chunk << 24 | first entry << 8 | entries
  __shared__ int s_cnt[KC];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool fetcher = wave >= WAVES;
  const int ftid = tid - 64 * WAVES;            // thread index among the fetching waves
  // Workgroups go to the eight XCDs round robin; giving XCD x the x-th eighth of the
  // tiles keeps neighbouring tiles, which gather many of the same rows, on one L2.
  const int tiles_per_xcd = gridDim.x >> 3;
  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  const int r0 = tile * TR;
  if constexpr (!SRC::kSegments) {
    if (notWanted(source.run_if)) return;
  }
  if (r0 >= R) {
    if constexpr (!SRC::kSegments) {
      if (tid == 0 && blockIdx.y == 0) source.filled[blockIdx.x] = 0;
    }
    return;
  }
  int slots = 0;  // filled map slots of this tile
  const unsigned long long lt_mask = (1ull << lane) - 1ull;

  for (int i = tid; i < (TR + 1) * ACC_STRIDE; i += NT) s_acc[i] = 0.f;

  // Pair lists that turned out not to be in order (a caller who changed the tensor
  // behind the library's back): the tile collects its pairs by reading all of them.
  bool in_order = true;
  if constexpr (SRC::kSegments) {
    in_order = *source.verdict != source.ticket;
    if (!in_order && source.leave_if_unordered) return;
    if (!in_order) {
      __syncthreads();
      scanAllPairsForTile<E, NT>(A, Q, source, K, r0, r0 + TR < R ? r0 + TR : R, C, blockIdx.y * C,
                                 s_acc, ACC_STRIDE);
    }
  }

  // per-lane constants of the multiply phase
  const char *a_bytes = reinterpret_cast<const char *>(A);
  // the workgroup owns result columns [blockIdx.y*C, (blockIdx.y+1)*C) of ldc
  const int col_group = blockIdx.y;
  const char *b_base = reinterpret_cast<const char *>(packedW) +
                       ((size_t)(col_group * GROUPS + wave * NB) * KB * 64 + lane) * 16;
  const uint32_t kBytesPerOffset = (uint32_t)(ldc / 16) * KB * 64 * 16;  // packed W[k]
  const int pair = lane & 15;
  const int quad = lane >> 4;
  char *acc_lane = reinterpret_cast<char *>(s_acc) + (wave * 16 * NB + 4 * quad) * 4;
  const char *stage_lane = s_stage + quad * 16;

  for (int kc = 0; kc < (in_order ? K : 0); kc += KC) {
    const int kn = (K - kc) < KC ? (K - kc) : KC;
    // A: the pairs of this wave's offsets; unconditional loads from clamped
    // addresses keep all of them in flight.
    int idx[KPW][NSEG];   // partner row, or -1
    int own[KPW][NSEG];   // result row inside the tile (pair lists only)
    if constexpr (SRC::kSegments) {
      // lane 2j + e fetches cut e of this wave's j-th offset
      int cut = 0;
      {
        const int kk = wave + (lane >> 1) * ALLW;
        if ((lane >> 1) < KPW && kk < kn)
          cut = source.cuts[(size_t)(kc + kk) * source.cut_stride + tile + (lane & 1)];
      }
      int first[KPW], count[KPW];
#pragma unroll
      for (int j = 0; j < KPW; ++j) {
        const int kk = wave + j * ALLW;
        first[j] = __shfl(cut, 2 * j, kWave);
        const int end = __shfl(cut, 2 * j + 1, kWave);
        int c = end - first[j];
        c = c < 0 ? 0 : (c > TR ? TR : c);
        count[j] = (kk < kn && source.counts.n[kk < kn ? kc + kk : kc] > 0) ? c : 0;
        const int k_safe = kk < kn ? kc + kk : kc;
        const int32_t *row_list = source.pairs + ((size_t)k_safe * 2 + source.row_col) * source.L;
        const int32_t *src_list = source.pairs + ((size_t)k_safe * 2 + source.src_col) * source.L;
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {
          int p = first[j] + seg * 64 + lane;
          p = p < 0 ? 0 : (p < source.L ? p : source.L - 1);
          own[j][seg] = row_list[p];
          idx[j][seg] = src_list[p];
        }
      }
#pragma unroll
      for (int j = 0; j < KPW; ++j)
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) asm volatile("" : "+v"(idx[j][seg]), "+v"(own[j][seg]));
#pragma unroll
      for (int j = 0; j < KPW; ++j) {
        const int kk = wave + j * ALLW;
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {
          if (seg * 64 + lane >= count[j]) idx[j][seg] = -1;
          own[j][seg] = (own[j][seg] - r0) & (TR - 1);
        }
        if (lane == 0 && kk < KC) s_cnt[kk] = count[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < KPW; ++j) {
        const int kk = wave + j * ALLW;
        const int k_safe = kk < kn ? kc + kk : kc;
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {
          const int r = r0 + seg * 64 + lane;
          idx[j][seg] = source.map[(size_t)k_safe * R + (r < R ? r : R - 1)];
          own[j][seg] = seg * 64 + lane;
        }
      }
      // Pinning the loaded values here keeps the loads above unconditional and all
      // in flight; selecting on them directly lets the compiler branch around
      // every single load and wait for it.
#pragma unroll
      for (int j = 0; j < KPW; ++j)
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) asm volatile("" : "+v"(idx[j][seg]));
#pragma unroll
      for (int j = 0; j < KPW; ++j) {
        const int kk = wave + j * ALLW;
        int c = 0;
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {
          const int r = r0 + seg * 64 + lane;
          if (!(kk < kn && r < R)) idx[j][seg] = -1;
          c += __popcll(__ballot(idx[j][seg] >= 0));
        }
        if (lane == 0 && kk < KC) s_cnt[kk] = c;
      }
    }
    __syncthreads();
    // every wave scans the counts: entries and blocks in front of each offset
    const int cnt = lane < KC ? s_cnt[lane < KC ? lane : 0] : 0;
    const int nb_mine = (cnt + 15) >> 4;
    const int ent_incl = waveInclusiveScan(cnt);
    const int blk_incl = waveInclusiveScan(nb_mine);
    const int total = __builtin_amdgcn_readlane(ent_incl, 63);
    const int nblk = __builtin_amdgcn_readlane(blk_incl, 63);
    slots += total;
    const int nbatch = (nblk + G - 1) / G;
    const int ent_first = ent_incl - cnt;
#pragma unroll
    for (int j = 0; j < KPW; ++j) {
      const int kk = wave + j * ALLW;
      int base = __shfl(ent_first, kk & 63, kWave);
#pragma unroll
      for (int seg = 0; seg < NSEG; ++seg) {
        const unsigned long long b = __ballot(idx[j][seg] >= 0);
        if (idx[j][seg] >= 0)
          s_ent[base + __popcll(b & lt_mask)] = ((uint32_t)idx[j][seg] << 8) | (uint32_t)own[j][seg];
        base += __popcll(b);
      }
    }
    // lane kk of the wave that scanned offset kk cuts its list into blocks
    if (lane < KC && (lane % ALLW) == wave) {
      const int first_blk = blk_incl - nb_mine;
      for (int b = 0; b < nb_mine; ++b) {
        const int left = cnt - 16 * b;
        s_blk[first_blk + b] = ((uint32_t)lane << 24) | ((uint32_t)(ent_first + 16 * b) << 8) |
                               (uint32_t)(left < 16 ? left : 16);
      }
    }
    if (wave == WAVES && nblk > 0) {
      // empty blocks that fill the last batch: offset and position of the last entry
      const int last_k = 63 - __builtin_clzll(__ballot(cnt > 0));
      if (lane < nbatch * G - nblk)
        s_blk[nblk + lane] = ((uint32_t)last_k << 24) | ((uint32_t)(total - 1) << 8);
    }
    __syncthreads();

    // B: the round a batch belongs to follows from the first entry of its first block
    const int last_round =
        nblk > 0 ? (int)((s_blk[(nbatch - 1) * G] >> 8) & 0xffffu) / STEP : 0;
    if (fetcher) {
      if (nblk > 0) {
        for (int round = 0; round <= last_round; ++round) {
          u32x4 piece[PT];
#pragma unroll
          for (int i = 0; i < PT; ++i) {
            const int p = ftid + i * 64 * FW;
            int ci = round * STEP + p / PPR;
            ci = ci < total ? ci : total - 1;
            const uint32_t src = s_ent[ci] >> 8;
            piece[i] = *reinterpret_cast<const u32x4 *>(a_bytes + (size_t)src * ROW_BYTES +
                                                        (p % PPR) * 16);
          }
          if (round > 0) __syncthreads();  // the multiplying waves have left the stage
#pragma unroll
          for (int i = 0; i < PT; ++i) {
            const int p = ftid + i * 64 * FW;
            *reinterpret_cast<u32x4 *>(&s_stage[(p / PPR) * STAGE_STRIDE + (p % PPR) * 16]) = piece[i];
          }
          __syncthreads();
        }
      }
    } else if (nblk > 0) {
      vec8 wnext[G][KB][NB];
      uint32_t dnext[G];
      int k_held[G];  // offset whose fragments slot g holds: a dense offset fills several
                      // batches in a row and its fragments are fetched once
#pragma unroll
      for (int g = 0; g < G; ++g) k_held[g] = -1;
      auto fetch_batch = [&](int b0) {
        const uint32_t dv = s_blk[b0 + (lane & (G - 1))];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          dnext[g] = (uint32_t)__builtin_amdgcn_readlane((int)dv, g);
          const int kk = (int)(dnext[g] >> 24);
          // (single-block batches only: with several slots the branch costs the other
          // instances more than the saved loads)
          if (G > 1 || kk != k_held[g]) {
            k_held[g] = kk;
            const char *bk = b_base + (size_t)(kc + kk) * kBytesPerOffset;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
              for (int nb = 0; nb < NB; ++nb)
                wnext[g][kb][nb] = *reinterpret_cast<const vec8 *>(bk + (nb * KB + kb) * 1024);
          }
        }
      };
      fetch_batch(0);
      __syncthreads();  // round 0 is staged
      int round = 0;
      for (int bt = 0; bt < nbatch; ++bt) {
        vec8 wcur[G][KB][NB];
        uint32_t dcur[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          dcur[g] = dnext[g];
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) wcur[g][kb][nb] = wnext[g][kb][nb];
        }
        if (bt + 1 < nbatch) fetch_batch((bt + 1) * G);
        // the stage moves on when the batch starts past the current round
        while ((int)((dcur[0] >> 8) & 0xffffu) >= (round + 1) * STEP) {
          __syncthreads();
          __syncthreads();
          ++round;
        }
        const int stage_first = round * STEP;
        vec8 afr[G][KB];
        int acc_row[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int first = (int)((dcur[g] >> 8) & 0xffffu);
          const int n = (int)(dcur[g] & 0xffu);
          const int e = first + (pair < n ? pair : 0);
          const uint32_t ent = s_ent[e];
          acc_row[g] = pair < n ? (int)(ent & 0xffu) : TR;
          const char *arow = stage_lane + (e - stage_first) * STAGE_STRIDE;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            afr[g][kb] = *reinterpret_cast<const vec8 *>(arow + kb * 64);
          if constexpr (kPartialFragment) {
            // the row ends after Q channels: the lanes of the upper quads would read the next
            // staged row; they multiply zero filter fragments, and zero keeps a NaN there out
            if (quad * E::kVec >= Q) afr[g][0] = vec8{};
          }
        }
        float4v prod[G][NB];
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            prod[g][nb] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
              prod[g][nb] = E::mfma(wcur[g][kb][nb], afr[g][kb], prod[g][nb]);
          }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          char *dst = acc_lane + acc_row[g] * (ACC_STRIDE * 4);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            // lane holds result columns 16*nb + 4*quad + (0..3) of its pair
            float4v old = *reinterpret_cast<float4v *>(dst + nb * 64);
            old += prod[g][nb];
            *reinterpret_cast<float4v *>(dst + nb * 64) = old;
          }
        }
      }
      // rounds the fetching wave staged beyond the last batch cannot exist:
      // last_round is the round of the last batch
    }
    __syncthreads();
  }
  constexpr int VALS = 16 / (int)sizeof(S);  // result values per 16-byte store
  for (int i = tid; i < TR * C / VALS; i += NT) {
    const int rr = i / (C / VALS);
    const int c0 = (i % (C / VALS)) * VALS;
    if (r0 + rr >= R) break;
    S tmp[VALS];
#pragma unroll
    for (int e = 0; e < VALS; ++e) E::store(&tmp[e], s_acc[rr * ACC_STRIDE + c0 + e]);
    *reinterpret_cast<uint4 *>(result + (size_t)(r0 + rr) * ldc + col_group * C + c0) =
        *reinterpret_cast<const uint4 *>(tmp);
  }
  if constexpr (!SRC::kSegments) {
    if (tid == 0 && blockIdx.y == 0) source.filled[blockIdx.x] = slots;
  }
}

// What a lane without a row of its own loads: a row of zeros in device memory.
__device__ __attribute__((aligned(256))) unsigned char kZeroRow[512];  // never written

// ---- MFMA gather convolution, one free-running wavefront per tile ---------------------
//
// The kernel above spends a tile's life waiting: cut positions, then pairs, then
// gathered rows round by round behind barriers, then a filter slice from L2 for every
// thinly filled offset, with two tiles a CU to overlap it all.  For results of up to 32
// columns a tile of 128 result rows fits a single wavefront that never meets a barrier:
// its fp32 accumulator tile and one 16-row stage slot are all the LDS it needs, so
// seven tiles share a CU, a layer of a few hundred thousand rows is resident at once,
// and what the wave waits for is hidden by its own requests running ahead in register
// rings:
//   unit      = up to 16 pairs of one offset, walked in offset order;
//   t + 10    the unit's pairs are requested (lane l: pair l % 16);
//   t + 5     its gathered rows (row-contiguous 16-byte pieces) and the offset's filter
//             fragments are requested;
//   t         rows go through the LDS slot (written row-major, read as MFMA operand
//             fragments), all column blocks are multiplied and the products added to the
//             pairs' fp32 rows, read from and written back to LDS 16 bytes a lane.
// Requests are unconditional (clamped addresses) so that the number of loads in flight
// at every point of the loop is fixed.  It reads pair lists only (SegmentSource).
// Measured against the kernel above on 120 000 rows with 2.2 pairs a row: 32 -> 32
// channels 26 us against 32 us; at 64 result columns (two waves a tile, 32 columns
// each) it loses, 43 us against 41 us, and is not used.
constexpr int kWaveTileRows = 128;
constexpr bool waveKernelShape(int elem_bytes, int Q, int C) {
  const int chunk = elem_bytes == 4 ? 16 : 32;
  return C <= 32 && Q * elem_bytes <= 256 && ((Q + chunk - 1) / chunk) * (C / 16) <= 8;
}
template <typename E, int Q, int C>
__global__ __launch_bounds__(64) void gatherConvWave(
    const typename E::storage *A, const typename E::storage *packedW, SegmentSource source, int R,
    int K, typename E::storage *result) {
  typedef typename E::vec8 vec8;
  typedef typename E::storage S;
  constexpr int NB = C / 16;                            // column blocks
  constexpr int KB = (Q + E::kChunk - 1) / E::kChunk;
  constexpr bool kPartialFragment = Q < E::kChunk;
  constexpr int TR = kWaveTileRows;
  constexpr int ACC_STRIDE = C + 4;
  constexpr int ROW_BYTES = Q * (int)sizeof(S);
  constexpr int STAGE_STRIDE = ROW_BYTES + 16;
  constexpr int PPR = ROW_BYTES / 16;                   // 16-byte pieces per row
  constexpr int RL = (16 * PPR + 63) / 64;              // wave-loads per unit of rows
  constexpr int EPL = 64 / PPR >= 16 ? 16 : 64 / PPR;   // rows per wave-load
  constexpr int NE = 12;   // pair ring (units) = units per trip of the unrolled loop
  constexpr int NR = 6;    // row and filter ring (units)
  constexpr int AHEAD_ROWS = 5;
  constexpr int AHEAD_PAIRS = 10;
  static_assert(PPR >= 2 && PPR <= 32 && AHEAD_ROWS < NR && AHEAD_PAIRS < NE && NE % NR == 0, "ring sizes");
  constexpr int ACC_QUADS = (TR + 1) * ACC_STRIDE / 4;

  __shared__ __attribute__((aligned(16))) float s_acc[(TR + 1) * ACC_STRIDE];
  __shared__ __attribute__((aligned(16))) char s_stage[16 * STAGE_STRIDE];

  const int lane = threadIdx.x;
  const int tiles_per_xcd = gridDim.x >> 3;  // neighbouring tiles on one XCD
  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  const int r0 = tile * TR;
  if (r0 >= R) return;

  // this tile's piece of every offset's list (lane l: offsets l and l + 64)
  const unsigned long long verdict = *source.verdict;
  int piece_first[2] = {0, 0}, piece_count[2] = {0, 0};
#pragma unroll
  for (int o = 0; o < 2; ++o) {
    const int k = lane + 64 * o;
    if (k < K) {
      const int32_t *c = source.cuts + (size_t)k * source.cut_stride + tile;
      piece_first[o] = c[0];
      piece_count[o] = c[1];
    }
  }
#pragma unroll 8
  for (int i = lane; i < ACC_QUADS; i += 64)
    reinterpret_cast<float4v *>(s_acc)[i] = float4v{0.f, 0.f, 0.f, 0.f};

  constexpr int VALS = 16 / (int)sizeof(S);
  auto write_out = [&]() {
    for (int i = lane; i < TR * C / VALS; i += 64) {
      const int rr = i / (C / VALS);
      const int c0 = (i % (C / VALS)) * VALS;
      if (r0 + rr >= R) break;
      S tmp[VALS];
#pragma unroll
      for (int e = 0; e < VALS; ++e) E::store(&tmp[e], s_acc[rr * ACC_STRIDE + c0 + e]);
      *reinterpret_cast<uint4 *>(result + (size_t)(r0 + rr) * C + c0) = *reinterpret_cast<const uint4 *>(tmp);
    }
  };
  if (verdict == source.ticket) {
    if (source.leave_if_unordered) return;
    // lists out of order: every pair of every offset is looked at
    scanAllPairsForTile<E, 64>(A, Q, source, K, r0, r0 + TR < R ? r0 + TR : R, C, 0, s_acc, ACC_STRIDE);
    write_out();
    return;
  }
  unsigned long long has[2];
#pragma unroll
  for (int o = 0; o < 2; ++o) {
    int c = piece_count[o] - piece_first[o];
    c = c < 0 ? 0 : (c > TR ? TR : c);
    if (lane + 64 * o >= K) c = 0;
    piece_count[o] = c;
    has[o] = __ballot(c > 0);
  }
  // first offset above `after` that has pairs in this tile, or 128
  auto next_offset = [&](int after) {
    const int from = after + 1;
    const unsigned long long lo = from < 64 ? (has[0] & (~0ull << from)) : 0ull;
    if (lo) return (int)__builtin_ctzll(lo);
    const unsigned long long hi = from <= 64 ? has[1] : (from < 128 ? (has[1] & (~0ull << (from - 64))) : 0ull);
    if (hi) return 64 + (int)__builtin_ctzll(hi);
    return 128;
  };
  auto of = [&](const int (&v)[2], int k) {
    const int a = __builtin_amdgcn_readlane(v[0], k & 63), b = __builtin_amdgcn_readlane(v[1], k & 63);
    return k < 64 ? a : b;
  };
  // the walk over units: offset, first pair and pair count of the unit a request is made for
  int walk_k = next_offset(-1);
  int walk_left = walk_k < 128 ? of(piece_count, walk_k) : 0;
  int walk_at = walk_k < 128 ? of(piece_first, walk_k) : 0;
  int unit_k[NE], unit_at[NE], unit_n[NE];
  auto next_unit = [&](int &k, int &at, int &n) {
    k = walk_k;
    at = walk_at;
    n = walk_left < 16 ? walk_left : 16;
    if (walk_k < 128) {
      walk_left -= n;
      walk_at += n;
      if (walk_left <= 0) {
        walk_k = next_offset(walk_k);
        walk_left = walk_k < 128 ? of(piece_count, walk_k) : 0;
        walk_at = walk_k < 128 ? of(piece_first, walk_k) : 0;
      }
    }
  };

  const char *a_bytes = reinterpret_cast<const char *>(A);
  const char *b_base = reinterpret_cast<const char *>(packedW) + (size_t)lane * 16;
  const uint32_t kBytesPerOffset = (uint32_t)(C / 16) * KB * 64 * 16;
  const int pair = lane & 15;
  const int quad = lane >> 4;
  char *acc_lane = reinterpret_cast<char *>(s_acc) + 4 * quad * 4;
  char *stage = s_stage;

  // Rows of up to 64 bytes are loaded by the lane that multiplies them, 16 bytes of its own
  // pair's row (the 16 rows of a unit are 16 cache lines either way); longer rows are
  // fetched row by row, half as many lines a load, and turned into fragments by the LDS slot.
  constexpr bool kDirectRows = ROW_BYTES <= 64;
  int pair_row[NE], pair_src[NE];
  u32x4 rows[NR][RL];
  vec8 w[NR][KB][NB];

  auto request_pairs = [&](int slot) {
    next_unit(unit_k[slot], unit_at[slot], unit_n[slot]);
    const int k = unit_k[slot] < K ? unit_k[slot] : 0;
    int p = unit_at[slot] + pair;
    p = p < 0 ? 0 : (p < source.L ? p : source.L - 1);
    const int32_t *list = source.pairs + (size_t)k * 2 * source.L;
    pair_row[slot] = list[(size_t)source.row_col * source.L + p];
    pair_src[slot] = list[(size_t)source.src_col * source.L + p];
    // The requests must stay where they are written, far ahead of their use: nothing that
    // may touch memory moves across this point, so the compiler cannot sink the loads
    // towards the instructions that consume them (and no register is named, so nothing
    // is waited for here).
    asm volatile("" ::: "memory");
  };
  auto request_rows = [&](int pslot, int rslot) {
    const int n = unit_n[pslot];
    const int k = unit_k[pslot] < K ? unit_k[pslot] : 0;
    if constexpr (kDirectRows) {
      static_assert(!kDirectRows || (RL == 1 && KB == 1), "one fragment a row");
      int g = pair_src[pslot];
      if (pair >= n || (unsigned)g >= (unsigned)source.n_src) g = 0;
      // (a lane beyond the row's channels reads the row of zeros)
      const char *from = quad * 16 < ROW_BYTES ? a_bytes + (size_t)g * ROW_BYTES + quad * 16
                                               : reinterpret_cast<const char *>(kZeroRow);
      rows[rslot][0] = *reinterpret_cast<const u32x4 *>(from);
    } else {
#pragma unroll
      for (int h = 0; h < RL; ++h) {
        const int e = lane / PPR + EPL * h;  // which pair's row this lane fetches a piece of
        int g = __shfl(pair_src[pslot], e & 15, kWave);
        if (e >= n || (unsigned)g >= (unsigned)source.n_src) g = 0;
        rows[rslot][h] = *reinterpret_cast<const u32x4 *>(a_bytes + (size_t)g * ROW_BYTES + (lane % PPR) * 16);
      }
    }
    const char *bk = b_base + (size_t)k * kBytesPerOffset;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        w[rslot][kb][nb] = *reinterpret_cast<const vec8 *>(bk + (nb * KB + kb) * 1024);
    asm volatile("" ::: "memory");
  };
  auto multiply = [&](int pslot, int rslot) {
    const int n = unit_n[pslot];
    const int acc_row = pair < n ? ((pair_row[pslot] - r0) & (TR - 1)) : TR;
    char *dst = acc_lane + acc_row * (ACC_STRIDE * 4);
    // (products summed from zero, then added: the arithmetic of the kernel above, so the
    // two give the same bits)
    float4v acc[NB], prod[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      acc[nb] = *reinterpret_cast<float4v *>(dst + nb * 64);
      prod[nb] = float4v{0.f, 0.f, 0.f, 0.f};
    }
    vec8 afr[KB];
    if constexpr (kDirectRows) {
      afr[0] = __builtin_bit_cast(vec8, rows[rslot][0]);
    } else {
#pragma unroll
      for (int h = 0; h < RL; ++h) {
        const int e = lane / PPR + EPL * h;
        if (16 * PPR >= 64 || lane < 16 * PPR)
          *reinterpret_cast<u32x4 *>(stage + e * STAGE_STRIDE + (lane % PPR) * 16) = rows[rslot][h];
      }
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
        afr[kb] = *reinterpret_cast<const vec8 *>(stage + pair * STAGE_STRIDE + kb * 64 + quad * 16);
      if constexpr (kPartialFragment) {
        if (quad * E::kVec >= Q) afr[0] = vec8{};
      }
    }
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) prod[nb] = E::mfma(w[rslot][kb][nb], afr[kb], prod[nb]);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      acc[nb] += prod[nb];
      *reinterpret_cast<float4v *>(dst + nb * 64) = acc[nb];
    }
  };

#pragma unroll
  for (int u = 0; u < AHEAD_PAIRS; ++u) request_pairs(u);
#pragma unroll
  for (int u = 0; u < AHEAD_ROWS; ++u) request_rows(u, u);
  bool more = unit_k[0] < 128;
  while (more) {
#pragma unroll
    for (int u = 0; u < NE; ++u) {
      // unit t = t0 + u: pair slot u, row slot u % NR
      if (more) {
        request_pairs((u + AHEAD_PAIRS) % NE);
        request_rows((u + AHEAD_ROWS) % NE, (u + AHEAD_ROWS) % NR);
        multiply(u, u % NR);
        more = unit_k[(u + 1) % NE] < 128;
      }
    }
  }
  write_out();
}

// ---- MFMA gather convolution for dense rulebooks -------------------------------
//
// When most rows of a tile have a partner at most offsets, compacting pairs buys
// little and the fp32 accumulate in LDS (a 16-byte read-modify-write per lane and
// 16 result columns, on arbitrary rows: bank conflicts) is what the kernel above
// spends its time on.  Here a tile is 128 result rows (256 below 128 channels), a wave
// of eight owns G = 1 (2) groups of 16 of them and all result columns, and accumulates
// them in registers over all offsets: no accumulator traffic at all.  The partner rows of an offset come from global memory straight into the
// operand registers of the lane that multiplies them (lane (row, quarter) loads 16
// bytes of its row per reduction chunk, one offset ahead), so no wave waits for
// another one's rows.  What the waves of a workgroup share is the offset's filter: its
// fragments travel from global memory into one of two LDS buffers (16 bytes per lane
// straight into LDS, one offset ahead, every wave a share of them) and every wave reads
// all of them from there, once per offset for all its row groups.  One barrier per
// offset hands the buffers over; it waits for LDS traffic only, and each wave waits for
// its own loads itself (__syncthreads() would make every wave wait for all loads in
// flight, the requests for the offset after included).  A lane whose row has no
// partner at the offset reads a row of zeros; a row group none of whose rows has one
// is skipped, and a wave without any skips the offset.
constexpr int kDenseChunk = 27;      // offsets whose row-map slice is resident in LDS at once
constexpr int kDenseMapBatch = 14;   // loads in flight per thread while a tile's row map is read
constexpr int kDenseWaves = 8;
// Row groups per wave: with two sets of partner rows a wave stays within 128 registers, four
// waves a SIMD.  (Four waves of twice the groups measured the same at 64 and 128 columns and
// 12 % slower at 16 and 32, where a wave has little to multiply between two barriers.)
constexpr int denseGroups(int Q, int C) { return (C >= 128 || Q >= 128) ? 1 : 2; }
constexpr int denseTileRows(int Q, int C) { return kDenseWaves * denseGroups(Q, C) * 16; }

template <typename E, int Q, int C, typename SRC>
__global__ __launch_bounds__(64 * kDenseWaves) __attribute__((amdgpu_waves_per_eu(4, 4))) void gatherConvDense(
    const typename E::storage *A, const typename E::storage *packedW, SRC source, int R,
    int K, int ldc, typename E::storage *result) {
  typedef typename E::vec8 vec8;
  typedef typename E::storage S;
  constexpr int WAVES = kDenseWaves;
  constexpr int G = denseGroups(Q, C);
  constexpr int TR = denseTileRows(Q, C);
  constexpr int NB = C / 16;                 // 16-column blocks, all of them in every wave
  constexpr int KC = kDenseChunk;
  constexpr int KB = (Q + E::kChunk - 1) / E::kChunk;
  // 16 channels of a 2-byte type: half a fragment, the lanes of the other half read zeros
  constexpr bool kHalfFragment = Q % E::kChunk != 0;
  constexpr int ROW_BYTES = Q * (int)sizeof(S);
  constexpr int FRAGS = NB * KB;             // 1 KiB filter fragments per offset
  constexpr int W_BYTES = FRAGS * 1024;
  constexpr int FPW = (FRAGS + WAVES - 1) / WAVES;
  // Offsets multiplied between two barriers: two where a filter is 4 KiB at most (a wave then
  // has little to multiply per offset, and the second set of rows fits the registers): 16 and
  // 32 column layers 7 % faster; at 64 x 64 the rows of two offsets spill.
  constexpr int OPP = W_BYTES <= 4096 ? 2 : 1;
  constexpr int POOL = 2 * OPP * W_BYTES;
  static_assert((Q % E::kChunk == 0 || (KB == 1 && Q % E::kVec == 0)) && C % 16 == 0,
                "whole fragments, or part of a single one");
  static_assert(G >= 1 && G <= 4, "one code path per set of row groups");

  __shared__ __attribute__((aligned(1024))) char s_w[POOL];
  __shared__ int s_map[KC][TR];   // partner row of (offset in chunk, tile row) or -1
  __shared__ int s_list[KC];      // offsets of the chunk that have a pair in this tile
  __shared__ int s_has[KC];
  __shared__ int s_first[KC];
  __shared__ int s_count;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tiles_per_xcd = gridDim.x >> 3;  // neighbouring tiles on one XCD, as above
  const int tile = (blockIdx.x & 7) * tiles_per_xcd + (blockIdx.x >> 3);
  const int r0 = tile * TR;
  if constexpr (!SRC::kSegments) {
    if (notWanted(source.run_if)) return;
  }
  if (r0 >= R) {
    if constexpr (!SRC::kSegments) {
      if (tid == 0 && blockIdx.y == 0) source.filled[blockIdx.x] = 0;
    }
    return;
  }
  const int col_group = blockIdx.y;
  if constexpr (SRC::kSegments) {
    if (*source.verdict == source.ticket && source.leave_if_unordered) return;
    if (*source.verdict == source.ticket) {
      // pair lists out of order: fp32 rows where the row map would be, 16 columns at a
      // time, every pair looked at by every workgroup
      float *acc = reinterpret_cast<float *>(&s_map[0][0]);
      constexpr int CP = 16;  // columns per pass
      static_assert(CP <= KC && C % CP == 0, "a pass of columns fits the row map");
      const int r_end = r0 + TR < R ? r0 + TR : R;
      for (int c0 = 0; c0 < C; c0 += CP) {
        for (int i = tid; i < TR * CP; i += WAVES * 64) acc[i] = 0.f;
        __syncthreads();
        scanAllPairsForTile<E, WAVES * 64>(A, Q, source, K, r0, r_end, CP, col_group * C + c0, acc, CP);
        for (int i = tid; i < TR * CP; i += WAVES * 64) {
          const int rr = i / CP, c = i % CP;
          if (r0 + rr < R) E::store(result + (size_t)(r0 + rr) * ldc + col_group * C + c0 + c, acc[i]);
        }
        __syncthreads();
      }
      return;
    }
  }
  const int pair = lane & 15;
  const int quad = lane >> 4;
  const char *a_lane = reinterpret_cast<const char *>(A) + quad * 16;
  const char *zero_lane = reinterpret_cast<const char *>(kZeroRow) + quad * 16;
  const char *w_base = reinterpret_cast<const char *>(packedW) +
                       (size_t)col_group * FRAGS * 1024 + lane * 16;
  const size_t kBytesPerOffset = (size_t)(ldc / 16) * KB * 1024;
  const uint32_t w_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)s_w;
  const int row_first = wave * (G * 16) + pair;  // this lane's row in its wave's first group

  float4v acc[G][NB];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[g][nb] = float4v{0.f, 0.f, 0.f, 0.f};
  int slots = 0;  // filled map slots this thread staged
  constexpr int NT = WAVES * 64;

  for (int kc = 0; kc < K; kc += KC) {
    const int kn = (K - kc) < KC ? (K - kc) : KC;
    __syncthreads();  // the chunk before is finished with s_map and the filter buffers
    if constexpr (SRC::kSegments) {
      // The pairs of an offset that fall into this tile are one piece of its list, between
      // two neighbouring entries of the cut table.
      if (tid < kn) {
        const int32_t *cut = source.cuts + (size_t)(kc + tid) * source.cut_stride + tile;
        const int first = cut[0];
        int count = cut[1] - first;
        count = count < 0 ? 0 : (count > TR ? TR : count);
        s_first[tid] = first;
        s_has[tid] = count;
      }
      for (int i = tid; i < kn * TR; i += NT) (&s_map[0][0])[i] = -1;
      __syncthreads();
      // a thread per (offset, pair of the piece): the partner goes to the result row's
      // position.  A thread's loads of one batch are all requested before the first is
      // used (a slot without a pair reads pair 0 of its offset and drops it).
      if (source.L > 0) {
        for (int base = tid; base < kn * TR; base += NT * kDenseMapBatch) {
          int own[kDenseMapBatch], partner[kDenseMapBatch], at[kDenseMapBatch];
#pragma unroll
          for (int u = 0; u < kDenseMapBatch; ++u) {
            const int slot = base + u * NT;
            int kk = slot / TR;
            const int q = slot % TR;
            kk = kk < kn ? kk : kn - 1;
            const bool live = slot < kn * TR && q < s_has[kk];
            int p = live ? s_first[kk] + q : 0;
            p = p < 0 ? 0 : (p < source.L ? p : source.L - 1);
            const int32_t *list = source.pairs + (size_t)(kc + kk) * 2 * source.L;
            own[u] = list[(size_t)source.row_col * source.L + p];
            partner[u] = list[(size_t)source.src_col * source.L + p];
            at[u] = live ? kk : -1;
          }
#pragma unroll
          for (int u = 0; u < kDenseMapBatch; ++u)
            if (at[u] >= 0) s_map[at[u]][(own[u] - r0) & (TR - 1)] = partner[u];
        }
      }
    } else {
      if (tid < kn) s_has[tid] = 0;
      __syncthreads();
      for (int base = tid; base < kn * TR; base += NT * kDenseMapBatch) {
        int v[kDenseMapBatch];
#pragma unroll
        for (int u = 0; u < kDenseMapBatch; ++u) {
          const int slot = base + u * NT;
          int kk = slot / TR;
          kk = kk < kn ? kk : kn - 1;
          const int r = r0 + slot % TR;
          v[u] = source.map[(size_t)(kc + kk) * R + (r < R ? r : R - 1)];
          if (slot >= kn * TR || r >= R) v[u] = -1;
        }
#pragma unroll
        for (int u = 0; u < kDenseMapBatch; ++u) {
          const int slot = base + u * NT;  // (a wave stays inside one offset)
          if (slot < kn * TR) s_map[slot / TR][slot % TR] = v[u];
          const unsigned long long m = __ballot(v[u] >= 0);
          if (m != 0ull && lane == 0) s_has[slot / TR] = 1;
          slots += v[u] >= 0;
        }
      }
    }
    __syncthreads();
    if (wave == 0) {
      const bool has = lane < kn && s_has[lane < kn ? lane : 0] != 0;
      const unsigned long long m = __ballot(has);
      if (has) s_list[__popcll(m & ((1ull << lane) - 1ull))] = lane;
      if (lane == 0) s_count = __popcll(m);
    }
    __syncthreads();
    const int items = s_count;
    if (items == 0) continue;

    // The partner rows of one offset, into the registers of the lanes that multiply them
    // (a lane without a partner reads zeros); returns which of the wave's row groups have
    // a partner at all.
    auto load_rows = [&](int item, vec8 (&rows)[G][KB]) -> int {
      const int kk = s_list[item];
      int present = 0;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int src = s_map[kk][row_first + g * 16];
        const bool mine = src >= 0;
        const bool read = mine && (!kHalfFragment || quad * E::kVec < Q);
        const char *row = read ? a_lane + (size_t)src * ROW_BYTES : zero_lane;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          rows[g][kb] = *reinterpret_cast<const vec8 *>(row + kb * 64);
        if (__ballot(mine) != 0ull) present |= 1 << g;
      }
      return present;
    };
    // The filter fragments of one offset into a buffer: fragment f by wave f % WAVES.
    auto request_filter = [&](int item, int buffer) {
      const char *wk = w_base + (size_t)(kc + s_list[item]) * kBytesPerOffset;
      const uint32_t buf = w_lds + buffer * W_BYTES;
#pragma unroll
      for (int t = 0; t < FPW; ++t) {
        const int f = wave + t * WAVES;
        if (FRAGS % WAVES != 0 && f >= FRAGS) break;
        requestToLds(wk + f * 1024, buf + f * 1024);
      }
    };
    // acc[g] += rows[g] x filter for the two row groups from G0 on that MASK names
    auto multiply = [&](auto g0_tag, auto mask_tag, const vec8 (&rows)[G][KB], const char *wbuf) {
      constexpr int G0 = decltype(g0_tag)::value;
      constexpr int MASK = decltype(mask_tag)::value;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const vec8 wf = *reinterpret_cast<const vec8 *>(wbuf + (nb * KB + kb) * 1024 + lane * 16);
          if constexpr ((MASK & 1) != 0) acc[G0][nb] = E::mfma(wf, rows[G0][kb], acc[G0][nb]);
          if constexpr ((MASK & 2) != 0 && G0 + 1 < G)
            acc[G0 + 1][nb] = E::mfma(wf, rows[G0 + 1][kb], acc[G0 + 1][nb]);
        }
    };
    auto multiply_present = [&](int present, const vec8 (&rows)[G][KB], const char *wbuf) {
      typedef std::integral_constant<int, 1> one;
      typedef std::integral_constant<int, 2> two;
      typedef std::integral_constant<int, 3> both;
      {
        typedef std::integral_constant<int, 0> first;
        const int bits = present & 3;
        if (bits == 3) multiply(first(), both(), rows, wbuf);
        else if (bits == 1) multiply(first(), one(), rows, wbuf);
        else if (bits == 2) multiply(first(), two(), rows, wbuf);
      }
      if constexpr (G == 4) {
        typedef std::integral_constant<int, 2> first;
        const int bits = (present >> 2) & 3;
        if (bits == 3) multiply(first(), both(), rows, wbuf);
        else if (bits == 1) multiply(first(), one(), rows, wbuf);
        else if (bits == 2) multiply(first(), two(), rows, wbuf);
      }
    };
    // Waits for everything this wave has requested.  The rows pass through an empty
    // statement that the compiler must take for their last writer: it then places its own
    // wait for their loads here, where it costs nothing, and not in front of their first
    // use, behind the requests for the offsets after, which it would wait for as well.
    auto landed = [&](vec8 (&rows)[OPP][G][KB]) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int o = 0; o < OPP; ++o)
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) asm volatile("" : "+v"(rows[o][g][kb]));
    };
    // requests rows and filters of the OPP offsets from `item` on into `rows` and LDS buffer
    // `buffer`; an offset past the last one repeats the last (its rows are not multiplied)
    auto request_phase = [&](int item, int buffer, vec8 (&rows)[OPP][G][KB], int (&present)[OPP]) {
#pragma unroll
      for (int o = 0; o < OPP; ++o) {
        const bool there = item + o < items;
        const int it = there ? item + o : items - 1;
        const int got = load_rows(it, rows[o]);
        present[o] = there ? got : 0;
        request_filter(it, buffer * OPP + o);
      }
    };
    // The OPP offsets from `item` on with the rows in `cur`, while the rows and the filters of
    // the next ones travel.  Everything requested here has landed when the barrier is
    // passed, and every wave has left the buffers that the phase after the next writes to.
    auto phase = [&](int item, const int (&present)[OPP], const vec8 (&cur)[OPP][G][KB],
                     vec8 (&nxt)[OPP][G][KB], int (&present_next)[OPP]) {
      const int buffer = (item / OPP) & 1;
      if (item + OPP < items) request_phase(item + OPP, buffer ^ 1, nxt, present_next);
#pragma unroll
      for (int o = 0; o < OPP; ++o)
        multiply_present(present[o], cur[o], s_w + (buffer * OPP + o) * W_BYTES);
      landed(nxt);
      ldsBarrier();
    };

    vec8 rows_a[OPP][G][KB], rows_b[OPP][G][KB];
    int present_a[OPP], present_b[OPP];
    request_phase(0, 0, rows_a, present_a);
    landed(rows_a);
    ldsBarrier();
    for (int i = 0; i < items; i += 2 * OPP) {
      phase(i, present_a, rows_a, rows_b, present_b);
      if (i + OPP < items) phase(i + OPP, present_b, rows_b, rows_a, present_a);
    }
  }
  // lane holds result columns 16*nb + 4*quad + (0..3) of row 16*g + pair of its wave's rows
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int r = r0 + row_first + g * 16;
    if (r >= R) continue;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      S *dst = result + (size_t)r * ldc + col_group * C + nb * 16 + quad * 4;
      S tmp[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) E::store(&tmp[e], acc[g][nb][e]);
      if constexpr (sizeof(S) == 2)
        *reinterpret_cast<uint2 *>(dst) = *reinterpret_cast<const uint2 *>(tmp);
      else
        *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(tmp);
    }
  }
  if constexpr (!SRC::kSegments) {
    // s_has is free again: the waves' slot counts meet there
    __syncthreads();
    int wave_slots = slots;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) wave_slots += __shfl_xor(wave_slots, d, kWave);
    if (lane == 0) s_has[wave] = wave_slots;
    __syncthreads();
    if (tid == 0 && blockIdx.y == 0) {
      int all = 0;
      for (int w = 0; w < WAVES; ++w) all += s_has[w];
      source.filled[blockIdx.x] = all;
    }
  }
}

// ---- pairs that lost their map slot -----------------------------------------------
// Runs behind every gather kernel and returns at once when the kernels found as many
// filled map slots as there are pairs inside their tensors (always, for a rulebook built
// from distinct coordinates).  Otherwise some pairs of one offset share a result row:
// every pair is looked up again, the first one that finds its partner in the slot claims
// it (the kernels have multiplied that one), and each of the others is added to its
// result row here.  The result rows are split into windows of kRepairPoolRows rows; a
// workgroup takes every gridDim.x-th window, reads all pairs and keeps those of its
// window, so no two workgroups touch the same row, map slot or shadow entry.  A touched
// row is rebuilt in the workgroup's fp32 pool (indexed through `shadow`): first the
// partners its map slots hold, as the kernel summed them, then the lost pairs as the
// scan meets them, and it is rounded into the result once, the same single rounding as
// any other row.  Which of the colliding pairs owned the slot depends on the order their
// stores landed in, so the last bits of such rows can differ from run to run; rows
// without collisions are not touched.
constexpr int kRepairPoolRows = 2048;
constexpr int kRepairBlocks = 32;

struct RepairScratch {
  int32_t *shadow;    // [R] pool row of a result row, or -1
  int32_t *pool_row;  // [kRepairBlocks, kRepairPoolRows] result row of a pool row
  float *pool;        // [kRepairBlocks, kRepairPoolRows, C]
};

template <typename E>
__global__ __launch_bounds__(256) void repairLostPairs(
    const typename E::storage *A, int Q, const typename E::storage *W, int64_t sK, int64_t sQ,
    int64_t sC, const int32_t *pairs, int L, int row_col, int src_col, int R, int n_src, int K,
    int row_base, OffsetCounts inl, const int32_t *dev_counts, int32_t *map,
    const int32_t *filled, int n_filled, const int32_t *accepted, int n_accepted, int C,
    RepairScratch scratch, typename E::storage *result, RunIf run_if) {
  if (notWanted(run_if)) return;
  __shared__ int s_found;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  if (tid == 0) s_found = 0;
  __syncthreads();
  // filled slots the gather kernel met, less the pairs the scatter put into the map
  int mine = 0;
  for (int i = tid; i < n_filled; i += 256) mine += filled[i];
  for (int i = tid; i < n_accepted; i += 256) mine -= accepted[i];
  mine = waveInclusiveScan(mine);
  if (lane == 63 && mine != 0) atomicAdd(&s_found, mine);
  __syncthreads();
  if (s_found == 0) return;

  __shared__ int s_row[256];
  __shared__ int s_src[256];
  __shared__ int s_wave_lost[4];
  __shared__ int s_pooled;  // pool rows in use
  int32_t *pool_row = scratch.pool_row + (size_t)blockIdx.x * kRepairPoolRows;
  float *pool = scratch.pool + (size_t)blockIdx.x * kRepairPoolRows * C;
  // Products of gathered rows with filter slices, summed into pool row `at`: below 256
  // result columns the workgroup is 256 / C groups of C threads, a group takes every
  // groups-th reduction channel and the groups' sums meet in shared memory, in group order.
  __shared__ float s_part[256];
  const int groups = C < 256 ? 256 / C : 1;
  const int g = C < 256 ? tid / C : 0;  // == groups: a thread without a part
  const int c_first = C < 256 ? tid % C : tid;
  // whole_row: every partner the map holds for result row `row` (claimed slots hold
  // -2 - partner), stored; else gathered row `row` times slice `k_one`, added.
  auto addProducts = [&](int at, int row, bool whole_row, int k_one) {
    for (int c = c_first; c < C; c += 256) {
      float part = 0.f;
      if (g < groups) {
        for (int kk = whole_row ? 0 : k_one; kk < (whole_row ? K : k_one + 1); ++kk) {
          int from = row;
          if (whole_row) {
            const int m = map[(size_t)kk * R + row];
            if (m == -1) continue;
            from = m >= 0 ? m : -2 - m;
          }
          const typename E::storage *a = A + (size_t)from * Q;
          const typename E::storage *w = W + (size_t)kk * sK + (size_t)c * sC;
          for (int q = g; q < Q; q += groups) part += E::load(a + q) * E::load(w + (size_t)q * sQ);
        }
      }
      if (groups > 1) {
        s_part[tid] = part;
        __syncthreads();
        if (g == 0) {
          part = 0.f;
          for (int gg = 0; gg < groups; ++gg) part += s_part[gg * C + c];
        }
      }
      if (g == 0) pool[(size_t)at * C + c] = whole_row ? part : pool[(size_t)at * C + c] + part;
      if (groups > 1) __syncthreads();
    }
  };
  const int n_windows = (R + kRepairPoolRows - 1) / kRepairPoolRows;
  for (int window = blockIdx.x; window < n_windows; window += gridDim.x) {
    const int r_lo = window * kRepairPoolRows;
    const int r_hi = r_lo + kRepairPoolRows < R ? r_lo + kRepairPoolRows : R;
    for (int i = r_lo + tid; i < r_hi; i += 256) scratch.shadow[i] = -1;
    if (tid == 0) s_pooled = 0;
    __syncthreads();
    for (int k = 0; k < K; ++k) {
      const int n = offsetCount(inl, dev_counts, k);
      const int32_t *base = pairs + (size_t)k * 2 * L;
      for (int p0 = 0; p0 < n; p0 += 256) {
        const int p = p0 + tid;
        int r = -1, src = -1;
        bool lost = false;
        if (p < n) {
          r = base[(size_t)row_col * L + p] - row_base;
          if (r >= r_lo && r < r_hi) {
            src = base[(size_t)src_col * L + p];
            if ((unsigned)src < (unsigned)n_src) {
              int32_t *slot = map + (size_t)k * R + r;
              // the claimed slot holds -2 - partner: no pair finds itself there twice
              lost = !(*slot == src && atomicCAS(slot, src, -2 - src) == src);
            }
          }
        }
        // most steps hold no pair of this window at all
        if (!__syncthreads_or(lost)) continue;
        // lost pairs of this step in pair order
        const unsigned long long b = __ballot(lost);
        if (lane == 0) s_wave_lost[wave] = __popcll(b);
        __syncthreads();
        int before = 0, total = 0;
        for (int w = 0; w < 4; ++w) {
          if (w < wave) before += s_wave_lost[w];
          total += s_wave_lost[w];
        }
        if (lost) {
          const int at = before + __popcll(b & ((1ull << lane) - 1ull));
          s_row[at] = r;
          s_src[at] = src;
        }
        __syncthreads();
        for (int i = 0; i < total; ++i) {
          const int row = s_row[i];
          int at = scratch.shadow[row];
          if (at < 0) {
            at = s_pooled;
            __syncthreads();  // everybody has read the pool's fill state
            if (tid == 0) {
              scratch.shadow[row] = at;
              pool_row[at] = row;
              s_pooled = at + 1;
            }
            // what the gather kernel summed: the partner every slot of the row holds
            addProducts(at, row, true, 0);
          }
          addProducts(at, s_src[i], false, k);
          __syncthreads();  // shadow and the pool row are in place for the next pair
        }
      }
    }
    // round the rebuilt rows into the result; the pool is free for the next window
    const int pooled = s_pooled;
    for (int i = 0; i < pooled; ++i) {
      const int r = pool_row[i];
      for (int c = tid; c < C; c += 256) E::store(result + (size_t)r * C + c, pool[(size_t)i * C + c]);
    }
    __syncthreads();
  }
}

// Number of map slots that hold a partner, added to *total (cleared beforehand).
__global__ __launch_bounds__(256) void countFilledSlots(const int32_t *map, size_t n, int32_t *total) {
  __shared__ int s_sum;
  if (threadIdx.x == 0) s_sum = 0;
  __syncthreads();
  int mine = 0;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    mine += map[i] >= 0 ? 1 : 0;
  mine = waveInclusiveScan(mine);
  if ((threadIdx.x & 63) == 63) atomicAdd(&s_sum, mine);
  __syncthreads();
  if (threadIdx.x == 0 && s_sum != 0) atomicAdd(total, s_sum);
}

// ---- backward filter -------------------------------------------------------------
// Where dW(k, ci, co) goes in filters_grad (element strides).
struct GradLayout {
  int64_t stride_k, stride_ci, stride_co;
};
__device__ __forceinline__ size_t gradOffset(const GradLayout &g, int k, int ci, int co) {
  return (size_t)(k * g.stride_k + ci * g.stride_ci + co * g.stride_co);
}

// One block = 32 x 64 tile of dW[k] over a contiguous slice of the offset's pairs.
template <typename E>
__global__ __launch_bounds__(256) void backwardFilterSimt(const typename E::storage *X,
                                                          const typename E::storage *dY,
                                                          const int32_t *pairs, int L,
                                                          int x_col, int n_in, int n_out, int Ci,
                                                          int Co, OffsetCounts inl,
                                                          const int32_t *dev_counts, int splits,
                                                          float *partial, GradLayout lay,
                                                          typename E::storage *dW) {
  constexpr int TI = 32, TO = 64, PC = 32;
  __shared__ float Xs[PC][TI + 1];
  __shared__ float Ys[PC][TO];
  __shared__ int s_in[PC];
  __shared__ int s_out[PC];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int tiles_o = (Co + TO - 1) / TO;
  const int ci0 = (blockIdx.x / tiles_o) * TI;
  const int co0 = (blockIdx.x % tiles_o) * TO;
  const int k = blockIdx.y;
  const int s = blockIdx.z;
  const int K = gridDim.y;
  const int n = offsetCount(inl, dev_counts, k);
  int per = (n + splits - 1) / splits;
  per = (per + PC - 1) / PC * PC;
  const int p_begin = s * per;
  const int p_end = (p_begin + per) < n ? (p_begin + per) : n;
  const int32_t *in_col = pairs + ((size_t)k * 2 + x_col) * L;
  const int32_t *out_col = pairs + ((size_t)k * 2 + 1 - x_col) * L;
  float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  for (int p0 = p_begin; p0 < p_end; p0 += PC) {
    if (tid < PC) {
      const int p = p0 + tid;
      int i = -1, o = -1;
      if (p < p_end) {
        i = in_col[p];
        o = out_col[p];
        if ((unsigned)i >= (unsigned)n_in || (unsigned)o >= (unsigned)n_out) i = o = -1;
      }
      s_in[tid] = i;
      s_out[tid] = o;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < PC * TI / 256; ++i) {
      const int e = tid + i * 256;
      const int p = e / TI, c = e % TI;
      const int row = s_in[p];
      Xs[p][c] = (row >= 0 && ci0 + c < Ci) ? E::load(X + (size_t)row * Ci + ci0 + c) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < PC * TO / 256; ++i) {
      const int e = tid + i * 256;
      const int p = e / TO, c = e % TO;
      const int row = s_out[p];
      Ys[p][c] = (row >= 0 && co0 + c < Co) ? E::load(dY + (size_t)row * Co + co0 + c) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int p = 0; p < PC; ++p) {
      const float a0 = Xs[p][ty * 2], a1 = Xs[p][ty * 2 + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = Ys[p][tx * 4 + j];
        acc[0][j] += a0 * b;
        acc[1][j] += a1 * b;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ci = ci0 + ty * 2 + i;
    if (ci >= Ci) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int co = co0 + tx * 4 + j;
      if (co >= Co) continue;
      const size_t e = ((size_t)k * Ci + ci) * Co + co;
      if (splits == 1) {
        E::store(dW + gradOffset(lay, k, ci, co), acc[i][j]);
      } else {
        partial[(size_t)s * K * Ci * Co + e] = acc[i][j];
      }
    }
  }
}

// dW[e] = sum over splits, in split order, rounded once.
template <typename E>
__global__ __launch_bounds__(256) void reduceFilterPartials(const float *partial, size_t n,
                                                            int splits, int Ci, int Co,
                                                            GradLayout lay,
                                                            typename E::storage *dW) {
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (size_t)gridDim.x * 256) {
    float s = 0.f;
    for (int i = 0; i < splits; ++i) s += partial[(size_t)i * n + e];
    const int co = (int)(e % Co);
    const size_t kc = e / Co;
    E::store(dW + gradOffset(lay, (int)(kc / Ci), (int)(kc % Ci), co), s);
  }
}

// ---- MFMA backward filter ----------------------------------------------------------
// dW[k] = X_k^T . dY_k over the pairs of offset k.  The pairs of every offset
// are cut into slices of slice_len pairs; one workgroup multiplies one slice of
// one offset and writes a fp32 Ci x Co partial tile, sliceSum adds the tiles of an
// offset in slice order (no float atomics, the same bits on every run).
struct SliceTable {
  int n[kMaxInlineK];      // pairs of the offset
  int first[kMaxInlineK];  // partial tiles in front of the offset's first slice
};

constexpr int kFilterStepPairs = 64;     // pairs multiplied per barrier
constexpr int kFilterIndexChunk = 1024;  // pair indices resident in LDS at once
constexpr int kFilterMaxSlices = 1024;   // about four workgroups per CU
// Many offsets with short lists (5 x 5 x 5) are cut into fewer slices: every slice costs a
// Ci x Co fp32 tile written and summed again (config 5a, 125 offsets: 137 us at 768 slices,
// 149 at 1024; the 27-offset network layers: 183 -> 165 us at 128 channels, 89 -> 77 at 64).
constexpr int kFilterMaxSlicesManyOffsets = 768;
constexpr int kFilterFewOffsets = 32;

// The order in which the workgroups take the slices: by the share of its offset's list that
// lies in front of a slice, so that the workgroups running at one time are at about the same
// rows of the feature and gradient tensors in all offsets (the lists ascend by row), and a
// row fetched for one offset is still in the L2 cache when the others want it.  Entry j names
// the offset of the j-th slice in that order; it is that offset's s-th slice when s earlier
// entries name the same offset.  Workgroup b takes entry (b % 8) * (grid / 8) + b / 8:
// neighbouring entries on one XCD, behind one L2.
struct SliceOrder {
  uint8_t offset[kFilterMaxSlices + kMaxInlineK];
};

struct SlicePlace {
  int k, slice;
};

// For all threads of a workgroup (one barrier inside).  k < 0: no slice for this workgroup.
__device__ __forceinline__ SlicePlace sliceOfWorkgroup(const SliceOrder &order, int total) {
  __shared__ int s_place[2];
  const int per_xcd = gridDim.x >> 3;
  const int j = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (threadIdx.x < 64) {
    int k = -1, earlier = 0;
    if (j < total) {
      k = order.offset[j];
      for (int i = threadIdx.x; i < j; i += 64) earlier += order.offset[i] == k;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) earlier += __shfl_xor(earlier, d, kWave);
    if (threadIdx.x == 0) {
      s_place[0] = k;
      s_place[1] = earlier;
    }
  }
  __syncthreads();
  SlicePlace at;
  at.k = s_place[0];
  at.slice = s_place[1];
  return at;
}

// Both operands are needed with the pair index running along the MFMA's K
// dimension, i.e. transposed relative to the row-major tensors: rows are
// gathered with 16-byte loads and written to LDS transposed ([channel][pair],
// element-sized stores), from where an operand fragment (8 consecutive pairs of
// one channel, 4 for float) is one 16-byte read.  A wave stages 32 pairs x two
// neighbouring 16-byte pieces at a time: every transposed store of the wave then
// writes two runs of 32 consecutive pairs, which no two lanes share a bank in
// (with a row's pieces spread over eight lanes the same stores hit 8 banks and
// took 28 cycles each).  Wave w multiplies the 16-row blocks w, w+4, ... of dW[k]
// against all column blocks.
template <typename E, int CI, int CO>
__global__ __launch_bounds__(256) void backwardFilterMfma(
    const typename E::storage *X, const typename E::storage *dY, const int32_t *pairs, int L,
    int x_col, int n_in, int n_out, int K, SliceTable tab, SliceOrder order, int total_slices,
    int slice_len, float *partial) {
  typedef typename E::vec8 vec8;
  typedef typename E::storage S;
  constexpr int SP = kFilterStepPairs;
  constexpr int EPP = 16 / (int)sizeof(S);          // elements per 16-byte piece
  constexpr int STRIDE = SP * (int)sizeof(S) + 16;  // bytes per channel row: 16 rows hit 64 distinct banks
  constexpr int XP = SP * CI / EPP;                 // 16-byte pieces of X per step
  constexpr int YP = SP * CO / EPP;
  constexpr int XT = XP / 256 > 0 ? XP / 256 : 1;
  constexpr int YT = YP / 256 > 0 ? YP / 256 : 1;
  constexpr int XU = XP / 64;  // staging units (32 pairs x 2 pieces) of X per step
  constexpr int YU = YP / 64;
  static_assert(SP == 64 && (CI / EPP) % 2 == 0 && (CO / EPP) % 2 == 0, "unit = 32 pairs x 2 pieces");
  constexpr int CBW = (CI / 16 + 3) / 4;  // row blocks per wave
  constexpr int COB = CO / 16;
  static_assert(XP % 256 == 0 || XP < 256, "piece split");
  static_assert(YP % 256 == 0 || YP < 256, "piece split");

  __shared__ __attribute__((aligned(16))) char s_x[CI * STRIDE];
  __shared__ __attribute__((aligned(16))) char s_y[CO * STRIDE];
  __shared__ int s_in[kFilterIndexChunk];
  __shared__ int s_out[kFilterIndexChunk];

  const SlicePlace at = sliceOfWorkgroup(order, total_slices);
  if (at.k < 0) return;
  const int k = at.k;
  const int n = tab.n[k];
  const int p_begin = at.slice * slice_len;
  if (p_begin >= n) return;
  const int p_end = p_begin + slice_len < n ? p_begin + slice_len : n;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int32_t *in_col = pairs + ((size_t)k * 2 + x_col) * L;
  const int32_t *out_col = pairs + ((size_t)k * 2 + 1 - x_col) * L;

  float4v acc[CBW][COB];
#pragma unroll
  for (int a = 0; a < CBW; ++a)
#pragma unroll
    for (int b = 0; b < COB; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};

  u32x4 xr[XT], yr[YT];
  auto fetch_step = [&](int local) {  // local = first pair of the step within the index chunk
#pragma unroll
    for (int i = 0; i < XT; ++i) {
      const int u = wave + i * 4;  // unit: pairs 32*(u&1).., pieces 2*(u>>1)..
      xr[i] = u32x4{0u, 0u, 0u, 0u};
      if (XU >= 4 || u < XU) {
        const int row = s_in[local + (u & 1) * 32 + (lane >> 1)];
        if (row >= 0)
          xr[i] = *reinterpret_cast<const u32x4 *>(X + (size_t)row * CI +
                                                   ((u >> 1) * 2 + (lane & 1)) * EPP);
      }
    }
#pragma unroll
    for (int i = 0; i < YT; ++i) {
      const int u = wave + i * 4;
      yr[i] = u32x4{0u, 0u, 0u, 0u};
      if (YU >= 4 || u < YU) {
        const int row = s_out[local + (u & 1) * 32 + (lane >> 1)];
        if (row >= 0)
          yr[i] = *reinterpret_cast<const u32x4 *>(dY + (size_t)row * CO +
                                                   ((u >> 1) * 2 + (lane & 1)) * EPP);
      }
    }
  };
  auto store_step = [&]() {
#pragma unroll
    for (int i = 0; i < XT; ++i) {
      const int u = wave + i * 4;
      if (XU >= 4 || u < XU) {
        const int pr = (u & 1) * 32 + (lane >> 1), c0 = ((u >> 1) * 2 + (lane & 1)) * EPP;
#pragma unroll
        for (int e = 0; e < EPP; ++e) {
          if constexpr (sizeof(S) == 2)
            *reinterpret_cast<u16 *>(&s_x[(c0 + e) * STRIDE + pr * 2]) =
                (u16)(xr[i][e >> 1] >> ((e & 1) * 16));
          else
            *reinterpret_cast<uint32_t *>(&s_x[(c0 + e) * STRIDE + pr * 4]) = xr[i][e];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < YT; ++i) {
      const int u = wave + i * 4;
      if (YU >= 4 || u < YU) {
        const int pr = (u & 1) * 32 + (lane >> 1), c0 = ((u >> 1) * 2 + (lane & 1)) * EPP;
#pragma unroll
        for (int e = 0; e < EPP; ++e) {
          if constexpr (sizeof(S) == 2)
            *reinterpret_cast<u16 *>(&s_y[(c0 + e) * STRIDE + pr * 2]) =
                (u16)(yr[i][e >> 1] >> ((e & 1) * 16));
          else
            *reinterpret_cast<uint32_t *>(&s_y[(c0 + e) * STRIDE + pr * 4]) = yr[i][e];
        }
      }
    }
  };

  for (int c_begin = p_begin; c_begin < p_end; c_begin += kFilterIndexChunk) {
    const int c_len = p_end - c_begin < kFilterIndexChunk ? p_end - c_begin : kFilterIndexChunk;
    const int c_pad = (c_len + SP - 1) / SP * SP;
    __syncthreads();  // the previous chunk's indices are no longer read
    for (int t = tid; t < c_pad; t += 256) {
      int i = -1, o = -1;
      if (t < c_len) {
        i = in_col[c_begin + t];
        o = out_col[c_begin + t];
        if ((unsigned)i >= (unsigned)n_in || (unsigned)o >= (unsigned)n_out) i = o = -1;
      }
      s_in[t] = i;
      s_out[t] = o;
    }
    __syncthreads();
    fetch_step(0);
    for (int local = 0; local < c_pad; local += SP) {
      __syncthreads();  // every wave has read the previous step's operands
      store_step();
      __syncthreads();
      if (local + SP < c_pad) fetch_step(local + SP);
#pragma unroll
      for (int kb = 0; kb < SP / E::kChunk; ++kb) {
        vec8 bfr[COB];
#pragma unroll
        for (int b = 0; b < COB; ++b)
          bfr[b] = *reinterpret_cast<const vec8 *>(
              &s_y[(b * 16 + (lane & 15)) * STRIDE + kb * 64 + (lane >> 4) * 16]);
#pragma unroll
        for (int a = 0; a < CBW; ++a) {
          const int cb = wave + a * 4;
          if (cb < CI / 16) {
            const vec8 afr = *reinterpret_cast<const vec8 *>(
                &s_x[(cb * 16 + (lane & 15)) * STRIDE + kb * 64 + (lane >> 4) * 16]);
#pragma unroll
            for (int b = 0; b < COB; ++b) acc[a][b] = E::mfma(afr, bfr[b], acc[a][b]);
          }
        }
      }
    }
  }
  // lane holds rows 4*(lane/16)+v, column lane%16 of every 16 x 16 block
  float *tile = partial + (size_t)(tab.first[k] + at.slice) * CI * CO;
#pragma unroll
  for (int a = 0; a < CBW; ++a) {
    const int cb = wave + a * 4;
    if (cb < CI / 16) {
#pragma unroll
      for (int b = 0; b < COB; ++b)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          tile[(size_t)(cb * 16 + 4 * (lane >> 4) + v) * CO + b * 16 + (lane & 15)] = acc[a][b][v];
    }
  }
}

// The same product for 2-byte elements and 32 to 128 channels on both sides, with the
// transposition done by the LDS read itself.  The gathered rows go from global memory
// straight into LDS as they are ([pair][channel], 16 bytes per lane, a pair without a
// valid row reads a row of zeros), one step of 64 (or 32) pairs ahead into the other of two
// buffers, and `ds_read_b64_tr_b16` hands a lane four consecutive pairs of one channel:
// within 16 lanes, lane i supplies the address of 4 channels of pair i / 4 and lane j
// receives channel j of the four pairs.  Two such reads are one operand fragment.  No
// element-sized stores, no registers for staging, one barrier per step.
//
// A row's 16-byte pieces are stored permuted (piece ^ f(pair)), since rows lie a
// multiple of the bank width apart: f spreads the eight pairs that half a wavefront
// reads at once over all 64 banks.  Waves are laid out 2 x 2 over the blocks of dW[k].
constexpr int filterRowSwizzle(int row_bytes, int pair) {
  return row_bytes == 256 ? (((pair & 1) << 1) | ((pair & 2) << 1) | (pair & 8))
       : row_bytes == 128 ? ((pair & 2) | ((pair & 8) >> 1))
       : row_bytes == 64  ? ((pair & 8) >> 2)
                          : 0;
}

template <typename E, int CI, int CO, int SP>
__global__ __launch_bounds__(256) void backwardFilterMfmaTr(
    const typename E::storage *X, const typename E::storage *dY, const int32_t *pairs, int L,
    int x_col, int n_in, int n_out, int K, SliceTable tab, SliceOrder order, int total_slices,
    int slice_len, float *partial) {
  typedef typename E::vec8 vec8;
  typedef typename E::storage S;
  typedef short v4i16 __attribute__((ext_vector_type(4)));
  typedef short v8i16 __attribute__((ext_vector_type(8)));
  static_assert(sizeof(S) == 2 && E::kChunk == 32, "2-byte elements, 32 pairs per fragment");
  static_assert(CI % 32 == 0 && CO % 32 == 0 && CI <= 128 && CO <= 128, "two row and column blocks per wave pair");
  // two chunks of row indices: with 128 channels on both sides the buffers leave 16 KiB of
  // half a CU's LDS
  constexpr int kIndexChunk = 512;
  constexpr int kChunkSteps = kIndexChunk / SP;
  constexpr int RBX = CI * 2, RBY = CO * 2;     // bytes per row
  constexpr int XN = SP * RBX / 1024;           // 1 KiB wave-loads per step
  constexpr int YN = SP * RBY / 1024;
  constexpr int AB = CI / 32, BB = CO / 32;     // 16-row / 16-column blocks per wave
  static_assert(SP == 32 || SP == 64, "one or two fragments per step");

  __shared__ __attribute__((aligned(1024))) char s_x[2][SP * RBX];
  __shared__ __attribute__((aligned(1024))) char s_y[2][SP * RBY];
  __shared__ int s_in[2][kIndexChunk];   // row indices of a chunk of pairs, and of the chunk after
  __shared__ int s_out[2][kIndexChunk];

  const SlicePlace at = sliceOfWorkgroup(order, total_slices);
  if (at.k < 0) return;
  const int k = at.k;
  const int n = tab.n[k];
  const int p_begin = at.slice * slice_len;
  if (p_begin >= n) return;
  const int p_end = p_begin + slice_len < n ? p_begin + slice_len : n;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wa = wave >> 1, wb = wave & 1;
  const int32_t *in_col = pairs + ((size_t)k * 2 + x_col) * L;
  const int32_t *out_col = pairs + ((size_t)k * 2 + 1 - x_col) * L;
  const uint32_t x_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)&s_x[0][0];
  const uint32_t y_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)&s_y[0][0];
  const char *zero_row = reinterpret_cast<const char *>(kZeroRow);

  float4v acc[AB][BB];
#pragma unroll
  for (int a = 0; a < AB; ++a)
#pragma unroll
    for (int b = 0; b < BB; ++b) acc[a][b] = float4v{0.f, 0.f, 0.f, 0.f};

  // One step's rows into a buffer: wave-load t of an operand covers 1 KiB of the buffer, lane
  // l its bytes [16 l, 16 l + 16), i.e. a fixed (pair, place) of the step.  Wave w issues
  // loads w, w + 4, ...: `locate` reads all row indices first and forms the addresses (one
  // LDS latency a step, not one a load), `request` issues load u of the wave's XM + YM.
  constexpr int XM = (XN + 3) / 4, YM = (YN + 3) / 4;
  struct StepLoads {
    const char *from[XM + YM];
  };
  // (live == false: a step that is not there; every lane then reads the row of zeros, so
  // that the requests need no branch around them)
  auto locate = [&](int step, bool live, StepLoads &loads) {
    const int *in = s_in[(step / kChunkSteps) & 1] + (step % kChunkSteps) * SP;
    const int *out = s_out[(step / kChunkSteps) & 1] + (step % kChunkSteps) * SP;
    int row[XM + YM];
#pragma unroll
    for (int u = 0; u < XM; ++u) row[u] = in[((wave + u * 4) * 1024 + lane * 16) / RBX];
#pragma unroll
    for (int u = 0; u < YM; ++u) row[XM + u] = out[((wave + u * 4) * 1024 + lane * 16) / RBY];
#pragma unroll
    for (int u = 0; u < XM + YM; ++u) {
      const bool is_x = u < XM;
      const int row_bytes = is_x ? RBX : RBY;
      const int byte = (wave + (is_x ? u : u - XM) * 4) * 1024 + lane * 16;
      const int piece = ((byte % row_bytes) / 16) ^ filterRowSwizzle(row_bytes, byte / row_bytes);
      const char *rows = reinterpret_cast<const char *>(is_x ? (const void *)X : (const void *)dY);
      loads.from[u] = (live && row[u] >= 0 ? rows + (size_t)row[u] * row_bytes : zero_row) + piece * 16;
    }
  };
  auto request = [&](const StepLoads &loads, int u, int buffer) {
    if (u < XM) {
      const int t = wave + u * 4;
      if (XN % 4 == 0 || t < XN) requestToLds(loads.from[u], x_lds + buffer * (SP * RBX) + t * 1024);
    } else if (u < XM + YM) {
      const int t = wave + (u - XM) * 4;
      if (YN % 4 == 0 || t < YN) requestToLds(loads.from[u], y_lds + buffer * (SP * RBY) + t * 1024);
    }
  };
  // fragment of block `block` (16 channels) for the 32 pairs from `pair0` on: lane (c, kq)
  // receives pairs pair0 + 8 kq + (0..7) of channel 16 block + c
  const int sub = lane & 15, kq = lane >> 4;
  auto fragment = [&](const char *buffer, int row_bytes, int block, int pair0) -> vec8 {
    const int pair = pair0 + 8 * kq + (sub >> 2);  // the four pairs after it have the same swizzle
    const int place = (block * 2 + ((sub & 3) >> 1)) ^ filterRowSwizzle(row_bytes, pair);
    const char *at = buffer + pair * row_bytes + place * 16 + (sub & 1) * 8;
    const v4i16 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) v4i16 *)(at));
    const v4i16 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) v4i16 *)(at + 4 * row_bytes));
    const v8i16 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(vec8, both);
  };

  // Row indices of chunk c: four pairs a thread, checked; -1 marks a pair that is not there.
  constexpr int IPT = kIndexChunk / 256;
  int idx_in[IPT], idx_out[IPT];
  auto fetch_indices = [&](int chunk) {
#pragma unroll
    for (int u = 0; u < IPT; ++u) {
      const int at = p_begin + chunk * kIndexChunk + u * 256 + tid;
      int i = -1, o = -1;
      if (at < p_end) {
        i = in_col[at];
        o = out_col[at];
      }
      idx_in[u] = i;
      idx_out[u] = o;
    }
  };
  auto store_indices = [&](int chunk) {
#pragma unroll
    for (int u = 0; u < IPT; ++u) {
      int i = idx_in[u], o = idx_out[u];
      if ((unsigned)i >= (unsigned)n_in || (unsigned)o >= (unsigned)n_out) i = o = -1;
      s_in[chunk & 1][u * 256 + tid] = i;
      s_out[chunk & 1][u * 256 + tid] = o;
    }
  };

  const int steps = (p_end - p_begin + SP - 1) / SP;
  fetch_indices(0);
  store_indices(0);
  __syncthreads();
  StepLoads next_rows;
  locate(0, true, next_rows);
#pragma unroll
  for (int u = 0; u < XM + YM; ++u) request(next_rows, u, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  ldsBarrier();
  for (int step = 0; step < steps; ++step) {
    const int cur = step & 1;
    const int in_chunk = step % kChunkSteps, chunk = step / kChunkSteps;
    // the chunk after this one: its indices are requested at the chunk's first step and are
    // in LDS one barrier before the chunk's last step asks for the next chunk's first rows
    const bool chunk_follows = (chunk + 1) * kChunkSteps < steps;
    if (in_chunk == 0 && chunk_follows) fetch_indices(chunk + 1);
    const bool ahead = step + 1 < steps;
    locate(ahead ? step + 1 : step, ahead, next_rows);
    const char *bx = s_x[cur], *by = s_y[cur];
    // (all requests first: they have one step's multiplies to land)
#pragma unroll
    for (int u = 0; u < XM + YM; ++u) request(next_rows, u, cur ^ 1);
#pragma unroll
    for (int kb = 0; kb < SP / 32; ++kb) {
      vec8 bfr[BB];
#pragma unroll
      for (int b = 0; b < BB; ++b) bfr[b] = fragment(by, RBY, wb * BB + b, kb * 32);
#pragma unroll
      for (int a = 0; a < AB; ++a) {
        const vec8 afr = fragment(bx, RBX, wa * AB + a, kb * 32);
#pragma unroll
        for (int b = 0; b < BB; ++b) acc[a][b] = E::mfma(afr, bfr[b], acc[a][b]);
      }
    }
    if (in_chunk == kChunkSteps - 2 && chunk_follows) store_indices(chunk + 1);
    // the next step's rows have landed, and every wave has left this step's buffers
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    ldsBarrier();
  }
  // lane holds rows 4*(lane/16)+v, column lane%16 of every 16 x 16 block
  float *tile = partial + (size_t)(tab.first[k] + at.slice) * CI * CO;
#pragma unroll
  for (int a = 0; a < AB; ++a)
#pragma unroll
    for (int b = 0; b < BB; ++b)
#pragma unroll
      for (int v = 0; v < 4; ++v)
        tile[(size_t)((wa * AB + a) * 16 + 4 * (lane >> 4) + v) * CO + (wb * BB + b) * 16 + (lane & 15)] =
            acc[a][b][v];
}

// dW[k] = sum of the offset's partial tiles, rounded once.  A block adds 256
// consecutive elements (four per lane): wave g of 16 takes the slices g, g+16, ...
// in eight independent running sums, the sums are combined pairwise in a fixed
// order, so the result depends on the slice count only, never on timing.
constexpr int kSliceSumWaves = 16;
template <typename E>
__global__ __launch_bounds__(64 * kSliceSumWaves) void sliceSum(const float *partial,
                                                                SliceTable tab, int slice_len,
                                                                int tile_elems, int Co,
                                                                GradLayout lay,
                                                                typename E::storage *dW) {
  constexpr int W = kSliceSumWaves;
  __shared__ float4v s_part[W][64];
  const int k = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int g = threadIdx.x >> 6;
  const int e = (blockIdx.x * 64 + lane) * 4;  // tile_elems is a multiple of 256
  const int slices = (tab.n[k] + slice_len - 1) / slice_len;
  float4v acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = float4v{0.f, 0.f, 0.f, 0.f};
  if (e < tile_elems) {
    const float *src = partial + (size_t)tab.first[k] * tile_elems + e;
    for (int i0 = g; i0 < slices; i0 += 8 * W) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + W * u;
        if (i < slices) acc[u] += *reinterpret_cast<const float4v *>(src + (size_t)i * tile_elems);
      }
    }
  }
  s_part[g][lane] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
  __syncthreads();
  if (g == 0 && e < tile_elems) {
    float4v t[W];
#pragma unroll
    for (int i = 0; i < W; ++i) t[i] = s_part[i][lane];
#pragma unroll
    for (int span = 1; span < W; span *= 2)
#pragma unroll
      for (int i = 0; i < W; i += 2 * span) t[i] += t[i + span];
#pragma unroll
    for (int v = 0; v < 4; ++v)
      E::store(dW + gradOffset(lay, k, (e + v) / Co, (e + v) % Co), t[0][v]);
  }
}

// The same sum on a flat grid for filters with many offsets, where most offsets own
// a handful of slices and a 1024-thread workgroup per 256 elements is mostly idle
// waves (at 125 offsets x 128 x 128: 8000 workgroups, dispatch-bound).  An offset with
// at most 16 slices is "thin": each wave sums one 256-element chunk on its own, so a
// workgroup covers 16 chunks and needs no barrier.  The additions are those of
// sliceSum in the same order (a wave's partial there is 0 + slice g when the offset
// has at most 16 slices), so both kernels give the same bits.
struct SumGrid {
  int first[kMaxInlineK];  // workgroups in front of the offset's first one
};
constexpr int kThinSlices = kSliceSumWaves;

template <typename E>
__global__ __launch_bounds__(64 * kSliceSumWaves) void sliceSumFlat(const float *partial,
                                                                    SliceTable tab, SumGrid grid,
                                                                    int K, int slice_len,
                                                                    int tile_elems, int Co,
                                                                    GradLayout lay,
                                                                    typename E::storage *dW) {
  constexpr int W = kSliceSumWaves;
  __shared__ float4v s_part[W][64];
  // last offset whose first workgroup is not behind this one
  int lo = 0, hi = K - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (grid.first[mid] <= (int)blockIdx.x) lo = mid; else hi = mid - 1;
  }
  const int k = lo;
  const int chunk = blockIdx.x - grid.first[k];
  const int lane = threadIdx.x & 63;
  const int g = threadIdx.x >> 6;
  const int slices = (tab.n[k] + slice_len - 1) / slice_len;
  const float *tiles = partial + (size_t)tab.first[k] * tile_elems;
  if (slices <= kThinSlices) {
    const int e = ((chunk * W + g) * 64 + lane) * 4;
    if (e >= tile_elems) return;
    float4v t[W];
#pragma unroll
    for (int i = 0; i < W; ++i) {
      t[i] = float4v{0.f, 0.f, 0.f, 0.f};
      if (i < slices) t[i] += *reinterpret_cast<const float4v *>(tiles + (size_t)i * tile_elems + e);
    }
#pragma unroll
    for (int span = 1; span < W; span *= 2)
#pragma unroll
      for (int i = 0; i < W; i += 2 * span) t[i] += t[i + span];
#pragma unroll
    for (int v = 0; v < 4; ++v)
      E::store(dW + gradOffset(lay, k, (e + v) / Co, (e + v) % Co), t[0][v]);
    return;
  }
  const int e = (chunk * 64 + lane) * 4;
  float4v acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = float4v{0.f, 0.f, 0.f, 0.f};
  {
    const float *src = tiles + e;
    for (int i0 = g; i0 < slices; i0 += 8 * W) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int i = i0 + W * u;
        if (i < slices) acc[u] += *reinterpret_cast<const float4v *>(src + (size_t)i * tile_elems);
      }
    }
  }
  s_part[g][lane] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
  __syncthreads();
  if (g == 0) {
    float4v t[W];
#pragma unroll
    for (int i = 0; i < W; ++i) t[i] = s_part[i][lane];
#pragma unroll
    for (int span = 1; span < W; span *= 2)
#pragma unroll
      for (int i = 0; i < W; i += 2 * span) t[i] += t[i + span];
#pragma unroll
    for (int v = 0; v < 4; ++v)
      E::store(dW + gradOffset(lay, k, (e + v) / Co, (e + v) % Co), t[0][v]);
  }
}

// ---- host side -----------------------------------------------------------------------

inline size_t alignUp(size_t v, size_t a = 256) { return (v + a - 1) / a * a; }

// Workspace blocks are carved from the caller's pointer rounded up to 256 bytes;
// the reported sizes include that slack.
constexpr size_t kBaseAlign = 256;
inline char *alignPtr(void *p) {
  if (p == nullptr) return nullptr;
  return reinterpret_cast<char *>(alignUp(reinterpret_cast<uintptr_t>(p), kBaseAlign));
}

inline int gridFor(size_t n, int cap = 8192) {
  size_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > (size_t)cap ? (size_t)cap : b));
}

// The backward filter's partial tiles are summed on the flat grid from this many
// workgroups on (or as the handle's kernel choice says; the two kernels give the same bits).
constexpr int kFlatSumFromBlocks = 2048;

// fp16/bf16: 16x16x32 MFMA; float: 16x16x4 MFMA; reduction channels in {16, 32, 64, 128}.
bool mfmaShapeOk(ElemType t, int Q, int C) {
  (void)t;  // 16 channels of a 2-byte type run as half-filled fragments
  const bool q_ok = (Q == 16 || Q == 32 || Q == 64 || Q == 128);
  const bool c_ok = (C == 16 || C == 32 || C == 64 || C == 128);
  return q_ok && c_ok;
}

struct GatherDims {
  int R;       // result rows
  int n_src;   // rows of the gathered tensor
  int Q;       // reduction channels
  int C;       // result channels
  int row_col, src_col;
  bool filter_forward;  // B(k, q, c) = W(k, ci = q, co = c); otherwise its transpose
};

GatherDims gatherDims(const ConvProblem &p, GatherDirection dir) {
  GatherDims d;
  d.filter_forward = dir == GatherDirection::kForward;
  if (d.filter_forward) {
    d.Q = p.Ci; d.C = p.Co;
  } else {
    d.Q = p.Co; d.C = p.Ci;
  }
  // The result rows are the pair column the operator writes through: column 1
  // for forward, column 0 for backward data, and the other way round for an
  // inverse convolution, which runs its partner's rulebook backwards.
  if (d.filter_forward != p.inverse) {
    d.R = p.num_out; d.n_src = p.L; d.row_col = 1; d.src_col = 0;
  } else {
    d.R = p.L; d.n_src = p.num_out; d.row_col = 0; d.src_col = 1;
  }
  return d;
}

// The list kernels take the per-offset tables by value and are asked for only when the
// caller has reason to believe the result-row column in order; a row map announced for
// the call is used instead.
bool listsUsable(const ConvProblem &p, const GatherDims &d) {
  (void)d;
  return p.list_trust != ListTrust::kNone && p.K <= kMaxInlineK && p.row_map == nullptr;
}

struct GatherWorkspace {
  int32_t *cuts = nullptr;              // [K, tiles + 1] cut positions of the pair lists
  unsigned long long *verdict = nullptr;
  int32_t *dev_counts = nullptr;
  int32_t *filled = nullptr;  // map slots the gather kernel's workgroups found filled
  int32_t *accepted = nullptr;  // pairs the map scatter's workgroups put into the map
  int map_rows = 0;           // result rows one map holds: the rows of a chunk
  int32_t *shadow = nullptr;  // repairLostPairs' scratch, touched only when pairs collide
  int32_t *pool_row = nullptr;
  float *pool = nullptr;
  int32_t *map = nullptr;
  void *packed = nullptr;
  size_t bytes = 0;
};

// Workgroups of repairLostPairs: one per window of result rows, kRepairBlocks at most.
int repairBlocks(int R) {
  const int windows = (R + kRepairPoolRows - 1) / kRepairPoolRows;
  return windows < 1 ? 1 : (windows > kRepairBlocks ? kRepairBlocks : windows);
}

// Entries of the `accepted` array the scatter kernels may write for K offsets of up to L pairs.
size_t scatterBlocksBound(int K, int L) {
  const size_t flat = (size_t)K * ((size_t)L / 256 + 1);
  const size_t grid = (size_t)K * 1024;
  return flat > grid ? flat : grid;
}

// The row map is built and used for a chunk of result rows at a time, so that it stays
// below kMapChunkBytes however many offsets and rows there are (a multiple of the repair
// window, hence of every tile height).
constexpr size_t kMapChunkBytes = 64u << 20;
int mapChunkRows(int K, int R) {
  size_t rows = kMapChunkBytes / ((size_t)K * 4);
  rows = rows / kRepairPoolRows * kRepairPoolRows;
  if (rows < (size_t)kRepairPoolRows) rows = kRepairPoolRows;
  return rows < (size_t)R ? (int)rows : R;
}

GatherWorkspace carveGather(const ConvProblem &p, const GatherDims &d, void *base) {
  GatherWorkspace ws;
  ws.map_rows = mapChunkRows(p.K, d.R);
  char *ptr = alignPtr(base);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *r = ptr ? ptr + off : nullptr;
    off += alignUp(bytes);
    return r;
  };
  if (p.K > kMaxInlineK) ws.dev_counts = reinterpret_cast<int32_t *>(take((size_t)p.K * 4));
  if (p.K <= kMaxInlineK) {
    // tiles of the narrowest kind (64 rows) bound the table
    ws.cuts = reinterpret_cast<int32_t *>(take((size_t)p.K * ((size_t)d.R / 64 + 2) * 4));
    ws.verdict = reinterpret_cast<unsigned long long *>(take(8));
  }
  ws.filled = reinterpret_cast<int32_t *>(take(((size_t)d.R / 32 + 16) * 4));
  ws.accepted = reinterpret_cast<int32_t *>(take(scatterBlocksBound(p.K, p.L) * 4));
  ws.shadow = reinterpret_cast<int32_t *>(take((size_t)ws.map_rows * 4));
  const size_t repair_blocks = (size_t)repairBlocks(ws.map_rows);
  ws.pool_row = reinterpret_cast<int32_t *>(take(repair_blocks * kRepairPoolRows * 4));
  ws.pool = reinterpret_cast<float *>(take(repair_blocks * kRepairPoolRows * d.C * 4));
  ws.map = reinterpret_cast<int32_t *>(take((size_t)p.K * ws.map_rows * 4));
  if (mfmaShapeOk(p.dtype, d.Q, d.C)) {
    // reduction channels are padded to whole 16-byte fragments (32 for the 2-byte types)
    const size_t chunk = 64 / elemSize(p.dtype);
    const size_t q_padded = ((size_t)d.Q + chunk - 1) / chunk * chunk;
    ws.packed = take((size_t)p.K * q_padded * d.C * elemSize(p.dtype));
  }
  ws.bytes = off + kBaseAlign;
  return ws;
}

// Writes n counts, carried in the kernel arguments, to dst.
__global__ void storeCounts(OffsetCounts c, int n, int32_t *dst) {
  const int i = threadIdx.x;
  if (i < n) dst[i] = c.n[i];
}

// Fills the by-value counts (K <= kMaxInlineK) or puts them into device memory: kMaxInlineK
// counts ride in the arguments of one small launch each, so the host neither allocates nor
// waits, and the call can be captured into a graph like any other.
hipError_t prepareCounts(const LaunchCtx &lc, const ConvProblem &p, OffsetCounts *inl,
                         int32_t *dev_counts, int *max_count) {
  auto clamped = [&](int k) {
    const int64_t n = p.indice_num[k];
    return (int)(n < 0 ? 0 : (n > p.L ? p.L : n));
  };
  int mx = 0;
  for (int k = 0; k < p.K; ++k) mx = clamped(k) > mx ? clamped(k) : mx;
  *max_count = mx;
  for (int k = 0; k < kMaxInlineK; ++k) inl->n[k] = 0;
  if (p.K <= kMaxInlineK) {
    for (int k = 0; k < p.K; ++k) inl->n[k] = clamped(k);
    return hipSuccess;
  }
  for (int k0 = 0; k0 < p.K; k0 += kMaxInlineK) {
    OffsetCounts part;
    const int n = p.K - k0 < kMaxInlineK ? p.K - k0 : kMaxInlineK;
    for (int i = 0; i < kMaxInlineK; ++i) part.n[i] = i < n ? clamped(k0 + i) : 0;
    storeCounts<<<1, kMaxInlineK, 0, lc.stream>>>(part, n, dev_counts + k0);
  }
  return hipGetLastError();
}

// A 128-column result with few pairs per (64-row tile, offset) runs as two
// 64-column halves over 128-row tiles: twice the entries in every block for
// the same accumulator size, at the price of gathering each row twice.
int mfmaTileCols(const ConvProblem &p, const GatherDims &d) {
  if (d.C != 128) return d.C;
  double pairs = 0;
  for (int k = 0; k < p.K; ++k) pairs += (double)p.indice_num[k];
  const double per_tile_offset = pairs * mfmaTileRows(128) / ((double)d.R * p.K);
  return per_tile_offset < 8.0 ? 64 : 128;
}

// Workgroups along x: tiles rounded up to a multiple of the XCD count.
int mfmaGridX(int R, int tile_cols) {
  const int tr = mfmaTileRows(tile_cols);
  return ((R + tr - 1) / tr + 7) / 8 * 8;
}
int denseGridX(int R, int Q, int C) {
  const int rows = denseTileRows(Q, C);
  return ((R + rows - 1) / rows + 7) / 8 * 8;
}

template <typename E, int Q, int C, typename SRC>
void launchMfmaInstance(const LaunchCtx &lc, const void *A, const void *packed,
                        const SRC &source, int R, int K, int ldc, void *result) {
  constexpr int NT = mfmaThreads(C);
  const dim3 grid(mfmaGridX(R, C), ldc / C);
  lc.begin("gatherConvMfma");
  gatherConvMfma<E, Q, C, SRC><<<grid, NT, 0, lc.stream>>>(
      static_cast<const typename E::storage *>(A),
      static_cast<const typename E::storage *>(packed), source, R, K, ldc,
      static_cast<typename E::storage *>(result));
  lc.end();
}

// `tile_cols` result columns per workgroup out of C: a narrower tile has more
// rows, so sparse rulebooks fill their 16-pair blocks better.
template <typename E, int Q, typename SRC>
void launchMfmaByC(const LaunchCtx &lc, int C, int tile_cols, const void *A, const void *packed,
                   const SRC &source, int R, int K, void *result) {
  switch (tile_cols) {
    case 16: launchMfmaInstance<E, Q, 16, SRC>(lc, A, packed, source, R, K, C, result); break;
    case 32: launchMfmaInstance<E, Q, 32, SRC>(lc, A, packed, source, R, K, C, result); break;
    case 64: launchMfmaInstance<E, Q, 64, SRC>(lc, A, packed, source, R, K, C, result); break;
    case 128: launchMfmaInstance<E, Q, 128, SRC>(lc, A, packed, source, R, K, C, result); break;
    default: break;
  }
}

template <typename E, typename SRC>
void launchMfma(const LaunchCtx &lc, int Q, int C, int tile_cols, const void *A, const void *packed,
                const SRC &source, int R, int K, void *result) {
  switch (Q) {
    case 16: launchMfmaByC<E, 16, SRC>(lc, C, tile_cols, A, packed, source, R, K, result); break;
    case 32: launchMfmaByC<E, 32, SRC>(lc, C, tile_cols, A, packed, source, R, K, result); break;
    case 64: launchMfmaByC<E, 64, SRC>(lc, C, tile_cols, A, packed, source, R, K, result); break;
    case 128: launchMfmaByC<E, 128, SRC>(lc, C, tile_cols, A, packed, source, R, K, result); break;
    default: break;
  }
}

template <typename E, int Q, int C>
void launchWaveInstance(const LaunchCtx &lc, const void *A, const void *packed,
                        const SegmentSource &source, int R, int K, void *result) {
  if constexpr (waveKernelShape((int)sizeof(typename E::storage), Q, C)) {
    const int grid = ((R + kWaveTileRows - 1) / kWaveTileRows + 7) / 8 * 8;
    lc.begin("gatherConvWave");
    gatherConvWave<E, Q, C><<<grid, 64, 0, lc.stream>>>(
        static_cast<const typename E::storage *>(A), static_cast<const typename E::storage *>(packed),
        source, R, K, static_cast<typename E::storage *>(result));
    lc.end();
  }
}

template <typename E>
void launchWave(const LaunchCtx &lc, int Q, int C, const void *A, const void *packed,
                const SegmentSource &source, int R, int K, void *result) {
#define WAVE_CASE(q)                                                                      \
  case q:                                                                                 \
    if (C == 16) launchWaveInstance<E, q, 16>(lc, A, packed, source, R, K, result);       \
    else launchWaveInstance<E, q, 32>(lc, A, packed, source, R, K, result);               \
    break;
  switch (Q) {
    WAVE_CASE(16)
    WAVE_CASE(32)
    WAVE_CASE(64)
    WAVE_CASE(128)
    default: break;
  }
#undef WAVE_CASE
}

bool useWaveKernel(const LaunchCtx &lc, ElemType t, int Q, int C) {
  if (lc.choices.wave_per_tile == 0) return false;
  return waveKernelShape((int)elemSize(t), Q, C);
}

// The register-accumulating kernel takes 16 to 128 result columns and 16 to 128 reduction
// channels (16 channels of a 2-byte type as half a fragment).
bool denseShapeOk(ElemType t, int Q, int C) {
  // fp32 rows of 128 channels leave no room for two sets of partner rows and the fragments
  if (t == ElemType::kFloat && Q > 64) return false;
  return (C == 16 || C == 32 || C == 64 || C == 128) && (Q == 16 || Q == 32 || Q == 64 || Q == 128);
}

bool useDenseKernel(const LaunchCtx &lc, const ConvProblem &p, const GatherDims &d) {
  if (!denseShapeOk(p.dtype, d.Q, d.C)) return false;
  if (lc.choices.dense_tiles >= 0) return lc.choices.dense_tiles == 1;
  // What the kernel costs goes with the (tile, offset) pieces that hold a pair at all, what
  // the pair-list kernels cost with the pairs.  Measured on 150000 rows, 3x3x3, fp16, as the
  // share of all (row, offset) slots that hold a pair from which the kernel wins:
  //   result columns   voxels strewn uniformly   scenes (filled sheets and walls)
  //   16, 32           0.35 (0.27: 45 us against 40 us, 0.51: 50 against 60)   0.04 (30 against 32)
  //   64               0.38 (0.27: 86 against 77, 0.51: 104 against 119)      0.15 (67 against 73)
  //   128              0.25 (175 against 183)                                  0.04 (88 against 98)
  // On strewn voxels every piece holds a few pairs; in a scene the pairs of an offset sit in
  // few pieces.  The host only knows the pair counts: sheets and walls show there as offsets
  // with far more pairs than the average offset (in-plane neighbours), which strewn voxels
  // never have.
  double pairs = 0, largest = 0, second = 0;
  for (int k = 0; k < p.K; ++k) {
    const double n = (double)p.indice_num[k];
    pairs += n;
    if (n > largest) {
      second = largest;
      largest = n;
    } else if (n > second) {
      second = n;
    }
  }
  const double fill = pairs / ((double)d.R * p.K);
  // (the largest count is the centre offset of a submanifold convolution: left out)
  const double mean_rest = p.K > 1 ? (pairs - largest) / (p.K - 1) : 0.0;
  const bool sheets = mean_rest > 0 && second >= 1.5 * mean_rest;
  if (d.C <= 32) return fill >= (sheets ? 0.04 : 0.35);
  if (d.C == 64) return fill >= (sheets ? 0.15 : 0.38);
  return fill >= (sheets ? 0.04 : 0.25);
}

template <typename E, int Q, int C, typename SRC>
void launchDenseInstance(const LaunchCtx &lc, const void *A, const void *packed, const SRC &source,
                         int R, int K, void *result) {
  const dim3 grid(denseGridX(R, Q, C), 1);
  lc.begin("gatherConvDense");
  gatherConvDense<E, Q, C, SRC><<<grid, 64 * kDenseWaves, 0, lc.stream>>>(
      static_cast<const typename E::storage *>(A), static_cast<const typename E::storage *>(packed),
      source, R, K, C, static_cast<typename E::storage *>(result));
  lc.end();
}

template <typename E, typename SRC>
void launchDense(const LaunchCtx &lc, int Q, int C, const void *A, const void *packed,
                 const SRC &source, int R, int K, void *result) {
  constexpr bool is_float = std::is_same<E, FloatElem>::value;
#define DENSE_BY_C(q)                                                                           \
  if (C == 16) launchDenseInstance<E, q, 16, SRC>(lc, A, packed, source, R, K, result);         \
  else if (C == 32) launchDenseInstance<E, q, 32, SRC>(lc, A, packed, source, R, K, result);    \
  else if (C == 64) launchDenseInstance<E, q, 64, SRC>(lc, A, packed, source, R, K, result);    \
  else launchDenseInstance<E, q, 128, SRC>(lc, A, packed, source, R, K, result);
  switch (Q) {
    case 16: DENSE_BY_C(16) break;
    case 32: DENSE_BY_C(32) break;
    case 64: DENSE_BY_C(64) break;
    case 128:
      if constexpr (!is_float) { DENSE_BY_C(128) }
      break;
    default: break;
  }
#undef DENSE_BY_C
}

// Row maps are built on the flat grid from this many workgroups of the per-offset grid on.
constexpr int kFlatScatterFromBlocks = 16384;

// Caller brackets this with its timing marks.  dev_counts != nullptr: more offsets
// than the inline tables hold, counts in device memory, grid kernel only.  Returns the
// number of workgroups, each of which writes one entry of `accepted`.
int enqueueScatterRowMap(const LaunchCtx &lc, const int32_t *pairs, int L, int K,
                         const OffsetCounts &inl, const int32_t *dev_counts, int max_count,
                         int row_col, int src_col, int row_base, int n_rows, int n_src,
                         int32_t *map, int32_t *accepted, RunIf run_if) {
  const int gx = (max_count + 255) / 256 > 1024 ? 1024 : (max_count + 255) / 256;
  if (dev_counts == nullptr && K <= kMaxInlineK &&
      (lc.choices.flat_scatter == 1 ||
       (lc.choices.flat_scatter != 0 && (long long)gx * K > kFlatScatterFromBlocks))) {
    OffsetBlocks ob;
    int blocks = 0;
    for (int k = 0; k < K; ++k) {
      ob.first[k] = blocks;
      blocks += inl.n[k] > 0 ? (inl.n[k] + 255) / 256 : 0;
    }
    if (blocks > 0)
      scatterRowMapFlat<<<blocks, 256, 0, lc.stream>>>(pairs, L, inl, ob, K, row_col, src_col,
                                                   row_base, n_rows, n_src, map, accepted, run_if);
    return blocks;
  }
  scatterRowMap<<<dim3(gx, K), 256, 0, lc.stream>>>(pairs, L, inl, dev_counts, row_col, src_col,
                                                 row_base, n_rows, n_src, map, accepted, run_if);
  return gx * K;
}

// The map of result rows [row_base, row_base + n_rows); returns the entries of ws.accepted written.
int launchScatterRowMap(const LaunchCtx &lc, const ConvProblem &p, const GatherDims &d,
                        const GatherWorkspace &ws, const OffsetCounts &inl, int max_count,
                        int row_base, int n_rows, RunIf run_if) {
  if (max_count <= 0) return 0;
  lc.begin("scatterRowMap");
  const int n = enqueueScatterRowMap(lc, p.indice_pairs, p.L, p.K, inl, ws.dev_counts, max_count,
                                     d.row_col, d.src_col, row_base, n_rows, d.n_src, ws.map, ws.accepted,
                                     run_if);
  lc.end();
  return n;
}

template <typename E>
void launchGatherTyped(const LaunchCtx &lc, const ConvProblem &p, const GatherDims &d,
                       const GatherWorkspace &ws, const OffsetCounts &inl, int max_count,
                       const void *gathered, const FilterView &f, bool use_mfma, void *result) {
  typedef typename E::storage S;
  // B(k, q, c): forward q = ci, c = co; backward data q = co, c = ci.
  const int64_t sQ = d.filter_forward ? f.stride_ci : f.stride_co;
  const int64_t sC = d.filter_forward ? f.stride_co : f.stride_ci;
  const bool single_chunk = p.row_map == nullptr && ws.map_rows >= d.R && lc.choices.small_map_chunks != 1;
  // Pair lists whose order nobody has reported yet: the call starts on them all the same,
  // and the row-map kernels are enqueued behind, each of them told to return at once unless
  // the first kernel found the lists out of order (then the list kernel returns at once
  // instead).  Worth it only where the row map is a single chunk of four launches.
  const bool speculate = p.list_trust == ListTrust::kUnknown && single_chunk && lc.choices.lists_on_trust != 0;
  const bool lists = use_mfma && listsUsable(p, d) && (p.list_trust == ListTrust::kInOrder || speculate);
  if (lists) {
    // Pair lists in order (as far as the caller knows: the first kernel checks): the
    // gather kernel reads them cut by tile, no row map.
    const bool dense = useDenseKernel(lc, p, d);
    const int tile_cols = dense ? d.C : mfmaTileCols(p, d);
    const int tile_rows = dense ? denseTileRows(d.Q, d.C) : mfmaTileRows(tile_cols);
    int tile_shift = 0;
    while ((1 << tile_shift) < tile_rows) ++tile_shift;
    const int n_tiles = (d.R + tile_rows - 1) / tile_rows;
    OffsetBlocks ob;
    int list_blocks = 0;
    for (int k = 0; k < kMaxInlineK; ++k) {
      ob.first[k] = list_blocks;
      const int per_block = 256 * kCutPairsPerThread;
      if (k < p.K) list_blocks += inl.n[k] > 0 ? (inl.n[k] + per_block - 1) / per_block : 1;
    }
    const size_t frags = (size_t)p.K * (d.C / 16) * ((d.Q + E::kChunk - 1) / E::kChunk) * 64;
    const int pack_blocks = gridFor(frags, 512);
    lc.begin("packFilterCutPairLists");
    packFilterCutPairLists<E><<<pack_blocks + list_blocks, 256, 0, lc.stream>>>(
        static_cast<const S *>(f.base), f.stride_k, sQ, sC, p.K, d.Q, d.C, static_cast<S *>(ws.packed),
        pack_blocks, p.indice_pairs, p.L, inl, ob, d.row_col, d.src_col, d.R, d.n_src, tile_shift,
        n_tiles, ws.cuts, ws.verdict, p.ticket);
    lc.end();
    SegmentSource src;
    src.pairs = p.indice_pairs;
    src.cuts = ws.cuts;
    src.verdict = ws.verdict;
    src.ticket = p.ticket;
    src.leave_if_unordered = speculate;
    src.L = p.L;
    src.row_col = d.row_col;
    src.src_col = d.src_col;
    src.n_src = d.n_src;
    src.cut_stride = n_tiles + 1;
    src.W = f.base;
    src.sK = f.stride_k;
    src.sQ = sQ;
    src.sC = sC;
    src.counts = inl;
    if (dense)
      launchDense<E, SegmentSource>(lc, d.Q, d.C, gathered, ws.packed, src, d.R, p.K, result);
    else if (tile_cols == d.C && useWaveKernel(lc, p.dtype, d.Q, d.C))
      launchWave<E>(lc, d.Q, d.C, gathered, ws.packed, src, d.R, p.K, result);
    else
      launchMfma<E, SegmentSource>(lc, d.Q, d.C, tile_cols, gathered, ws.packed, src, d.R, p.K, result);
    if (!speculate || lc.choices.lists_on_trust == 1) return;
  }
  // What follows runs always, or (behind lists taken on trust) only when they failed the check.
  const RunIf run_if = lists ? RunIf{ws.verdict, p.ticket} : RunIf{nullptr, 0};
  const bool own_map = p.row_map == nullptr;  // else: built ahead, nothing to clear or fill
  // A map of the library's own covers a chunk of result rows at a time: filled, used by the
  // gather kernel for those rows, checked for lost pairs, and filled again for the next rows.
  int chunk_rows = own_map ? ws.map_rows : d.R;
  if (own_map && lc.choices.small_map_chunks == 1 && chunk_rows > kRepairPoolRows) chunk_rows = kRepairPoolRows;
  const bool dense = use_mfma && useDenseKernel(lc, p, d);
  const int tile_cols = use_mfma && !dense ? mfmaTileCols(p, d) : d.C;
  for (int row_base = 0; row_base < d.R; row_base += chunk_rows) {
    const int rows = d.R - row_base < chunk_rows ? d.R - row_base : chunk_rows;
    const size_t map_elems = (size_t)p.K * rows;
    const int32_t *entries = own_map ? ws.map : p.row_map;
    S *result_rows = static_cast<S *>(result) + (size_t)row_base * d.C;
    int n_filled = 0;    // workgroups along x of the gather kernel = slot counts it leaves
    int n_accepted = 0;  // workgroups of the map scatter = counts of pairs it leaves
    if (use_mfma) {
      // the filter is repacked with the first chunk's map fill (the list kernels' first
      // launch has done it already where they ran)
      const size_t frags = (size_t)p.K * (d.C / 16) * ((d.Q + E::kChunk - 1) / E::kChunk) * 64;
      const int fill_blocks = own_map ? gridFor(map_elems / 4 + 1, 2048) : 0;
      const int pack_blocks = row_base == 0 && !lists ? gridFor(frags, 512) : 0;
      if (fill_blocks + pack_blocks > 0) {
        lc.begin("fillMapPackFilter");
        fillMapPackFilter<E><<<fill_blocks + pack_blocks, 256, 0, lc.stream>>>(
            ws.map, map_elems, fill_blocks, static_cast<const S *>(f.base), f.stride_k, sQ, sC, p.K,
            d.Q, d.C, static_cast<S *>(ws.packed), run_if);
        lc.end();
      }
      if (own_map) n_accepted = launchScatterRowMap(lc, p, d, ws, inl, max_count, row_base, rows, run_if);
      const MapSource map = {entries, ws.filled, run_if};
      if (dense) {
        n_filled = denseGridX(rows, d.Q, d.C);
        launchDense<E, MapSource>(lc, d.Q, d.C, gathered, ws.packed, map, rows, p.K, result_rows);
      } else {
        n_filled = mfmaGridX(rows, tile_cols);
        launchMfma<E, MapSource>(lc, d.Q, d.C, tile_cols, gathered, ws.packed, map, rows, p.K, result_rows);
      }
    } else {
      if (own_map) {
        lc.begin("fillInt32");
        fillInt32<<<gridFor(map_elems), 256, 0, lc.stream>>>(ws.map, map_elems, -1);
        lc.end();
        n_accepted = launchScatterRowMap(lc, p, d, ws, inl, max_count, row_base, rows, run_if);
      }
      dim3 grid((rows + 31) / 32, (d.C + 63) / 64);
      n_filled = (int)grid.x;
      lc.begin("gatherConvSimt");
      gatherConvSimt<E><<<grid, 256, 0, lc.stream>>>(static_cast<const S *>(gathered), d.Q,
                                                  static_cast<const S *>(f.base), f.stride_k, sQ, sC,
                                                  entries, rows, p.K, inl, ws.dev_counts, d.C,
                                                  ws.filled, result_rows);
      lc.end();
    }
    if (p.distinct_pairs || !own_map) continue;  // a map built ahead was checked when it was built
    // returns at once unless pairs of one offset share a result row
    lc.begin("repairLostPairs");
    repairLostPairs<E><<<repairBlocks(rows), 256, 0, lc.stream>>>(
        static_cast<const S *>(gathered), d.Q, static_cast<const S *>(f.base), f.stride_k, sQ, sC,
        p.indice_pairs, p.L, d.row_col, d.src_col, rows, d.n_src, p.K, row_base, inl, ws.dev_counts,
        ws.map, ws.filled, n_filled, ws.accepted, n_accepted, d.C,
        RepairScratch{ws.shadow, ws.pool_row, ws.pool}, result_rows, run_if);
    lc.end();
  }
}

struct FilterGradWorkspace {
  int32_t *dev_counts = nullptr;
  float *partial = nullptr;
  int splits = 1;
  size_t bytes = 0;
};

bool filterMfmaShapeOk(const ConvProblem &p) {
  auto ok = [](int c) { return c == 16 || c == 32 || c == 64 || c == 128; };
  return ok(p.Ci) && ok(p.Co) && p.K <= kMaxInlineK;
}

// Slices the MFMA kernels cut the pair lists into at most: kFilterMaxSlices (fewer for many
// offsets), or what a capped workspace leaves beside one tile per offset.
int filterMaxSlices(const ConvProblem &p) {
  const int most = p.K <= kFilterFewOffsets ? kFilterMaxSlices : kFilterMaxSlicesManyOffsets;
  if (p.max_partial_tiles <= 0) return most;
  const int room = p.max_partial_tiles - p.K;
  return room < 1 ? 1 : (room > most ? most : room);
}

int filterGradSplits(const ConvProblem &p) {
  // Bounded by the tensor shape only, so the workspace query and the launch
  // agree whatever indice_num holds.
  int s = (p.L + 4095) / 4096;
  if (s < 1) s = 1;
  if (s > 32) s = 32;
  return s;
}

FilterGradWorkspace carveFilterGrad(const ConvProblem &p, void *base) {
  FilterGradWorkspace ws;
  char *ptr = alignPtr(base);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *r = ptr ? ptr + off : nullptr;
    off += alignUp(bytes);
    return r;
  };
  if (p.K > kMaxInlineK) ws.dev_counts = reinterpret_cast<int32_t *>(take((size_t)p.K * 4));
  ws.splits = filterGradSplits(p);
  size_t tiles = ws.splits > 1 ? (size_t)ws.splits * p.K : 0;
  // the MFMA path writes at most filterMaxSlices + K partial tiles
  if (filterMfmaShapeOk(p) && (size_t)filterMaxSlices(p) + p.K > tiles)
    tiles = (size_t)filterMaxSlices(p) + p.K;
  if (tiles > 0) ws.partial = reinterpret_cast<float *>(take(tiles * p.Ci * p.Co * 4));
  ws.bytes = off + kBaseAlign;
  return ws;
}

// filters_grad is [K, Ci, Co] unless the caller asked for another layout.
GradLayout gradLayout(const ConvProblem &p) {
  GradLayout g;
  if (p.grad_stride_k == 0 && p.grad_stride_ci == 0 && p.grad_stride_co == 0) {
    g.stride_k = (int64_t)p.Ci * p.Co; g.stride_ci = p.Co; g.stride_co = 1;
  } else {
    g.stride_k = p.grad_stride_k; g.stride_ci = p.grad_stride_ci; g.stride_co = p.grad_stride_co;
  }
  return g;
}

template <typename E, int CI, int CO>
void launchFilterMfmaInstance(const LaunchCtx &lc, const ConvProblem &p, const SliceTable &tab,
                              const SliceOrder &order, int slice_len, int total_slices, float *partial, const void *features,
                              const void *output_grad, void *filters_grad) {
  typedef typename E::storage S;
  constexpr bool kTransposingReads = sizeof(S) == 2 && CI >= 32 && CO >= 32;
  const int grid = (total_slices + 7) / 8 * 8;
  lc.begin(kTransposingReads && lc.choices.filter_stores != 1 ? "backwardFilterMfmaTr" : "backwardFilterMfma");
  if (total_slices > 0) {
    if constexpr (kTransposingReads) {
      if (lc.choices.filter_stores != 1) {
        // Steps of 32 pairs halve the row buffers: below 128 x 128 channels more workgroups
        // share a CU then, which pays when the slices are long (network 64 x 64: 101 -> 88 us;
        // on slices of a few steps the shorter steps only add barriers: config 4 23.7 -> 25.3 us).
        const bool short_steps = CI + CO < 256 && slice_len >= 2048;
        auto kernel = short_steps ? backwardFilterMfmaTr<E, CI, CO, 32> : backwardFilterMfmaTr<E, CI, CO, 64>;
        kernel<<<grid, 256, 0, lc.stream>>>(
            static_cast<const S *>(features), static_cast<const S *>(output_grad), p.indice_pairs,
            p.L, p.inverse ? 1 : 0, p.inverse ? p.num_out : p.L, p.inverse ? p.L : p.num_out, p.K,
            tab, order, total_slices, slice_len, partial);
      } else {
        backwardFilterMfma<E, CI, CO><<<grid, 256, 0, lc.stream>>>(
            static_cast<const S *>(features), static_cast<const S *>(output_grad), p.indice_pairs,
            p.L, p.inverse ? 1 : 0, p.inverse ? p.num_out : p.L, p.inverse ? p.L : p.num_out, p.K,
            tab, order, total_slices, slice_len, partial);
      }
    } else {
      backwardFilterMfma<E, CI, CO><<<grid, 256, 0, lc.stream>>>(
          static_cast<const S *>(features), static_cast<const S *>(output_grad), p.indice_pairs,
          p.L, p.inverse ? 1 : 0, p.inverse ? p.num_out : p.L, p.inverse ? p.L : p.num_out, p.K,
          tab, order, total_slices, slice_len, partial);
    }
  }
  lc.end();
  // Many offsets of few slices each: the flat grid, on which such an offset takes a
  // sixteenth of the workgroups (same bits).
  constexpr int kChunks = CI * CO / 256;
  SumGrid sg;
  int blocks = 0;
  for (int k = 0; k < p.K; ++k) {
    const int sl = (tab.n[k] + slice_len - 1) / slice_len;
    sg.first[k] = blocks;
    blocks += sl <= kThinSlices ? (kChunks + kSliceSumWaves - 1) / kSliceSumWaves : kChunks;
  }
  const int flat_mode = lc.choices.flat_slice_sum;
  const bool flat = flat_mode == 1 || (flat_mode < 0 && kChunks * p.K > kFlatSumFromBlocks);
  lc.begin("sliceSum");
  if (flat)
    sliceSumFlat<E><<<blocks, 64 * kSliceSumWaves, 0, lc.stream>>>(
        partial, tab, sg, p.K, slice_len, CI * CO, CO, gradLayout(p), static_cast<S *>(filters_grad));
  else
    sliceSum<E><<<dim3(kChunks, p.K), 64 * kSliceSumWaves, 0, lc.stream>>>(
        partial, tab, slice_len, CI * CO, CO, gradLayout(p), static_cast<S *>(filters_grad));
  lc.end();
}

template <typename E, int CI>
void launchFilterMfmaByCo(const LaunchCtx &lc, const ConvProblem &p, const SliceTable &tab,
                          const SliceOrder &order, int slice_len, int total_slices, float *partial, const void *features,
                          const void *output_grad, void *filters_grad) {
  switch (p.Co) {
    case 16: launchFilterMfmaInstance<E, CI, 16>(lc, p, tab, order, slice_len, total_slices, partial, features, output_grad, filters_grad); break;
    case 32: launchFilterMfmaInstance<E, CI, 32>(lc, p, tab, order, slice_len, total_slices, partial, features, output_grad, filters_grad); break;
    case 64: launchFilterMfmaInstance<E, CI, 64>(lc, p, tab, order, slice_len, total_slices, partial, features, output_grad, filters_grad); break;
    case 128: launchFilterMfmaInstance<E, CI, 128>(lc, p, tab, order, slice_len, total_slices, partial, features, output_grad, filters_grad); break;
    default: break;
  }
}

// Slice length from the real pair count: about kFilterMaxSlices workgroups
// whatever the density, and never more than kFilterMaxSlices + K partial tiles.
template <typename E>
void launchFilterMfma(const LaunchCtx &lc, const ConvProblem &p, const FilterGradWorkspace &ws,
                      const OffsetCounts &inl, const void *features, const void *output_grad,
                      void *filters_grad) {
  {
    SliceTable tab;
    long long total = 0;
    for (int k = 0; k < p.K; ++k) total += inl.n[k];
    // (the larger number of slices only where they stay long: a fourth workgroup a CU does not
    // fit, and a second round of short slices costs more than it spreads; config 3, 404 000
    // pairs: 24 us at 701 slices, 31 us at 789)
    int max_slices = filterMaxSlices(p);
    if (total < (long long)kFilterMaxSlices * 2048 && max_slices > kFilterMaxSlicesManyOffsets)
      max_slices = kFilterMaxSlicesManyOffsets;
    int slice_len = (int)((total + max_slices - 1) / max_slices);
    slice_len = (slice_len + kFilterStepPairs - 1) / kFilterStepPairs * kFilterStepPairs;
    // A slice has fixed costs (the first rows' round trip, a Ci x Co fp32 tile written and summed
    // again): few pairs are not cut finer than this, at the price of idle CUs (config 5b, 128 x
    // 128, 400 000 pairs: 56 -> 46 us at 1024; config 2, 32 x 32, 205 000 pairs: 22.5 -> 19 us at 512).
    const int least = p.Ci * p.Co >= 128 * 128 ? 1024 : 512;
    if (slice_len < least) slice_len = least;
    int first = 0;
    for (int k = 0; k < kMaxInlineK; ++k) {
      const int n = k < p.K ? inl.n[k] : 0;
      const int slices = (n + slice_len - 1) / slice_len;
      tab.n[k] = n;
      tab.first[k] = first;
      first += slices;
    }
    // slices in the order of the share of their offset's list in front of them, in `steps`
    // steps of that share (as many as the longest list has slices)
    SliceOrder order;
    int steps = 1, next[kMaxInlineK], count[kMaxInlineK];
    for (int k = 0; k < p.K; ++k) {
      next[k] = 0;
      count[k] = (tab.n[k] + slice_len - 1) / slice_len;
      if (count[k] > steps) steps = count[k];
    }
    int placed = 0;
    for (int t = 0; t < steps; ++t)
      for (int k = 0; k < p.K; ++k)
        while (next[k] < count[k] && (long long)next[k] * steps < (long long)(t + 1) * count[k]) {
          order.offset[placed++] = (uint8_t)k;
          ++next[k];
        }
    switch (p.Ci) {
      case 16: launchFilterMfmaByCo<E, 16>(lc, p, tab, order, slice_len, first, ws.partial, features, output_grad, filters_grad); break;
      case 32: launchFilterMfmaByCo<E, 32>(lc, p, tab, order, slice_len, first, ws.partial, features, output_grad, filters_grad); break;
      case 64: launchFilterMfmaByCo<E, 64>(lc, p, tab, order, slice_len, first, ws.partial, features, output_grad, filters_grad); break;
      case 128: launchFilterMfmaByCo<E, 128>(lc, p, tab, order, slice_len, first, ws.partial, features, output_grad, filters_grad); break;
      default: break;
    }
  }
}

template <typename E>
void launchFilterGradTyped(const LaunchCtx &lc, const ConvProblem &p,
                           const FilterGradWorkspace &ws, const OffsetCounts &inl,
                           const void *features, const void *output_grad, void *filters_grad) {
  typedef typename E::storage S;
  // The MFMA path moves rows with 16-byte loads.
  const bool ptr_ok = ((reinterpret_cast<uintptr_t>(features) |
                        reinterpret_cast<uintptr_t>(output_grad)) & 15u) == 0;
  if (filterMfmaShapeOk(p) && ptr_ok && lc.choices.gather_simt != 1) {
    launchFilterMfma<E>(lc, p, ws, inl, features, output_grad, filters_grad);
    return;
  }
  const int tiles = ((p.Ci + 31) / 32) * ((p.Co + 63) / 64);
  dim3 grid(tiles, p.K, ws.splits);
  lc.begin("backwardFilterSimt");
  backwardFilterSimt<E><<<grid, 256, 0, lc.stream>>>(
      static_cast<const S *>(features), static_cast<const S *>(output_grad), p.indice_pairs, p.L,
      p.inverse ? 1 : 0, p.inverse ? p.num_out : p.L, p.inverse ? p.L : p.num_out, p.Ci, p.Co, inl,
      ws.dev_counts, ws.splits, ws.partial, gradLayout(p), static_cast<S *>(filters_grad));
  lc.end();
  if (ws.splits > 1) {
    const size_t n = (size_t)p.K * p.Ci * p.Co;
    lc.begin("reduceFilterPartials");
    reduceFilterPartials<E><<<gridFor(n), 256, 0, lc.stream>>>(
        ws.partial, n, ws.splits, p.Ci, p.Co, gradLayout(p), static_cast<S *>(filters_grad));
    lc.end();
  }
}

}  // namespace

size_t gatherConvWorkspaceBytes(const ConvProblem &p, GatherDirection dir) {
  return carveGather(p, gatherDims(p, dir), nullptr).bytes;
}

hipError_t launchGatherConv(const LaunchCtx &lc, const ConvProblem &p, GatherDirection dir,
                            const void *gathered, const FilterView &filters, void *workspace,
                            void *result) {
  const GatherDims d = gatherDims(p, dir);
  const GatherWorkspace ws = carveGather(p, d, workspace);
  OffsetCounts inl;
  int max_count = 0;
  hipError_t err = prepareCounts(lc, p, &inl, ws.dev_counts, &max_count);
  if (err != hipSuccess) return err;

  // The MFMA kernel moves rows with 16-byte accesses and packs a partner row
  // into 24 bits of a list entry.
  const bool ptr_ok =
      ((reinterpret_cast<uintptr_t>(gathered) | reinterpret_cast<uintptr_t>(result)) & 15u) == 0;
  const bool use_mfma = mfmaShapeOk(p.dtype, d.Q, d.C) && ptr_ok && d.n_src <= (1 << 24) &&
                        lc.choices.gather_simt != 1;
  switch (p.dtype) {
    case ElemType::kHalf:
      launchGatherTyped<HalfElem>(lc, p, d, ws, inl, max_count, gathered, filters, use_mfma, result);
      break;
    case ElemType::kBFloat16:
      launchGatherTyped<BFloat16Elem>(lc, p, d, ws, inl, max_count, gathered, filters, use_mfma, result);
      break;
    case ElemType::kFloat:
      launchGatherTyped<FloatElem>(lc, p, d, ws, inl, max_count, gathered, filters, use_mfma, result);
      break;
  }
  return hipGetLastError();
}

RowMapShape rowMapShape(const ConvProblem &p, GatherDirection dir) {
  const GatherDims d = gatherDims(p, dir);
  return RowMapShape{p.K, p.L, d.R, d.n_src, d.row_col};
}

// entries [K, rows] | filled-slot counter | per-offset counts [K] (for K beyond the inline limit)
size_t rowMapBytes(int K, int rows) {
  return alignUp((size_t)K * rows * 4) + alignUp(4) + alignUp((size_t)K * 4) + kBaseAlign;
}

hipError_t buildRowMap(const LaunchCtx &lc, const int32_t *indice_pairs, const int64_t *indice_num,
                       const RowMapShape &shape, void *row_map, int32_t *filled_host) {
  const size_t map_elems = (size_t)shape.K * shape.rows;
  int32_t *map = static_cast<int32_t *>(row_map);
  int32_t *counter = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(map) + alignUp(map_elems * 4));
  int32_t *dev_counts = reinterpret_cast<int32_t *>(reinterpret_cast<char *>(counter) + alignUp(4));
  ConvProblem p;
  p.K = shape.K;
  p.L = shape.L;
  p.indice_pairs = indice_pairs;
  p.indice_num = indice_num;
  OffsetCounts inl;
  int max_count = 0;
  hipError_t err = prepareCounts(lc, p, &inl, shape.K > kMaxInlineK ? dev_counts : nullptr, &max_count);
  if (err != hipSuccess) return err;
  lc.begin("fillInt32");
  fillInt32<<<gridFor(map_elems), 256, 0, lc.stream>>>(map, map_elems, -1);
  lc.end();
  fillInt32<<<1, 256, 0, lc.stream>>>(counter, 1, 0);
  if (max_count > 0) {
    lc.begin("scatterRowMap");
    enqueueScatterRowMap(lc, indice_pairs, shape.L, shape.K, inl,
                         shape.K > kMaxInlineK ? dev_counts : nullptr, max_count, shape.row_column,
                         1 - shape.row_column, 0, shape.rows, shape.source_rows, map, nullptr, RunIf{nullptr, 0});
    lc.end();
  }
  if (filled_host == nullptr) return hipGetLastError();
  lc.begin("countFilledSlots");
  countFilledSlots<<<gridFor(map_elems, 1024), 256, 0, lc.stream>>>(map, map_elems, counter);
  lc.end();
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  return hipMemcpyAsync(filled_host, counter, 4, hipMemcpyDeviceToHost, lc.stream);
}

size_t backwardFilterWorkspaceBytes(const ConvProblem &p) {
  return carveFilterGrad(p, nullptr).bytes;
}

bool backwardFilterLaunchesOnly(const ConvProblem &p) { return p.K <= kMaxInlineK; }

hipError_t launchBackwardFilter(const LaunchCtx &lc, const ConvProblem &p, const void *features,
                                const void *output_grad, void *workspace, void *filters_grad) {
  const FilterGradWorkspace ws = carveFilterGrad(p, workspace);
  OffsetCounts inl;
  int max_count = 0;
  hipError_t err = prepareCounts(lc, p, &inl, ws.dev_counts, &max_count);
  if (err != hipSuccess) return err;
  switch (p.dtype) {
    case ElemType::kHalf:
      launchFilterGradTyped<HalfElem>(lc, p, ws, inl, features, output_grad, filters_grad);
      break;
    case ElemType::kBFloat16:
      launchFilterGradTyped<BFloat16Elem>(lc, p, ws, inl, features, output_grad,
                                          filters_grad);
      break;
    case ElemType::kFloat:
      launchFilterGradTyped<FloatElem>(lc, p, ws, inl, features, output_grad, filters_grad);
      break;
  }
  return hipGetLastError();
}

}  // namespace sparse_conv
}  // namespace mluop
