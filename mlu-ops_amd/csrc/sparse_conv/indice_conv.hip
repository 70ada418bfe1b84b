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
#include <cstdlib>
#include <type_traits>

#include "sparse_conv/indice_conv.h"

namespace mluop {
namespace sparse_conv {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

constexpr int kWave = 64;
constexpr int kMaxInlineK = 128;

// Pair counts per offset, passed by value for the common small kernel volumes.
struct OffsetCounts {
  int n[kMaxInlineK];
};

__device__ __forceinline__ int offsetCount(const OffsetCounts &inl, const int32_t *dev, int k) {
  return dev != nullptr ? dev[k] : inl.n[k];
}

// ---- element types ---------------------------------------------------------

struct HalfElem {
  typedef _Float16 storage;
  typedef half8 vec8;
  static __device__ __forceinline__ float load(const storage *p) { return (float)*p; }
  static __device__ __forceinline__ void store(storage *p, float v) { *p = (_Float16)v; }
  static __device__ __forceinline__ float4v mfma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

struct BFloat16Elem {
  typedef u16 storage;
  typedef bf16x8 vec8;
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
  static __device__ __forceinline__ float load(const storage *p) { return *p; }
  static __device__ __forceinline__ void store(storage *p, float v) { *p = v; }
};

// ---- row map ---------------------------------------------------------------

__global__ __launch_bounds__(256) void fillInt32(int32_t *dst, size_t n, int32_t value) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  for (; i < n; i += stride) dst[i] = value;
}

// map[k][row] = partner row, for the first indice_num[k] pairs of every offset.
// row_col / src_col select which pair column owns the result row (1 for
// forward, 0 for backward data).  Indices outside their tensor are ignored.
__global__ __launch_bounds__(256) void scatterRowMap(const int32_t *pairs, int L,
                                                     OffsetCounts inl, const int32_t *dev_counts,
                                                     int row_col, int src_col, int n_rows,
                                                     int n_src, int32_t *map) {
  const int k = blockIdx.y;
  const int n = offsetCount(inl, dev_counts, k);
  const int32_t *base = pairs + (size_t)k * 2 * L;
  for (int p = blockIdx.x * 256 + threadIdx.x; p < n; p += gridDim.x * 256) {
    const int r = base[(size_t)row_col * L + p];
    const int s = base[(size_t)src_col * L + p];
    if ((unsigned)r < (unsigned)n_rows && (unsigned)s < (unsigned)n_src)
      map[(size_t)k * n_rows + r] = s;
  }
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
                                                      typename E::storage *result) {
  constexpr int TR = 32, TC = 64, QC = 32;
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
}

// ---- MFMA gather convolution ---------------------------------------------------

// Filter repacked into 16x16x32 B-operand fragments:
// packed[(((k*(C/16) + nb)*(Q/32) + kb)*64 + lane)*8 + e]
//   = B(k, q = kb*32 + 8*(lane/16) + e, c = nb*16 + lane%16).
template <typename E>
__global__ __launch_bounds__(256) void packFilterFragments(const typename E::storage *W,
                                                           int64_t sK, int64_t sQ, int64_t sC,
                                                           int K, int Q, int C,
                                                           typename E::storage *packed) {
  const size_t total = (size_t)K * (C / 16) * (Q / 32) * 64;
  for (size_t t = (size_t)blockIdx.x * 256 + threadIdx.x; t < total;
       t += (size_t)gridDim.x * 256) {
    const int lane = (int)(t & 63);
    size_t rest = t >> 6;
    const int kb = (int)(rest % (Q / 32));
    rest /= (Q / 32);
    const int nb = (int)(rest % (C / 16));
    const int k = (int)(rest / (C / 16));
    const int c = nb * 16 + (lane & 15);
    const int qb = kb * 32 + 8 * (lane >> 4);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      packed[t * 8 + e] = W[(size_t)k * sK + (size_t)(qb + e) * sQ + (size_t)c * sC];
  }
}

constexpr int mfmaTileRows(int C) {
  // fp32 accumulator tile of at most 32 KiB: four workgroups share a CU's LDS.
  return C <= 32 ? 256 : (C <= 64 ? 128 : 64);
}
constexpr int mfmaColBlocksPerWave(int C) { return C >= 128 ? 2 : 1; }
constexpr int mfmaBlocksInFlight(int Q, int C) {
  // Register budget: each block in flight holds Q/32 A fragments and
  // Q/32 * column-blocks B fragments (4 VGPRs each).
  return (Q / 32) * (1 + mfmaColBlocksPerWave(C)) <= 4 ? 4 : 2;
}

constexpr int kOffsetChunk = 9;  // offsets whose pair lists are resident in LDS at once

// Workgroup = TR result rows x all C columns; wave w owns columns
// [w*16*NB, (w+1)*16*NB) of the fp32 accumulator tile in LDS, so no two waves
// ever touch the same accumulator element and every element sees its
// contributions in ascending offset order.
//
// Per chunk of kOffsetChunk offsets:
//   A   lanes hold map[k][row] for all offsets of the chunk (loaded while the
//       previous chunk was being multiplied), ballot which rows have a partner
//       and compact the (row, partner) entries of every offset into LDS lists;
//       one wave turns the list lengths into a flat list of 16-entry blocks;
//   B   every wave walks the block list, several blocks in flight: gather 16
//       partner rows as the MFMA A operand (zero rows pad a short block),
//       multiply by its B fragments of W[k], add the 16 x 16*NB result into
//       the accumulator rows of the entries.
// The accumulator tile is stored with its 16-column groups XOR-swizzled by the
// row index so that the four rows a wave updates at once fall into different
// LDS banks more often than not.
template <typename E, int Q, int C>
__global__ __launch_bounds__(64 * (C / 16 / mfmaColBlocksPerWave(C)))
void gatherConvMfma(const typename E::storage *A, const typename E::storage *packedW,
                    const int32_t *map, int R, int K, OffsetCounts inl,
                    const int32_t *dev_counts, typename E::storage *result) {
  typedef typename E::vec8 vec8;
  constexpr int NB = mfmaColBlocksPerWave(C);
  constexpr int WAVES = C / 16 / NB;
  constexpr int NT = 64 * WAVES;
  constexpr int TR = mfmaTileRows(C);
  constexpr int NSEG = TR / 64;
  constexpr int SEG_ITERS = (NSEG + WAVES - 1) / WAVES;  // segments a wave scans
  constexpr int KB = Q / 32;
  constexpr int KC = kOffsetChunk;
  constexpr int D = mfmaBlocksInFlight(Q, C);
  constexpr int GROUPS = C / 16;  // 16-column groups per accumulator row (power of two)
  constexpr int MAX_BLOCKS = KC * (TR / 16);

  __shared__ float s_acc[TR * C];
  __shared__ int32_t s_src[KC][TR];
  __shared__ __attribute__((aligned(4))) uint8_t s_row[KC][TR];
  __shared__ int s_cnt[KC][NSEG];
  __shared__ int s_tot[KC];
  __shared__ uint16_t s_blk[MAX_BLOCKS];
  __shared__ int s_nblk;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r0 = blockIdx.x * TR;
  const int grp0 = wave * NB;  // first 16-column group of this wave
  const unsigned long long lt_mask = (1ull << lane) - 1ull;

  for (int i = tid; i < TR * C; i += NT) s_acc[i] = 0.f;

  // map entries of the chunk being prepared, per segment this wave scans
  int idx[SEG_ITERS][KC];
  auto load_chunk = [&](int kc) {
#pragma unroll
    for (int it = 0; it < SEG_ITERS; ++it) {
      const int seg = wave + it * WAVES;
      const int r = r0 + seg * 64 + lane;
#pragma unroll
      for (int kk = 0; kk < KC; ++kk) {
        // Unconditional loads from clamped addresses keep all of them in flight;
        // offsets without pairs hold -1 everywhere in the map.
        const bool ok = seg < NSEG && kc + kk < K && r < R;
        const int k_safe = kc + kk < K ? kc + kk : K - 1;
        const int r_safe = (seg < NSEG && r < R) ? r : R - 1;
        const int v = map[(size_t)k_safe * R + r_safe];
        idx[it][kk] = ok ? v : -1;
      }
    }
  };
  load_chunk(0);

  for (int kc = 0; kc < K; kc += KC) {
    const int kn = (K - kc) < KC ? (K - kc) : KC;
    // A: per-segment hit counts, then compaction into the per-offset lists.
#pragma unroll
    for (int it = 0; it < SEG_ITERS; ++it) {
      const int seg = wave + it * WAVES;
      if (seg < NSEG) {
#pragma unroll
        for (int kk = 0; kk < KC; ++kk) {
          const unsigned long long b = __ballot(idx[it][kk] >= 0);
          if (lane == 0) s_cnt[kk][seg] = __popcll(b);
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < SEG_ITERS; ++it) {
      const int seg = wave + it * WAVES;
      if (seg < NSEG) {
#pragma unroll
        for (int kk = 0; kk < KC; ++kk) {
          const unsigned long long b = __ballot(idx[it][kk] >= 0);
          if (idx[it][kk] >= 0) {
            int slot = __popcll(b & lt_mask);
#pragma unroll
            for (int s = 0; s < NSEG; ++s)
              if (s < seg) slot += s_cnt[kk][s];
            s_row[kk][slot] = (uint8_t)(seg * 64 + lane);
            s_src[kk][slot] = idx[it][kk];
          }
        }
      }
    }
    if (wave == 0) {
      // list lengths -> flat list of blocks (offset-in-chunk << 8 | block number)
      int tot = 0;
      if (lane < kn) {
#pragma unroll
        for (int s = 0; s < NSEG; ++s) tot += s_cnt[lane][s];
      }
      if (lane < KC) s_tot[lane] = tot;
      const int nb = (tot + 15) >> 4;
      int incl = nb;
#pragma unroll
      for (int off = 1; off < 32; off <<= 1) {
        const int t = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += t;
      }
      const int first = incl - nb;
      for (int b = 0; b < nb; ++b) s_blk[first + b] = (uint16_t)((lane << 8) | b);
      if (lane == KC - 1) s_nblk = incl;
    }
    __syncthreads();
    // next chunk's map entries travel while this chunk is multiplied
    if (kc + KC < K) load_chunk(kc + KC);

    // B: blocks of 16 entries, D blocks in flight per wave.
    const int nblk = s_nblk;
    for (int i0 = 0; i0 < nblk; i0 += D) {
      int blk_kk[D], blk_left[D];
      uint32_t blk_rows[D];
      vec8 afr[D][KB];
      vec8 bfr[D][KB][NB];
#pragma unroll
      for (int d = 0; d < D; ++d) {
        blk_kk[d] = -1;
        if (i0 + d < nblk) {
          const int e = s_blk[i0 + d];
          blk_kk[d] = e >> 8;
          const int b0 = (e & 0xff) << 4;
          blk_left[d] = s_tot[blk_kk[d]] - b0;  // entries from b0 on (>= 1)
          const int slot = b0 + (lane & 15);
          int src = -1;
          if ((lane & 15) < blk_left[d]) src = s_src[blk_kk[d]][slot];
          blk_rows[d] = *reinterpret_cast<const uint32_t *>(&s_row[blk_kk[d]][b0 + 4 * (lane >> 4)]);
          const vec8 zero = {};
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            afr[d][kb] = zero;
            if (src >= 0)
              afr[d][kb] = *reinterpret_cast<const vec8 *>(A + (size_t)src * Q + kb * 32 +
                                                           (lane >> 4) * 8);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
              const size_t frag =
                  ((size_t)(kc + blk_kk[d]) * GROUPS + (grp0 + nb)) * KB + kb;
              bfr[d][kb][nb] = *reinterpret_cast<const vec8 *>(packedW + (frag * 64 + lane) * 8);
            }
          }
        }
      }
#pragma unroll
      for (int d = 0; d < D; ++d) {
        if (blk_kk[d] < 0) continue;
        float4v acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          acc[nb] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) acc[nb] = E::mfma(afr[d][kb], bfr[d][kb][nb], acc[nb]);
        }
        // lane holds result rows 4*(lane/16)+v (v = 0..3) of the block, column lane%16
        float *cell[NB][4];
        float old[NB][4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int row = (blk_rows[d] >> (8 * v)) & 0xff;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const int grp = (grp0 + nb) ^ (row & (GROUPS - 1));
            cell[nb][v] = &s_acc[row * C + grp * 16 + (lane & 15)];
          }
        }
        const int live = blk_left[d] - 4 * (lane >> 4);  // rows v < live exist
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) old[nb][v] = v < live ? *cell[nb][v] : 0.f;
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
            if (v < live) *cell[nb][v] = old[nb][v] + acc[nb][v];
        }
      }
    }
    __syncthreads();  // lists are rewritten by the next chunk
  }
  for (int i = tid; i < TR * C / 8; i += NT) {
    const int r = i / (C / 8);
    const int c8 = (i % (C / 8)) * 8;
    if (r0 + r >= R) break;
    const int grp = (c8 >> 4) ^ (r & (GROUPS - 1));
    const float *src_row = &s_acc[r * C + grp * 16 + (c8 & 15)];
    typename E::storage tmp[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) E::store(&tmp[e], src_row[e]);
    *reinterpret_cast<uint4 *>(result + (size_t)(r0 + r) * C + c8) =
        *reinterpret_cast<const uint4 *>(tmp);
  }
}

// ---- backward filter -------------------------------------------------------------
// One block = 32 x 64 tile of dW[k] over a contiguous slice of the offset's pairs.
template <typename E>
__global__ __launch_bounds__(256) void backwardFilterSimt(const typename E::storage *X,
                                                          const typename E::storage *dY,
                                                          const int32_t *pairs, int L, int n_in,
                                                          int n_out, int Ci, int Co,
                                                          OffsetCounts inl,
                                                          const int32_t *dev_counts, int splits,
                                                          float *partial,
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
  const int32_t *in_col = pairs + (size_t)k * 2 * L;
  const int32_t *out_col = in_col + L;
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
        E::store(dW + e, acc[i][j]);
      } else {
        partial[(size_t)s * K * Ci * Co + e] = acc[i][j];
      }
    }
  }
}

// dW[e] = sum over splits, in split order, rounded once.
template <typename E>
__global__ __launch_bounds__(256) void reduceFilterPartials(const float *partial, size_t n,
                                                            int splits,
                                                            typename E::storage *dW) {
  for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += (size_t)gridDim.x * 256) {
    float s = 0.f;
    for (int i = 0; i < splits; ++i) s += partial[(size_t)i * n + e];
    E::store(dW + e, s);
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

bool forceSimt() {
  const char *v = getenv("MLUOP_SPCONV_FORCE_SIMT");
  return v != nullptr && v[0] == '1';
}

bool mfmaShapeOk(ElemType t, int Q, int C) {
  if (t == ElemType::kFloat) return false;
  const bool q_ok = (Q == 32 || Q == 64 || Q == 128);
  const bool c_ok = (C == 16 || C == 32 || C == 64 || C == 128);
  return q_ok && c_ok;
}

struct GatherDims {
  int R;       // result rows
  int n_src;   // rows of the gathered tensor
  int Q;       // reduction channels
  int C;       // result channels
  int row_col, src_col;
};

GatherDims gatherDims(const ConvProblem &p, GatherDirection dir) {
  GatherDims d;
  if (dir == GatherDirection::kForward) {
    d.R = p.num_out; d.n_src = p.L; d.Q = p.Ci; d.C = p.Co; d.row_col = 1; d.src_col = 0;
  } else {
    d.R = p.L; d.n_src = p.num_out; d.Q = p.Co; d.C = p.Ci; d.row_col = 0; d.src_col = 1;
  }
  return d;
}

struct GatherWorkspace {
  int32_t *dev_counts = nullptr;
  int32_t *map = nullptr;
  void *packed = nullptr;
  size_t bytes = 0;
};

GatherWorkspace carveGather(const ConvProblem &p, const GatherDims &d, void *base) {
  GatherWorkspace ws;
  char *ptr = alignPtr(base);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char *r = ptr ? ptr + off : nullptr;
    off += alignUp(bytes);
    return r;
  };
  if (p.K > kMaxInlineK) ws.dev_counts = reinterpret_cast<int32_t *>(take((size_t)p.K * 4));
  ws.map = reinterpret_cast<int32_t *>(take((size_t)p.K * d.R * 4));
  if (mfmaShapeOk(p.dtype, d.Q, d.C))
    ws.packed = take((size_t)p.K * d.Q * d.C * elemSize(p.dtype));
  ws.bytes = off + kBaseAlign;
  return ws;
}

// Fills the by-value counts (K <= kMaxInlineK) or uploads them.  The int32
// staging vector is consumed by a synchronous-with-host pageable copy.
hipError_t prepareCounts(const LaunchCtx &lc, const ConvProblem &p, OffsetCounts *inl,
                         int32_t *dev_counts, int *max_count) {
  int mx = 0;
  for (int k = 0; k < p.K; ++k) {
    int64_t n = p.indice_num[k];
    if (n < 0) n = 0;
    if (n > p.L) n = p.L;
    if ((int)n > mx) mx = (int)n;
  }
  *max_count = mx;
  for (int k = 0; k < kMaxInlineK; ++k) inl->n[k] = 0;
  if (p.K <= kMaxInlineK) {
    for (int k = 0; k < p.K; ++k) {
      int64_t n = p.indice_num[k];
      inl->n[k] = (int)(n < 0 ? 0 : (n > p.L ? p.L : n));
    }
    return hipSuccess;
  }
  int32_t *tmp = static_cast<int32_t *>(malloc((size_t)p.K * 4));
  if (tmp == nullptr) return hipErrorOutOfMemory;
  for (int k = 0; k < p.K; ++k) {
    int64_t n = p.indice_num[k];
    tmp[k] = (int)(n < 0 ? 0 : (n > p.L ? p.L : n));
  }
  hipError_t err = hipMemcpyAsync(dev_counts, tmp, (size_t)p.K * 4, hipMemcpyHostToDevice, lc.stream);
  if (err == hipSuccess) err = hipStreamSynchronize(lc.stream);
  free(tmp);
  return err;
}

template <typename E, int Q, int C>
void launchMfmaInstance(const LaunchCtx &lc, const void *A, const void *packed,
                        const int32_t *map, int R, int K, const OffsetCounts &inl,
                        const int32_t *dev_counts, void *result) {
  constexpr int NT = 64 * (C / 16 / mfmaColBlocksPerWave(C));
  constexpr int TR = mfmaTileRows(C);
  const int blocks = (R + TR - 1) / TR;
  lc.begin("gatherConvMfma");
  gatherConvMfma<E, Q, C><<<blocks, NT, 0, lc.stream>>>(
      static_cast<const typename E::storage *>(A),
      static_cast<const typename E::storage *>(packed), map, R, K, inl, dev_counts,
      static_cast<typename E::storage *>(result));
  lc.end();
}

template <typename E, int Q>
void launchMfmaByC(const LaunchCtx &lc, int C, const void *A, const void *packed,
                   const int32_t *map, int R, int K, const OffsetCounts &inl,
                   const int32_t *dev_counts, void *result) {
  switch (C) {
    case 16: launchMfmaInstance<E, Q, 16>(lc, A, packed, map, R, K, inl, dev_counts, result); break;
    case 32: launchMfmaInstance<E, Q, 32>(lc, A, packed, map, R, K, inl, dev_counts, result); break;
    case 64: launchMfmaInstance<E, Q, 64>(lc, A, packed, map, R, K, inl, dev_counts, result); break;
    case 128: launchMfmaInstance<E, Q, 128>(lc, A, packed, map, R, K, inl, dev_counts, result); break;
    default: break;
  }
}

template <typename E>
void launchMfma(const LaunchCtx &lc, int Q, int C, const void *A, const void *packed,
                const int32_t *map, int R, int K, const OffsetCounts &inl,
                const int32_t *dev_counts, void *result) {
  switch (Q) {
    case 32: launchMfmaByC<E, 32>(lc, C, A, packed, map, R, K, inl, dev_counts, result); break;
    case 64: launchMfmaByC<E, 64>(lc, C, A, packed, map, R, K, inl, dev_counts, result); break;
    case 128: launchMfmaByC<E, 128>(lc, C, A, packed, map, R, K, inl, dev_counts, result); break;
    default: break;
  }
}

template <typename E>
void launchGatherTyped(const LaunchCtx &lc, const ConvProblem &p, const GatherDims &d,
                       const GatherWorkspace &ws, const OffsetCounts &inl, const void *gathered,
                       const FilterView &f, bool use_mfma, void *result) {
  typedef typename E::storage S;
  // B(k, q, c): forward q = ci, c = co; backward data q = co, c = ci.
  const int64_t sQ = d.row_col == 1 ? f.stride_ci : f.stride_co;
  const int64_t sC = d.row_col == 1 ? f.stride_co : f.stride_ci;
  if (use_mfma) {
    if constexpr (!std::is_same<E, FloatElem>::value) {
      const size_t frags = (size_t)p.K * (d.C / 16) * (d.Q / 32) * 64;
      lc.begin("packFilterFragments");
      packFilterFragments<E><<<gridFor(frags), 256, 0, lc.stream>>>(
          static_cast<const S *>(f.base), f.stride_k, sQ, sC, p.K, d.Q, d.C,
          static_cast<S *>(ws.packed));
      lc.end();
      launchMfma<E>(lc, d.Q, d.C, gathered, ws.packed, ws.map, d.R, p.K, inl, ws.dev_counts,
                    result);
    }
    return;
  }
  dim3 grid((d.R + 31) / 32, (d.C + 63) / 64);
  lc.begin("gatherConvSimt");
  gatherConvSimt<E><<<grid, 256, 0, lc.stream>>>(static_cast<const S *>(gathered), d.Q,
                                              static_cast<const S *>(f.base), f.stride_k, sQ, sC,
                                              ws.map, d.R, p.K, inl, ws.dev_counts, d.C,
                                              static_cast<S *>(result));
  lc.end();
}

struct FilterGradWorkspace {
  int32_t *dev_counts = nullptr;
  float *partial = nullptr;
  int splits = 1;
  size_t bytes = 0;
};

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
  if (ws.splits > 1)
    ws.partial = reinterpret_cast<float *>(take((size_t)ws.splits * p.K * p.Ci * p.Co * 4));
  ws.bytes = off + kBaseAlign;
  return ws;
}

template <typename E>
void launchFilterGradTyped(const LaunchCtx &lc, const ConvProblem &p,
                           const FilterGradWorkspace &ws, const OffsetCounts &inl,
                           const void *features, const void *output_grad, void *filters_grad) {
  typedef typename E::storage S;
  const int tiles = ((p.Ci + 31) / 32) * ((p.Co + 63) / 64);
  dim3 grid(tiles, p.K, ws.splits);
  lc.begin("backwardFilterSimt");
  backwardFilterSimt<E><<<grid, 256, 0, lc.stream>>>(
      static_cast<const S *>(features), static_cast<const S *>(output_grad), p.indice_pairs, p.L,
      p.L, p.num_out, p.Ci, p.Co, inl, ws.dev_counts, ws.splits, ws.partial,
      static_cast<S *>(filters_grad));
  lc.end();
  if (ws.splits > 1) {
    const size_t n = (size_t)p.K * p.Ci * p.Co;
    lc.begin("reduceFilterPartials");
    reduceFilterPartials<E><<<gridFor(n), 256, 0, lc.stream>>>(ws.partial, n, ws.splits,
                                                            static_cast<S *>(filters_grad));
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

  const size_t map_elems = (size_t)p.K * d.R;
  lc.begin("fillInt32");
  fillInt32<<<gridFor(map_elems), 256, 0, lc.stream>>>(ws.map, map_elems, -1);
  lc.end();
  if (max_count > 0) {
    dim3 grid((max_count + 255) / 256 > 1024 ? 1024 : (max_count + 255) / 256, p.K);
    lc.begin("scatterRowMap");
    scatterRowMap<<<grid, 256, 0, lc.stream>>>(p.indice_pairs, p.L, inl, ws.dev_counts, d.row_col,
                                            d.src_col, d.R, d.n_src, ws.map);
    lc.end();
  }
  // The MFMA kernel moves rows with 16-byte accesses.
  const bool ptr_ok =
      ((reinterpret_cast<uintptr_t>(gathered) | reinterpret_cast<uintptr_t>(result)) & 15u) == 0;
  const bool use_mfma = mfmaShapeOk(p.dtype, d.Q, d.C) && ptr_ok && !forceSimt();
  switch (p.dtype) {
    case ElemType::kHalf:
      launchGatherTyped<HalfElem>(lc, p, d, ws, inl, gathered, filters, use_mfma, result);
      break;
    case ElemType::kBFloat16:
      launchGatherTyped<BFloat16Elem>(lc, p, d, ws, inl, gathered, filters, use_mfma, result);
      break;
    case ElemType::kFloat:
      launchGatherTyped<FloatElem>(lc, p, d, ws, inl, gathered, filters, false, result);
      break;
  }
  return hipGetLastError();
}

size_t backwardFilterWorkspaceBytes(const ConvProblem &p) {
  return carveFilterGrad(p, nullptr).bytes;
}

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
