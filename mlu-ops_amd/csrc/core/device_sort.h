// Stable least-significant-digit radix sort of (key, 32-bit value) pairs and prefix sums of
// 32-bit counts, for the operators that group points by cell (voxelization, dynamic
// point-to-voxel scatter).  Included by their .hip files; every function enqueues kernels
// only: no memset, no copy, no wait, no allocation, so a caller may capture the launches
// into a HIP graph.
//
// One pass sorts by 8 bits of the key in three launches:
//   sortCount     a workgroup counts the digits of its tile of 1024 pairs into hist[digit][tile];
//   scanDigitRows a wave per digit turns its row of counters into exclusive prefix sums (the
//                 pairs of the digit in earlier tiles) and leaves the digit's total;
//   sortScatter   the same tiles again: a wave owns 256 consecutive pairs, takes them 64 at
//                a time in order, and a pair's place among the pairs of its digit is
//                (pairs of lower digits) + (of the digit in earlier tiles) + (in earlier waves of the tile) +
//                (in earlier chunks of the wave) + (in lower lanes of the chunk), which is what
//                keeps equal keys in their input order.
// In the scatter, lanes that hold the same digit find each other with eight ballots (one per
// bit), so a digit that nearly every key shares costs what a rare one costs; the only atomics
// are the count's integer adds in LDS.
#ifndef MLUOP_AMD_CORE_DEVICE_SORT_H_
#define MLUOP_AMD_CORE_DEVICE_SORT_H_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace mluop {
namespace device_sort {

constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kSortThreads = 256;
constexpr int kSortWaves = kSortThreads / 64;
constexpr int kSortChunks = 4;                            // chunks of 64 pairs a wave takes
constexpr int kSortWaveItems = 64 * kSortChunks;          // 256
constexpr int kSortTile = kSortWaves * kSortWaveItems;    // 1024 (1 200 000 pairs: 28.6 us a pass; 2048: 30.8; 4096: 47)
constexpr int kScanChunks = 16;                           // prefix sums: 4096 counts a workgroup
constexpr int kScanTile = kSortWaves * 64 * kScanChunks;
constexpr int kScanThreads = 1024;
static_assert(kSortThreads == kRadix, "thread d of a workgroup owns digit d");

inline size_t tilesFor(size_t n) { return (n + kSortTile - 1) / kSortTile; }

// Bytes of device memory the functions below want behind `workspace` (256-byte aligned).
inline size_t workspaceBytes(size_t n) {
  const size_t tiles = tilesFor(n) + 1;
  return ((size_t)(kRadix + 1) * (tiles + 1) * sizeof(uint32_t) + 16 + 255) / 256 * 256 + 256;
}

__device__ __forceinline__ uint32_t waveInclusiveSum(uint32_t v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t up = __shfl_up(v, d, 64);
    if (lane >= d) v += up;
  }
  return v;
}

// The lanes of the wave whose `digit` equals this lane's, among the lanes of `valid`.
__device__ __forceinline__ unsigned long long lanesWithSameDigit(uint32_t digit, bool valid) {
  unsigned long long peers = __ballot(valid);
#pragma unroll
  for (int b = 0; b < kRadixBits; ++b) {
    const bool bit = (digit >> b) & 1u;
    const unsigned long long with = __ballot(bit);
    peers &= bit ? with : ~with;
  }
  return peers;
}

template <typename K>
__global__ __launch_bounds__(kSortThreads) void sortCount(const K *__restrict__ keys, size_t n, int shift,
                                                          uint32_t *__restrict__ hist, int tiles) {
  __shared__ uint32_t s_count[kRadix];
  const int tid = threadIdx.x;
  s_count[tid] = 0;
  __syncthreads();
  const size_t base = (size_t)blockIdx.x * kSortTile;
  K key[kSortTile / kSortThreads];
#pragma unroll
  for (int j = 0; j < kSortTile / kSortThreads; ++j) {
    const size_t i = base + (size_t)j * kSortThreads + tid;
    key[j] = i < n ? keys[i] : (K)0;
  }
  // (integer adds in LDS: the order they land in does not matter for a count)
#pragma unroll
  for (int j = 0; j < kSortTile / kSortThreads; ++j)
    if (base + (size_t)j * kSortThreads + tid < n) atomicAdd(&s_count[(uint32_t)(key[j] >> shift) & (kRadix - 1)], 1u);
  __syncthreads();
  hist[(size_t)tid * tiles + blockIdx.x] = s_count[tid];
}

// data[0..m) -> exclusive prefix sums in place, by one workgroup, in rounds of 16 counters a
// thread (four 16-byte loads in flight); `data` is 16-byte aligned and has room for m rounded
// up to a multiple of four.
constexpr int kScanPerThread = 16;
static __global__ __launch_bounds__(kScanThreads) void scanCounters(uint32_t *data, size_t m) {
  __shared__ uint32_t s_wave[kScanThreads / 64];
  __shared__ uint32_t s_round_total;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t carry = 0;
  for (size_t round0 = 0; round0 < m; round0 += (size_t)kScanThreads * kScanPerThread) {
    const size_t begin = round0 + (size_t)tid * kScanPerThread;
    uint4 q[kScanPerThread / 4];
#pragma unroll
    for (int u = 0; u < kScanPerThread / 4; ++u) {
      const size_t i = begin + 4 * u;
      q[u] = i < m ? *reinterpret_cast<const uint4 *>(data + i) : make_uint4(0, 0, 0, 0);
      // (the words of a last, partial group that lie past m count as zero)
      if (i + 1 >= m) q[u].y = 0;
      if (i + 2 >= m) q[u].z = 0;
      if (i + 3 >= m) q[u].w = 0;
    }
    uint32_t sum = 0;
#pragma unroll
    for (int u = 0; u < kScanPerThread / 4; ++u) sum += q[u].x + q[u].y + q[u].z + q[u].w;
    const uint32_t incl = waveInclusiveSum(sum);
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    if (wave == 0) {
      const uint32_t w = lane < kScanThreads / 64 ? s_wave[lane] : 0;
      const uint32_t wi = waveInclusiveSum(w);
      if (lane < kScanThreads / 64) s_wave[lane] = wi - w;
      if (lane == 63) s_round_total = wi;
    }
    __syncthreads();
    uint32_t run = carry + s_wave[wave] + incl - sum;
#pragma unroll
    for (int u = 0; u < kScanPerThread / 4; ++u) {
      const size_t i = begin + 4 * u;
      uint4 o;
      o.x = run; run += q[u].x;
      o.y = run; run += q[u].y;
      o.z = run; run += q[u].z;
      o.w = run; run += q[u].w;
      if (i < m) *reinterpret_cast<uint4 *>(data + i) = o;
    }
    carry += s_round_total;
    __syncthreads();
  }
}

// hist[digit][0..tiles) -> exclusive prefix sums along the row, one wave per digit; the row's
// total goes to totals[digit].
static __global__ __launch_bounds__(64) void scanDigitRows(uint32_t *hist, int tiles, uint32_t *totals) {
  const int lane = threadIdx.x;
  uint32_t *row = hist + (size_t)blockIdx.x * tiles;
  uint32_t carry = 0;
  for (int t0 = 0; t0 < tiles; t0 += 64 * 8) {
    // lane l: eight consecutive counters
    uint32_t v[8];
    uint32_t sum = 0;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = t0 + lane * 8 + u;
      v[u] = t < tiles ? row[t] : 0u;
      sum += v[u];
    }
    const uint32_t incl = waveInclusiveSum(sum);
    uint32_t run = carry + incl - sum;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = t0 + lane * 8 + u;
      if (t < tiles) row[t] = run;
      run += v[u];
    }
    carry += __shfl(incl, 63, 64);
  }
  if (lane == 0) totals[blockIdx.x] = carry;
}

// (VALUES false: keys only; a caller whose value fits beside its key in 64 bits sorts the
// packed words as keys and halves the scattered stores)
template <typename K, bool VALUES>
__global__ __launch_bounds__(kSortThreads) void sortScatter(const K *__restrict__ keys_in,
                                                            const uint32_t *__restrict__ vals_in,
                                                            K *__restrict__ keys_out,
                                                            uint32_t *__restrict__ vals_out, size_t n, int shift,
                                                            const uint32_t *__restrict__ hist, int tiles,
                                                            const uint32_t *__restrict__ totals) {
  __shared__ uint32_t s_count[kSortWaves][kRadix];  // pairs of a digit per wave, then in the waves before
  __shared__ uint32_t s_first[kRadix];              // where the tile's first pair of a digit goes
  __shared__ uint32_t s_wave_total[kSortWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kSortWaves * kRadix; i += kSortThreads) (&s_count[0][0])[i] = 0;
  __syncthreads();
  const size_t base = (size_t)blockIdx.x * kSortTile + (size_t)wave * kSortWaveItems;
  K key[kSortChunks];
  uint32_t val[kSortChunks], place[kSortChunks];
#pragma unroll
  for (int j = 0; j < kSortChunks; ++j) {
    const size_t i = base + (size_t)j * 64 + lane;
    key[j] = i < n ? keys_in[i] : (K)0;
    val[j] = (VALUES && i < n) ? vals_in[i] : 0u;
  }
  volatile uint32_t *mine = s_count[wave];
  const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
  for (int j = 0; j < kSortChunks; ++j) {
    const bool valid = base + (size_t)j * 64 + lane < n;
    const uint32_t digit = (uint32_t)(key[j] >> shift) & (kRadix - 1);
    const unsigned long long peers = lanesWithSameDigit(digit, valid);
    const int leader = valid ? __ffsll((long long)peers) - 1 : lane;
    uint32_t before = 0;  // pairs of the digit in the wave's earlier chunks
    if (valid && lane == leader) {
      before = mine[digit];
      mine[digit] = before + (uint32_t)__popcll(peers);
    }
    before = __shfl(before, leader, 64);
    place[j] = before + (uint32_t)__popcll(peers & below);
  }
  __syncthreads();
  {
    // thread d: the waves' counts of digit d become the counts of the waves before
    uint32_t run = 0;
#pragma unroll
    for (int w = 0; w < kSortWaves; ++w) {
      const uint32_t c = s_count[w][tid];
      s_count[w][tid] = run;
      run += c;
    }
    // pairs of lower digits in all tiles + pairs of this digit in earlier tiles
    const uint32_t all = totals[tid];
    const uint32_t incl = waveInclusiveSum(all);
    if (lane == 63) s_wave_total[wave] = incl;
    __syncthreads();
    uint32_t lower = incl - all;
    for (int w = 0; w < wave; ++w) lower += s_wave_total[w];
    s_first[tid] = lower + hist[(size_t)tid * tiles + blockIdx.x];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < kSortChunks; ++j) {
    if (base + (size_t)j * 64 + lane < n) {
      const uint32_t digit = (uint32_t)(key[j] >> shift) & (kRadix - 1);
      const size_t to = (size_t)s_first[digit] + s_count[wave][digit] + place[j];
      keys_out[to] = key[j];
      if (VALUES) vals_out[to] = val[j];
    }
  }
}

// Sorts the n pairs (keys_a[i], vals_a[i]) by the lowest `bits` bits of the key, equal keys
// in input order.  Both pairs of arrays are written; *in_b tells which holds the result
// (true: keys_b / vals_b).  vals_a == nullptr: keys only.  `workspace`: workspaceBytes(n) bytes.
template <typename K>
hipError_t sortPairs(hipStream_t stream, void *workspace, K *keys_a, K *keys_b, uint32_t *vals_a,
                     uint32_t *vals_b, size_t n, int bits, bool *in_b) {
  *in_b = false;
  if (n == 0 || bits <= 0) return hipSuccess;
  const int tiles = (int)tilesFor(n);
  uint32_t *totals = reinterpret_cast<uint32_t *>((reinterpret_cast<uintptr_t>(workspace) + 255) / 256 * 256);
  uint32_t *hist = totals + kRadix;
  K *kin = keys_a, *kout = keys_b;
  uint32_t *vin = vals_a, *vout = vals_b;
  for (int shift = 0; shift < bits; shift += kRadixBits) {
    sortCount<K><<<tiles, kSortThreads, 0, stream>>>(kin, n, shift, hist, tiles);
    scanDigitRows<<<kRadix, 64, 0, stream>>>(hist, tiles, totals);
    if (vals_a != nullptr)
      sortScatter<K, true><<<tiles, kSortThreads, 0, stream>>>(kin, vin, kout, vout, n, shift, hist, tiles, totals);
    else
      sortScatter<K, false><<<tiles, kSortThreads, 0, stream>>>(kin, nullptr, kout, nullptr, n, shift, hist, tiles,
                                                                totals);
    K *tk = kin;
    kin = kout;
    kout = tk;
    uint32_t *tv = vin;
    vin = vout;
    vout = tv;
    *in_b = !*in_b;
  }
  return hipGetLastError();
}

// Keys only.
template <typename K>
hipError_t sortKeys(hipStream_t stream, void *workspace, K *keys_a, K *keys_b, size_t n, int bits, bool *in_b) {
  return sortPairs<K>(stream, workspace, keys_a, keys_b, nullptr, nullptr, n, bits, in_b);
}

// ---- prefix sums over n counts --------------------------------------------------------

// (BITS: the counts are the numbers of set bits of the words of `in`)
template <bool BITS>
__global__ __launch_bounds__(kSortThreads) void scanTileSums(const uint32_t *__restrict__ in, size_t n,
                                                             uint32_t *__restrict__ sums) {
  __shared__ uint32_t s_wave[kSortWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t base = (size_t)blockIdx.x * kScanTile;
  uint32_t sum = 0;
#pragma unroll
  for (int j = 0; j < kScanTile / kSortThreads; ++j) {
    const size_t i = base + (size_t)j * kSortThreads + tid;
    const uint32_t word = i < n ? in[i] : 0u;
    sum += BITS ? (uint32_t)__popc(word) : word;
  }
  const uint32_t incl = waveInclusiveSum(sum);
  if (lane == 63) s_wave[wave] = incl;
  __syncthreads();
  if (tid == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kSortWaves; ++w) t += s_wave[w];
    sums[blockIdx.x] = t;
  }
}

template <bool INCLUSIVE, bool BITS>
__global__ __launch_bounds__(kSortThreads) void scanTiles(const uint32_t *__restrict__ in,
                                                          uint32_t *__restrict__ out, size_t n,
                                                          const uint32_t *__restrict__ tile_first) {
  __shared__ uint32_t s_wave[kSortWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t base = (size_t)blockIdx.x * kScanTile + (size_t)wave * (64 * kScanChunks);
  uint32_t v[kScanChunks];
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kScanChunks; ++j) {
    const size_t i = base + (size_t)j * 64 + lane;
    const uint32_t word = i < n ? in[i] : 0u;
    v[j] = BITS ? (uint32_t)__popc(word) : word;
    mine += v[j];
  }
  // the wave's total, then the waves before it
  uint32_t wave_total = mine;
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) wave_total += __shfl_xor(wave_total, d, 64);
  if (lane == 0) s_wave[wave] = wave_total;
  __syncthreads();
  uint32_t run = tile_first[blockIdx.x];
  for (int w = 0; w < wave; ++w) run += s_wave[w];
#pragma unroll
  for (int j = 0; j < kScanChunks; ++j) {
    const size_t i = base + (size_t)j * 64 + lane;
    const uint32_t incl = waveInclusiveSum(v[j]);
    if (i < n) out[i] = run + (INCLUSIVE ? incl : incl - v[j]);
    run += __shfl(incl, 63, 64);
  }
}

// out[i] = c[0] + ... + c[i] (inclusive) or without c[i] (exclusive), where c[i] = in[i], or
// the number of set bits of in[i] with `count_bits`.  `workspace` as above.
inline hipError_t prefixSums(hipStream_t stream, void *workspace, const uint32_t *in, uint32_t *out,
                             size_t n, bool inclusive, bool count_bits = false) {
  if (n == 0) return hipSuccess;
  const int tiles = (int)((n + kScanTile - 1) / kScanTile);
  uint32_t *sums = reinterpret_cast<uint32_t *>((reinterpret_cast<uintptr_t>(workspace) + 255) / 256 * 256);
  if (count_bits)
    scanTileSums<true><<<tiles, kSortThreads, 0, stream>>>(in, n, sums);
  else
    scanTileSums<false><<<tiles, kSortThreads, 0, stream>>>(in, n, sums);
  scanCounters<<<1, kScanThreads, 0, stream>>>(sums, (size_t)tiles);
  if (count_bits) {
    if (inclusive)
      scanTiles<true, true><<<tiles, kSortThreads, 0, stream>>>(in, out, n, sums);
    else
      scanTiles<false, true><<<tiles, kSortThreads, 0, stream>>>(in, out, n, sums);
  } else {
    if (inclusive)
      scanTiles<true, false><<<tiles, kSortThreads, 0, stream>>>(in, out, n, sums);
    else
      scanTiles<false, false><<<tiles, kSortThreads, 0, stream>>>(in, out, n, sums);
  }
  return hipGetLastError();
}

}  // namespace device_sort
}  // namespace mluop

#endif  // MLUOP_AMD_CORE_DEVICE_SORT_H_
