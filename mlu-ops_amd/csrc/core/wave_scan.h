// Inclusive prefix sum over the 64 lanes of a wavefront with DPP moves: four
// shifts inside each row of 16 lanes, then lane 15 of rows 0 and 2 is added to
// rows 1 and 3, and lane 31 to rows 2 and 3.  Six dependent VALU operations
// instead of six LDS-crossbar shuffles.  All 64 lanes must be active.
#ifndef MLUOP_AMD_CORE_WAVE_SCAN_H_
#define MLUOP_AMD_CORE_WAVE_SCAN_H_

#include <hip/hip_runtime.h>

#include <cstdint>

namespace mluop {

__device__ __forceinline__ int waveInclusiveScan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2, 3
  return v;
}

// Inclusive running maximum (unsigned) over the lanes, same moves.
__device__ __forceinline__ uint32_t waveInclusiveMax(uint32_t v) {
  auto step = [](uint32_t x, uint32_t from) { return x > from ? x : from; };
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false));
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false));
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false));
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false));
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false));
  v = step(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false));
  return v;
}

// Inclusive OR over runs of lanes with equal `key` (keys must not decrease from lane to
// lane, and no key is 0xffffffff): afterwards the last lane of a run holds the OR of the
// whole run's (lo, hi).  Same moves; a lane takes the other lane's value when its key is
// the same.
__device__ __forceinline__ void waveRunInclusiveOr(uint32_t key, uint32_t *lo, uint32_t *hi) {
#define MLUOP_RUN_OR_STEP(ctrl, rows)                                                          \
  {                                                                                            \
    const uint32_t k_from = (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)key, ctrl, rows, 0xf, false); \
    const uint32_t lo_from = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)*lo, ctrl, rows, 0xf, false); \
    const uint32_t hi_from = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)*hi, ctrl, rows, 0xf, false); \
    if (k_from == key) {                                                                       \
      *lo |= lo_from;                                                                          \
      *hi |= hi_from;                                                                          \
    }                                                                                          \
  }
  MLUOP_RUN_OR_STEP(0x111, 0xf)
  MLUOP_RUN_OR_STEP(0x112, 0xf)
  MLUOP_RUN_OR_STEP(0x114, 0xf)
  MLUOP_RUN_OR_STEP(0x118, 0xf)
  MLUOP_RUN_OR_STEP(0x142, 0xa)
  MLUOP_RUN_OR_STEP(0x143, 0xc)
#undef MLUOP_RUN_OR_STEP
}

}  // namespace mluop

#endif  // MLUOP_AMD_CORE_WAVE_SCAN_H_
