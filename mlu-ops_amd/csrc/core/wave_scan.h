// Inclusive prefix sum over the 64 lanes of a wavefront with DPP moves: four
// shifts inside each row of 16 lanes, then lane 15 of rows 0 and 2 is added to
// rows 1 and 3, and lane 31 to rows 2 and 3.  Six dependent VALU operations
// instead of six LDS-crossbar shuffles.  All 64 lanes must be active.
#ifndef MLUOP_AMD_CORE_WAVE_SCAN_H_
#define MLUOP_AMD_CORE_WAVE_SCAN_H_

#include <hip/hip_runtime.h>

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

}  // namespace mluop

#endif  // MLUOP_AMD_CORE_WAVE_SCAN_H_
