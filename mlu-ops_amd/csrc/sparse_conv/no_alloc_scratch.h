// The library-held scratch memory behind mluOpExtIndiceConvolutionBackwardFilterNoAlloc.
#ifndef MLUOP_AMD_SPARSE_CONV_NO_ALLOC_SCRATCH_H_
#define MLUOP_AMD_SPARSE_CONV_NO_ALLOC_SCRATCH_H_

#include <hip/hip_runtime_api.h>

namespace mluop {
namespace sparse_conv {

// Looks up the address of the scratch array on `device`, which must be the current device,
// and keeps it.  Called once per device when a handle is created; later calls return at once.
hipError_t lookUpNoAllocScratch(int device);

}  // namespace sparse_conv
}  // namespace mluop

#endif  // MLUOP_AMD_SPARSE_CONV_NO_ALLOC_SCRATCH_H_
