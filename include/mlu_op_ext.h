/*
 * mlu_op_ext.h -- small extensions of the MI355X library that the reference
 * API does not have.  Nothing here is needed to use the operators.
 */
#ifndef MLUOP_AMD_MLU_OP_EXT_H_
#define MLUOP_AMD_MLU_OP_EXT_H_

#include "mlu_op.h"

#if defined(__cplusplus)
extern "C" {
#endif

/* Per-kernel device timing.  The reference offers kernel tracing through
 * environment switches that wrap every kernel invocation
 * (core/kernel_tracing.cpp:41-120, core/mlu_op_trace.cpp:50-100); here the
 * handle records a HIP event pair around every kernel it enqueues while timing
 * is enabled.  Enabling (or re-enabling) clears earlier records.  Recording
 * costs two event records per launch, so leave it off in production. */
mluOpStatus_t MLUOP_WIN_API mluOpExtSetKernelTiming(mluOpHandle_t handle, int enable);

/* Waits for the handle's queue, then reports how many launches were recorded. */
mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTimingCount(mluOpHandle_t handle, int *count);

/* Name and duration in milliseconds of recorded launch `index` (launch order).
 * The name points at a string literal owned by the library. */
mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTiming(mluOpHandle_t handle, int index,
                                                    const char **name, float *milliseconds);

#if defined(__cplusplus)
}
#endif

#endif /* MLUOP_AMD_MLU_OP_EXT_H_ */
