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

/* Kernel choices of the sparse convolution operators.  Where two kernels compute the same
 * result the shape decides between them; the parity tests switch each one on and off through
 * this call and compare.  value: -1 the shape decides (the default), 0 never, 1 whenever the
 * kernel can run the shape.  The choice belongs to the handle and holds until changed.  (The
 * reference selects kernels by shape only; its test-time switches are environment variables
 * of the test runner, pb_gtest/src/runtime.cpp.) */
typedef enum {
  MLUOP_EXT_KERNEL_GATHER_SIMT = 0,    /* plain SIMT kernels instead of the MFMA ones */
  MLUOP_EXT_KERNEL_DENSE_TILES = 1,    /* register-accumulating gather kernel */
  MLUOP_EXT_KERNEL_WAVE_PER_TILE = 2,  /* one-wavefront-per-tile gather kernel */
  MLUOP_EXT_KERNEL_FLAT_SLICE_SUM = 3, /* backward filter: partial tiles summed on a flat grid */
  MLUOP_EXT_KERNEL_FLAT_SCATTER = 4,   /* row maps built on a flat grid */
  MLUOP_EXT_KERNEL_SMALL_MAP_CHUNKS = 5, /* 1: row maps cover 2048 result rows at a time instead of
                                            as many as 64 MiB hold (runs the chunked path on small inputs) */
  MLUOP_EXT_KERNEL_FILTER_STORES = 6,   /* 1: backward filter transposes its operands with element-sized
                                           LDS stores also for 2-byte types of 32 to 128 channels, where
                                           transposing LDS reads are the default */
  MLUOP_EXT_KERNEL_LISTS_ON_TRUST = 7   /* forward on a rulebook of this handle whose report (were the input
                                           rows in cell order?) has not reached the host yet, as under graph
                                           capture or without any wait between the two calls.  -1: start on
                                           the pair lists and enqueue the row-map kernels behind them; the
                                           first kernel's check decides on the device which of the two do the
                                           work, the others return at once.  0: build the row map.  1: a test
                                           switch: the pair lists only; a call whose lists fail the check
                                           leaves its output as it was */
} mluOpExtKernelChoice_t;

mluOpStatus_t MLUOP_WIN_API mluOpExtSetKernelChoice(mluOpHandle_t handle,
                                                    mluOpExtKernelChoice_t which, int value);

/* Waits for the handle's queue, then reports how many launches were recorded. */
mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTimingCount(mluOpHandle_t handle, int *count);

/* Name and duration in milliseconds of recorded launch `index` (launch order).
 * The name points at a string literal owned by the library. */
mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTiming(mluOpHandle_t handle, int index,
                                                    const char **name, float *milliseconds);

/* Modes of the indice-convolution operators that the reference rejects
 * (kernels/sparse_conv/indice_convolution_forward/indice_convolution_forward.cpp:74-78,
 * indice_convolution_backward_data.cpp:129-132, indice_convolution_backward_filter.cpp:185).
 * Off by default: a fresh handle answers them with the reference's status codes.
 * With `enable` non-zero the three operators accept
 *   - inverse = 1: the sparse inverse convolution of the PyTorch sparse-convolution
 *     stacks (spconv / mmcv SparseInverseConv3d).  The operator runs the rulebook of
 *     its partner layer backwards: input-side rows (features, input_grad) are taken
 *     through pair column 1, output-side rows (features_out, output_grad) through
 *     column 0, so indice_pairs.dim[2] must equal the row count of the output-side
 *     tensor (num_act_out for the forward operator) and the filter stays
 *     W(k, ci, co) of this layer;
 *   - a filters_grad descriptor tagged NHWC / NDHWC ([Co, (kd,) kh, kw, Ci]) or
 *     NCHW / NCDHW ([Co, Ci, (kd,) kh, kw]) in mluOpIndiceConvolutionBackwardFilter,
 *     written in that layout (the reference reads the dimensions positionally as
 *     (kd,) kh, kw, Ci, Co whatever the tag says). */
mluOpStatus_t MLUOP_WIN_API mluOpExtSetSparseConvExtendedModes(mluOpHandle_t handle, int enable);

/* mluOpIndiceConvolutionForward and mluOpIndiceConvolutionBackwardData add every pair of
 * indice_pairs, as the reference does, also when several pairs of one offset name the same
 * result row (which mluOpGetIndicePairs produces for repeated input coordinates, and made-up
 * pair tensors can hold anywhere).  Finding out costs one small kernel behind every call.  A
 * caller whose coordinates are distinct (voxelized point clouds are) can promise so: with
 * `promised` non-zero that kernel is not launched, and a rulebook that breaks the promise loses
 * all but one of such pairs.  Off by default. */
mluOpStatus_t MLUOP_WIN_API mluOpExtSetDistinctPairsPromise(mluOpHandle_t handle, int promised);

/* Row maps kept across calls.  mluOpIndiceConvolutionForward and ...BackwardData turn the pair
 * lists into a [K, rows] map (partner row of every result row at every offset, or -1) on every
 * call: the reference API (mlu_op.h:10321-10448, :9625-9773) hands them nothing else to keep.
 * Layers that share a rulebook, and the forward and backward pass of each, can build the map
 * once.  No counterpart in the reference.
 *
 *   mluOpExtGetRowMapSize  bytes of a map buffer for `rows` result rows.
 *   mluOpExtBuildRowMap    fills `row_map` (device memory of that size, owned by the caller) on
 *                          the handle's queue and waits for the queue once.  `row_column` is the
 *                          pair column that names the result rows: 1 for a forward convolution
 *                          (and an inverse layer's backward data), 0 for backward data (and an
 *                          inverse layer's forward); `rows` / `source_rows` are the row counts
 *                          of the result and of the gathered tensor, the one that column 0
 *                          indexes being indice_pairs.dim[2].  `*lost_pairs` returns how many
 *                          pairs found no slot of their own (several pairs of one offset naming
 *                          one result row, or rows outside their tensors): such a map is not
 *                          recorded and cannot be used; call the operators without it.
 *                          With mluOpExtSetDistinctPairsPromise in force `lost_pairs` may be
 *                          NULL: the build then neither counts nor waits, and the promise
 *                          stands in for the verdict.
 *   mluOpExtUseRowMap      announces a recorded map for the next mluOpIndiceConvolutionForward
 *                          or ...BackwardData call on this handle, which must be given the same
 *                          indice_pairs pointer, shapes and direction the map was built for
 *                          (BAD_PARAM otherwise) and then launches neither the map kernels nor
 *                          the check for colliding pairs.  The announcement ends with that call,
 *                          whatever it returns.  The pair tensor must not have changed since the
 *                          map was built.  NULL withdraws an announcement.
 *   mluOpExtForgetRowMap   drops the record of a buffer about to be freed (NULL: all records). */
mluOpStatus_t MLUOP_WIN_API mluOpExtGetRowMapSize(const mluOpTensorDescriptor_t indice_pairs_desc,
                                                  int64_t rows, size_t *size);
mluOpStatus_t MLUOP_WIN_API mluOpExtBuildRowMap(mluOpHandle_t handle,
                                                const mluOpTensorDescriptor_t indice_pairs_desc,
                                                const void *indice_pairs, const int64_t indice_num[],
                                                int64_t rows, int64_t source_rows, int row_column,
                                                void *row_map, size_t size, int64_t *lost_pairs);
mluOpStatus_t MLUOP_WIN_API mluOpExtUseRowMap(mluOpHandle_t handle, const void *row_map);
mluOpStatus_t MLUOP_WIN_API mluOpExtForgetRowMap(mluOpHandle_t handle, const void *row_map);

/* mluOpIndiceConvolutionBackwardFilter for callers that cannot allocate device memory (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc) and therefore have
 * no workspace to hand over.  No counterpart in the reference.  Same arguments and checks as
 * mluOpIndiceConvolutionBackwardFilter (mlu_op.h), without `workspace` and `workspace_size`:
 * the partial sums live in an array of MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES that the library
 * holds on every GPU it runs on until the process ends.  The call allocates and frees nothing,
 * does not wait for the queue, follows the handle's kernel choices and is left out of its
 * per-kernel timing (which creates events).  Shapes of the matrix-core kernels (16 to 128
 * channels) whose usual number of partial tiles exceeds the array are cut into fewer, longer
 * slices: the result then agrees with the workspace entry point within the accuracy standard
 * (the additions are grouped differently), and bit for bit otherwise (up to 64 x 64 channels at
 * 27 offsets).  MLUOP_STATUS_NOT_SUPPORTED when the array is too small all the same (the generic
 * kernels' tiles at large channel counts) or with more than 128 kernel offsets.  All calls on
 * one GPU share the array:
 * calls that can overlap there (different queues, different handles) race and must be ordered
 * by the caller. */
#define MLUOP_EXT_NO_ALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
mluOpStatus_t MLUOP_WIN_API mluOpExtIndiceConvolutionBackwardFilterNoAlloc(
    mluOpHandle_t handle, const mluOpTensorDescriptor_t features_desc, const void *features,
    const mluOpTensorDescriptor_t output_grad_desc, const void *output_grad,
    const mluOpTensorDescriptor_t indice_pairs_desc, const void *indice_pairs,
    const int64_t indice_num[], const int64_t inverse, const int64_t subm,
    const mluOpTensorDescriptor_t filters_grad_desc, void *filters_grad);

#if defined(__cplusplus)
}
#endif

#endif /* MLUOP_AMD_MLU_OP_EXT_H_ */
