/*
 * mlu_op.h -- C ABI of the MI355X-native sparse-convolution library.
 *
 * This header declares the subset of the Cambricon mlu-ops public API
 * (reference: mlu_op.h, v1.11.1) that the sparse_conv path needs: handle,
 * tensor descriptor, sparse-convolution descriptor, rulebook construction
 * (mluOpGetIndicePairs) and the three indice-convolution operators with their
 * workspace queries.  Enum values, argument order and argument meaning are
 * those of the reference, so a caller compiled against the reference header
 * links against this library unchanged, with one substitution:
 * the queue type `cnrtQueue_t` is a `hipStream_t` here (both are opaque
 * pointers; the typedef below keeps the header free of HIP includes).
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, returns a
 * status code and never throws.
 */
#ifndef MLUOP_AMD_MLU_OP_H_
#define MLUOP_AMD_MLU_OP_H_

/* reference mlu_op.h:30-39 */
#define MLUOP_MAJOR 1
#define MLUOP_MINOR 11
#define MLUOP_PATCHLEVEL 1
#define MLUOP_VERSION (MLUOP_MAJOR * 1000 + MLUOP_MINOR * 100 + MLUOP_PATCHLEVEL)
#define MLUOP_DIM_MAX 8

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifndef MLUOP_WIN_API
#define MLUOP_WIN_API
#endif

#if defined(__cplusplus)
extern "C" {
#endif

/* reference mlu_op.h:63-94 */
typedef enum {
  MLUOP_STATUS_SUCCESS            = 0,
  MLUOP_STATUS_NOT_INITIALIZED    = 1,
  MLUOP_STATUS_ALLOC_FAILED       = 2,
  MLUOP_STATUS_BAD_PARAM          = 3,
  MLUOP_STATUS_INTERNAL_ERROR     = 4,
  MLUOP_STATUS_ARCH_MISMATCH      = 5,
  MLUOP_STATUS_EXECUTION_FAILED   = 6,
  MLUOP_STATUS_NOT_SUPPORTED      = 7,
  MLUOP_STATUS_NUMERICAL_OVERFLOW = 8,
} mluOpStatus_t;

/* reference mlu_op.h:115-140 */
typedef enum {
  MLUOP_LAYOUT_NCHW  = 0,
  MLUOP_LAYOUT_NHWC  = 1,
  MLUOP_LAYOUT_HWCN  = 2,
  MLUOP_LAYOUT_NDHWC = 3,
  MLUOP_LAYOUT_ARRAY = 4,
  MLUOP_LAYOUT_NCDHW = 5,
  MLUOP_LAYOUT_TNC   = 6,
  MLUOP_LAYOUT_NTC   = 7,
  MLUOP_LAYOUT_NC    = 8,
  MLUOP_LAYOUT_NLC   = 9,
  MLUOP_LAYOUT_NCL   = 10,
} mluOpTensorLayout_t;

/* reference mlu_op.h:169-189 */
typedef enum {
  MLUOP_DTYPE_INVALID       = 0,
  MLUOP_DTYPE_HALF          = 1,
  MLUOP_DTYPE_FLOAT         = 2,
  MLUOP_DTYPE_DOUBLE        = 14,
  MLUOP_DTYPE_INT8          = 3,
  MLUOP_DTYPE_INT16         = 4,
  MLUOP_DTYPE_INT31         = 5,
  MLUOP_DTYPE_INT32         = 6,
  MLUOP_DTYPE_INT64         = 9,
  MLUOP_DTYPE_UINT8         = 7,
  MLUOP_DTYPE_UINT16        = 13,
  MLUOP_DTYPE_UINT32        = 11,
  MLUOP_DTYPE_UINT64        = 12,
  MLUOP_DTYPE_BOOL          = 8,
  MLUOP_DTYPE_COMPLEX_HALF  = 15,
  MLUOP_DTYPE_COMPLEX_FLOAT = 16,
  MLUOP_DTYPE_BFLOAT16      = 17,
} mluOpDataType_t;

/* reference mlu_op.h:215-220 */
typedef enum {
  MLUOP_ATOMICS_NOT_ALLOWED = 1,
  MLUOP_ATOMICS_ALLOWED     = 2,
} mluOpAtomicsMode_t;

/* reference mlu_op.h:225-235 */
typedef enum {
  MLUOP_ROUND_HALF_TO_EVEN  = 0,
  MLUOP_ROUND_HALF_UP       = 1,
  MLUOP_ROUND_HALF_OFF_ZERO = 2,
} mluOpQuantizeRoundMode_t;

/* reference mlu_op.h:260-266 */
typedef enum {
  MLUOP_POINTER_MODE_HOST   = 0,
  MLUOP_POINTER_MODE_DEVICE = 1,
} mluOpPointerMode_t;

/* Opaque objects (reference mlu_op.h:404, :889, :1161). */
typedef struct mluOpContext *mluOpHandle_t;
typedef struct mluOpTensorStruct *mluOpTensorDescriptor_t;
typedef struct mluOpSparseConvolutionStruct *mluOpSparseConvolutionDescriptor_t;

/* The reference's cnrtQueue_t; on this platform the queue is a hipStream_t. */
typedef struct ihipStream_t *mluOpQueue_t;

/* ------------------------------------------------------------------------
 * Runtime management (reference mlu_op.h:455-874, core/context.cpp:158-380)
 * ---------------------------------------------------------------------- */

/* Binds a new handle to the calling thread's current HIP device.  The queue
 * starts as the NULL (default) stream; attach one with mluOpSetQueue.
 * Replaces reference mlu_op.h:455-456. */
mluOpStatus_t MLUOP_WIN_API mluOpCreate(mluOpHandle_t *handle);
/* reference mlu_op.h:529-530 */
mluOpStatus_t MLUOP_WIN_API mluOpDestroy(mluOpHandle_t handle);
/* reference mlu_op.h:570-571; queue may be NULL. */
mluOpStatus_t MLUOP_WIN_API mluOpSetQueue(mluOpHandle_t handle, mluOpQueue_t queue);
/* reference mlu_op.h:607-608 */
mluOpStatus_t MLUOP_WIN_API mluOpGetQueue(mluOpHandle_t handle, mluOpQueue_t *queue);
/* reference mlu_op.h:646; returns the enumerator's name. */
const char *MLUOP_WIN_API mluOpGetErrorString(mluOpStatus_t status);
/* reference mlu_op.h:681-682 */
mluOpStatus_t MLUOP_WIN_API mluOpGetSizeOfDataType(mluOpDataType_t data_type, size_t *size);
/* reference mlu_op.h:722 */
void MLUOP_WIN_API mluOpGetLibVersion(int *major, int *minor, int *patch);
/* reference mlu_op.h:760-798 */
mluOpStatus_t MLUOP_WIN_API mluOpSetQuantizeRoundMode(mluOpHandle_t handle,
                                                      mluOpQuantizeRoundMode_t round_mode);
mluOpStatus_t MLUOP_WIN_API mluOpGetQuantizeRoundMode(mluOpHandle_t handle,
                                                      mluOpQuantizeRoundMode_t *round_mode);
/* reference mlu_op.h:836-874; default is MLUOP_ATOMICS_NOT_ALLOWED. */
mluOpStatus_t MLUOP_WIN_API mluOpSetAtomicsMode(mluOpHandle_t handle,
                                                mluOpAtomicsMode_t atomics_mode);
mluOpStatus_t MLUOP_WIN_API mluOpGetAtomicsMode(mluOpHandle_t handle,
                                                mluOpAtomicsMode_t *atomics_mode);

/* ------------------------------------------------------------------------
 * Tensor descriptor (reference mlu_op.h:1232-2573, core/tensor.cpp:559-857)
 * ---------------------------------------------------------------------- */
/* reference mlu_op.h:1232-1233 */
mluOpStatus_t MLUOP_WIN_API mluOpCreateTensorDescriptor(mluOpTensorDescriptor_t *desc);
/* reference mlu_op.h:1405-1407 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptor(mluOpTensorDescriptor_t desc,
                                                     mluOpTensorLayout_t layout,
                                                     mluOpDataType_t dtype,
                                                     int dimNb,
                                                     const int dimSize[]);
/* reference mlu_op.h:1510-1515 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptor_v2(mluOpTensorDescriptor_t desc,
                                                        mluOpTensorLayout_t layout,
                                                        mluOpDataType_t dtype,
                                                        int dimNb,
                                                        const int64_t dimSize[]);
/* reference mlu_op.h:1814-1820 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorEx(mluOpTensorDescriptor_t desc,
                                                       mluOpTensorLayout_t layout,
                                                       mluOpDataType_t dtype,
                                                       int dimNb,
                                                       const int dimSize[],
                                                       const int dimStride[]);
/* reference mlu_op.h:1873-1879 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorEx_v2(mluOpTensorDescriptor_t desc,
                                                          mluOpTensorLayout_t layout,
                                                          mluOpDataType_t dtype,
                                                          int dimNb,
                                                          const int64_t dimSize[],
                                                          const int64_t dimStride[]);
/* reference mlu_op.h:1431-1458 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorPointerMode(mluOpTensorDescriptor_t desc,
                                                                mluOpPointerMode_t pointer_mode);
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorPointerMode(mluOpTensorDescriptor_t desc,
                                                                mluOpPointerMode_t *pointer_mode);
/* reference mlu_op.h:2008-2009 */
mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorOnchipDataType(mluOpTensorDescriptor_t desc,
                                                                   mluOpDataType_t onchip_dtype);
/* reference mlu_op.h:2417-2418 */
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorOnchipDataType(
    const mluOpTensorDescriptor_t desc, mluOpDataType_t *onchip_dtype);
/* reference mlu_op.h:2172-2174 */
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptor(const mluOpTensorDescriptor_t desc,
                                                     mluOpTensorLayout_t *layout,
                                                     mluOpDataType_t *dtype,
                                                     int *dimNb,
                                                     int dimSize[]);
/* reference mlu_op.h:2220-2225 */
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptor_v2(const mluOpTensorDescriptor_t desc,
                                                        mluOpTensorLayout_t *layout,
                                                        mluOpDataType_t *dtype,
                                                        int *dimNb,
                                                        int64_t dimSize[]);
/* reference mlu_op.h:2273-2279 */
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorEx(const mluOpTensorDescriptor_t desc,
                                                       mluOpTensorLayout_t *layout,
                                                       mluOpDataType_t *dtype,
                                                       int *dimNb,
                                                       int dimSize[],
                                                       int dimStride[]);
/* reference mlu_op.h:2327-2333 */
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorEx_v2(const mluOpTensorDescriptor_t desc,
                                                          mluOpTensorLayout_t *layout,
                                                          mluOpDataType_t *dtype,
                                                          int *dimNb,
                                                          int64_t dimSize[],
                                                          int64_t dimStride[]);
/* reference mlu_op.h:2376-2377 */
size_t MLUOP_WIN_API mluOpGetTensorElementNum(const mluOpTensorDescriptor_t desc);
/* reference mlu_op.h:1760-1761 */
mluOpStatus_t MLUOP_WIN_API mluOpResetTensorDescriptor(mluOpTensorDescriptor_t desc);
/* reference mlu_op.h:2572-2573 */
mluOpStatus_t MLUOP_WIN_API mluOpDestroyTensorDescriptor(mluOpTensorDescriptor_t desc);

/* ------------------------------------------------------------------------
 * Sparse-convolution descriptor
 * (reference mlu_op.h:1271-1311, :1606-1654; get_indice_pairs_structs.cpp:31-134)
 * ---------------------------------------------------------------------- */
/* reference mlu_op.h:1271-1272; NULL -> NOT_INITIALIZED. */
mluOpStatus_t MLUOP_WIN_API
mluOpCreateSparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t *desc);
/* reference mlu_op.h:1310-1311; NULL -> EXECUTION_FAILED. */
mluOpStatus_t MLUOP_WIN_API
mluOpDestroySparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t desc);
/* reference mlu_op.h:1606-1618.  dimNb must be 5; pad/stride/dilation and the
 * three spaces have dimNb-2 entries in (d, h, w) order; output_space is given
 * by the caller, never derived; transpose and inverse must be 0. */
mluOpStatus_t MLUOP_WIN_API
mluOpSetSparseConvolutionDescriptor(mluOpSparseConvolutionDescriptor_t desc,
                                    int dimNb,
                                    int batch_size,
                                    const int pad[],
                                    const int stride[],
                                    const int dilation[],
                                    const int input_space[],
                                    const int filter_space[],
                                    const int output_space[],
                                    const int sub_m,
                                    const int transpose,
                                    const int inverse);
/* reference mlu_op.h:1653-1654.  Written by mluOpGetIndicePairs in regular
 * (sub_m == 0) mode only; submanifold callers use the input row count. */
mluOpStatus_t MLUOP_WIN_API
mluOpGetSparseConvolutionNumActOut(mluOpSparseConvolutionDescriptor_t desc, int *num_act_out);

/* ------------------------------------------------------------------------
 * Rulebook construction (reference mlu_op.h:8597-8680,
 * kernels/sparse_conv/get_indice_pairs/get_indice_pairs.cpp:237-277)
 *
 *   indices      [L, 4]    int32 device, rows (n, d, h, w)
 *   indice_pairs [K, 2, L] int32 device, [k,0,:] input row, [k,1,:] output
 *                          row, ascending input row inside an offset, tail -1
 *   out_indices  [M, 4]    int32 device, rows >= num_act_out are -1
 *   indice_num   [K]       int32 device
 * All work is enqueued on the handle's queue.  In regular mode the call also
 * waits for the queue once, to return num_act_out through the descriptor.
 * ---------------------------------------------------------------------- */
mluOpStatus_t MLUOP_WIN_API
mluOpGetIndicePairs(mluOpHandle_t handle,
                    const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
                    const mluOpTensorDescriptor_t indices_desc,
                    const void *indices,
                    void *workspace,
                    const size_t workspace_size,
                    const mluOpTensorDescriptor_t indice_pairs_desc,
                    void *indice_pairs,
                    const mluOpTensorDescriptor_t out_indices_desc,
                    void *out_indices,
                    const mluOpTensorDescriptor_t indice_num_desc,
                    void *indice_num);

/* reference mlu_op.h:8673-8680 */
mluOpStatus_t MLUOP_WIN_API
mluOpGetIndicePairsWorkspaceSize(mluOpHandle_t handle,
                                 const mluOpSparseConvolutionDescriptor_t sparse_conv_desc,
                                 const mluOpTensorDescriptor_t indices_desc,
                                 const mluOpTensorDescriptor_t indice_pairs_desc,
                                 const mluOpTensorDescriptor_t out_indices_desc,
                                 const mluOpTensorDescriptor_t indice_num_desc,
                                 size_t *workspace_size);

/* ------------------------------------------------------------------------
 * Indice convolution forward (reference mlu_op.h:10321-10448,
 * kernels/sparse_conv/indice_convolution_forward/indice_convolution_forward.cpp:581-686)
 *
 *   features     [L, Ci]       device, half / float / bfloat16
 *   filters      5-D           device, NDHWC [Co,kd,kh,kw,Ci], NCDHW
 *                              [Co,Ci,kd,kh,kw] or ARRAY [kd,kh,kw,Ci,Co]
 *   indice_pairs [K, 2, L]     int32 device
 *   indice_num   [K]           int64 HOST array
 *   features_out [num_act_out, Co]
 * bfloat16 is an extension; the reference accepts half and float only.
 * ---------------------------------------------------------------------- */
mluOpStatus_t MLUOP_WIN_API
mluOpGetIndiceConvolutionForwardWorkspaceSize(mluOpHandle_t handle,
                                              const mluOpTensorDescriptor_t features_desc,
                                              const mluOpTensorDescriptor_t filters_desc,
                                              const mluOpTensorDescriptor_t indice_pairs_desc,
                                              const mluOpTensorDescriptor_t features_out_desc,
                                              const int64_t indice_num[],
                                              const int64_t num_act_out,
                                              const int64_t inverse,
                                              const int64_t sub_m,
                                              size_t *workspace_size);

mluOpStatus_t MLUOP_WIN_API
mluOpIndiceConvolutionForward(mluOpHandle_t handle,
                              const mluOpTensorDescriptor_t features_desc,
                              const void *features,
                              const mluOpTensorDescriptor_t filters_desc,
                              const void *filters,
                              const mluOpTensorDescriptor_t indice_pairs_desc,
                              const void *indice_pairs,
                              const int64_t indice_num[],
                              const int64_t num_act_out,
                              const int64_t inverse,
                              const int64_t sub_m,
                              void *workspace,
                              size_t workspace_size,
                              const mluOpTensorDescriptor_t features_out_desc,
                              void *features_out);

/* ------------------------------------------------------------------------
 * Indice convolution backward data (reference mlu_op.h:9625-9773,
 * kernels/sparse_conv/indice_convolution_backward_data/
 * indice_convolution_backward_data.cpp:358-959)
 *
 *   output_grad [num_act_out, Co], filters 4-D or 5-D (NHWC, NCHW, HWCN,
 *   NDHWC, NCDHW, ARRAY = (kd,)kh,kw,Ci,Co), input_grad [L, Ci].
 * ---------------------------------------------------------------------- */
mluOpStatus_t MLUOP_WIN_API
mluOpGetIndiceConvolutionBackwardDataWorkspaceSize(mluOpHandle_t handle,
                                                   const mluOpTensorDescriptor_t output_grad_desc,
                                                   const mluOpTensorDescriptor_t filters_desc,
                                                   const mluOpTensorDescriptor_t indice_pairs_desc,
                                                   const mluOpTensorDescriptor_t input_grad_desc,
                                                   const int64_t indice_num[],
                                                   const int64_t inverse,
                                                   size_t *workspace_size);

mluOpStatus_t MLUOP_WIN_API
mluOpIndiceConvolutionBackwardData(mluOpHandle_t handle,
                                   const mluOpTensorDescriptor_t output_grad_desc,
                                   const void *output_grad,
                                   const mluOpTensorDescriptor_t filters_desc,
                                   const void *filters,
                                   const mluOpTensorDescriptor_t indice_pairs_desc,
                                   const void *indice_pairs,
                                   const int64_t indice_num[],
                                   const int64_t inverse,
                                   const int64_t sub_m,
                                   void *workspace,
                                   const size_t workspace_size,
                                   const mluOpTensorDescriptor_t input_grad_desc,
                                   void *input_grad);

/* ------------------------------------------------------------------------
 * Indice convolution backward filter (reference mlu_op.h:9837-9947,
 * kernels/sparse_conv/indice_convolution_backward_filter/
 * indice_convolution_backward_filter.cpp:536-620)
 *
 *   features [L, Ci], output_grad [num_act_out, Co],
 *   filters_grad (kd,)kh,kw,Ci,Co whatever its layout tag.  The sum over
 *   pairs is always carried in fp32; the on-chip data type of filters_grad
 *   may be set to float to say so explicitly.
 * ---------------------------------------------------------------------- */
mluOpStatus_t MLUOP_WIN_API
mluOpGetIndiceConvolutionBackwardFilterWorkspaceSize(mluOpHandle_t handle,
                                                     const mluOpTensorDescriptor_t features_desc,
                                                     const mluOpTensorDescriptor_t output_grad_desc,
                                                     const mluOpTensorDescriptor_t indice_pairs_desc,
                                                     const mluOpTensorDescriptor_t filters_grad_desc,
                                                     const int64_t indice_num[],
                                                     const int64_t inverse,
                                                     const int64_t sub_m,
                                                     size_t *workspace_size);

mluOpStatus_t MLUOP_WIN_API
mluOpIndiceConvolutionBackwardFilter(mluOpHandle_t handle,
                                     const mluOpTensorDescriptor_t features_desc,
                                     const void *features,
                                     const mluOpTensorDescriptor_t output_grad_desc,
                                     const void *output_grad,
                                     const mluOpTensorDescriptor_t indice_pairs_desc,
                                     const void *indice_pairs,
                                     const int64_t indice_num[],
                                     const int64_t inverse,
                                     const int64_t sub_m,
                                     void *workspace,
                                     const size_t workspace_size,
                                     const mluOpTensorDescriptor_t filters_grad_desc,
                                     void *filters_grad);

/* ---------------------------------------------------------------------------
 * Hard voxelization: the step in front of the sparse convolutions, which turns a
 * point cloud into the voxel coordinates and features they consume.
 * ------------------------------------------------------------------------- */

/* reference mlu_op.h:5941-5953 (kernels/voxelization/voxelization.cpp:174-222).
 * Bytes of workspace mluOpVoxelization needs for these shapes.  Left untouched
 * when max_points or max_voxels is 0 (nothing to do), as in the reference. */
mluOpStatus_t MLUOP_WIN_API
mluOpGetVoxelizationWorkspaceSize(mluOpHandle_t handle,
                                  const mluOpTensorDescriptor_t points_desc,
                                  const mluOpTensorDescriptor_t voxel_size_desc,
                                  const mluOpTensorDescriptor_t coors_range_desc,
                                  const int32_t max_points,
                                  const int32_t max_voxels,
                                  const int32_t NDim,
                                  const bool deterministic,
                                  const mluOpTensorDescriptor_t voxels_desc,
                                  const mluOpTensorDescriptor_t coors_desc,
                                  const mluOpTensorDescriptor_t num_points_per_voxel_desc,
                                  const mluOpTensorDescriptor_t voxel_num_desc,
                                  size_t *size);

/* reference mlu_op.h:6050-6071 (kernels/voxelization/voxelization.cpp:224-367).
 * points [N, F] float (x, y, z first), voxel_size [3] and coors_range [6]
 * (x/y/z minima, then maxima) float, all in device memory.  Outputs, zero
 * filled first: voxels [max_voxels, max_points, F] float, coors [max_voxels, 3]
 * int32 as (z, y, x), num_points_per_voxel [max_voxels] int32, voxel_num [1]
 * int32.  Cells are numbered in the order of their first point; a cell keeps
 * its first max_points points, and cells past max_voxels are dropped.  Only
 * deterministic = true and NDim = 3 are accepted (BAD_PARAM otherwise). */
mluOpStatus_t MLUOP_WIN_API
mluOpVoxelization(mluOpHandle_t handle,
                  const mluOpTensorDescriptor_t points_desc,
                  const void *points,
                  const mluOpTensorDescriptor_t voxel_size_desc,
                  const void *voxel_size,
                  const mluOpTensorDescriptor_t coors_range_desc,
                  const void *coors_range,
                  const int32_t max_points,
                  const int32_t max_voxels,
                  const int32_t NDim,
                  const bool deterministic,
                  void *workspace,
                  size_t workspace_size,
                  const mluOpTensorDescriptor_t voxels_desc,
                  void *voxels,
                  const mluOpTensorDescriptor_t coors_desc,
                  void *coors,
                  const mluOpTensorDescriptor_t num_points_per_voxel_desc,
                  void *num_points_per_voxel,
                  const mluOpTensorDescriptor_t voxel_num_desc,
                  void *voxel_num);

/* ---------------------------------------------------------------------------
 * Dynamic point-to-voxel scatter (forward): the other upstream step, which groups
 * points by their voxel coordinate and reduces their features.
 * ------------------------------------------------------------------------- */

/* reference mlu_op.h:361-365 */
typedef enum {
  MLUOP_REDUCE_DSUM  = 0, /* not accepted by mluOpDynamicPointToVoxelForward */
  MLUOP_REDUCE_DMEAN = 1,
  MLUOP_REDUCE_DMAX  = 2,
} mluOpReduceMode_t;

/* reference mlu_op.h:3767-3771 (kernels/dynamic_point_to_voxel/
 * dynamic_point_to_voxel_forward/dynamic_point_to_voxel_forward.cpp:195-232). */
mluOpStatus_t MLUOP_WIN_API
mluOpGetDynamicPointToVoxelForwardWorkspaceSize(mluOpHandle_t handle,
                                                const mluOpTensorDescriptor_t feats_desc,
                                                const mluOpTensorDescriptor_t coors_desc,
                                                size_t *workspace_size);

/* reference mlu_op.h:3865-3883 (same file :234-380).  feats [N, C] float, coors
 * [N, 3] int32 (rows with a negative coordinate are rewritten to -1,-1,-1 in
 * place and belong to no voxel).  Outputs with M <= N rows: voxel_feats [M, C]
 * (max or mean over the points of a voxel; rows past voxel_num hold -inf for
 * max and 0 for mean), voxel_coors [M, 3] (distinct triples in ascending
 * order), point2voxel_map [N] (voxel of every point, -1 for none),
 * voxel_points_count [M], voxel_num [1].  reduce_type: MLUOP_REDUCE_DMAX or
 * MLUOP_REDUCE_DMEAN (BAD_PARAM otherwise).  The call synchronises the stream
 * once (it reads the largest coordinate back to size its sorts). */
mluOpStatus_t MLUOP_WIN_API
mluOpDynamicPointToVoxelForward(const mluOpHandle_t handle,
                                const mluOpReduceMode_t reduce_type,
                                const mluOpTensorDescriptor_t feats_desc,
                                const void *feats,
                                const mluOpTensorDescriptor_t coors_desc,
                                void *coors,
                                void *workspace,
                                const size_t workspace_size,
                                const mluOpTensorDescriptor_t voxel_feats_desc,
                                void *voxel_feats,
                                const mluOpTensorDescriptor_t voxel_coors_desc,
                                void *voxel_coors,
                                const mluOpTensorDescriptor_t point2voxel_map_desc,
                                void *point2voxel_map,
                                const mluOpTensorDescriptor_t voxel_points_count_desc,
                                void *voxel_points_count,
                                const mluOpTensorDescriptor_t voxel_num_desc,
                                void *voxel_num);

/* reference mlu_op.h:3750 region, mluOpGetDynamicPointToVoxelBackwardWorkspaceSize
 * (kernels/dynamic_point_to_voxel/dynamic_point_to_voxel_backward/
 * dynamic_point_to_voxel_backward.cpp:336-364): N * C ints. */
mluOpStatus_t MLUOP_WIN_API
mluOpGetDynamicPointToVoxelBackwardWorkspaceSize(const mluOpHandle_t handle,
                                                 const mluOpReduceMode_t reduce_type,
                                                 const mluOpTensorDescriptor_t grad_voxel_feats_desc,
                                                 const mluOpTensorDescriptor_t feats_desc,
                                                 const mluOpTensorDescriptor_t voxel_feats_desc,
                                                 const mluOpTensorDescriptor_t point2voxel_map_desc,
                                                 const mluOpTensorDescriptor_t voxel_points_count_desc,
                                                 const mluOpTensorDescriptor_t voxel_num_desc,
                                                 size_t *workspace_size);

/* reference mlu_op.h:3707-3725 (same file :177-334).  Gradient of the max
 * reduction (MLUOP_REDUCE_DMAX only, BAD_PARAM otherwise): grad_feats [N, C] is
 * zero except that, for every voxel and feature, the first point whose feature
 * equals the voxel's maximum receives grad_voxel_feats[voxel, feature]. */
mluOpStatus_t MLUOP_WIN_API
mluOpDynamicPointToVoxelBackward(const mluOpHandle_t handle,
                                 const mluOpReduceMode_t reduce_type,
                                 const mluOpTensorDescriptor_t grad_voxel_feats_desc,
                                 const void *grad_voxel_feats,
                                 const mluOpTensorDescriptor_t feats_desc,
                                 const void *feats,
                                 const mluOpTensorDescriptor_t voxel_feats_desc,
                                 const void *voxel_feats,
                                 const mluOpTensorDescriptor_t point2voxel_map_desc,
                                 const void *point2voxel_map,
                                 const mluOpTensorDescriptor_t voxel_points_count_desc,
                                 const void *voxel_points_count,
                                 const mluOpTensorDescriptor_t voxel_num_desc,
                                 const void *voxel_num,
                                 void *workspace,
                                 const size_t workspace_size,
                                 const mluOpTensorDescriptor_t grad_feats_desc,
                                 void *grad_feats);

#if defined(__cplusplus)
}
#endif

#endif /* MLUOP_AMD_MLU_OP_H_ */
