// Internal definitions shared by the host side of the library: the objects
// behind the opaque handles of mlu_op.h, logging and the parameter-check
// macros.  Nothing in here is part of the ABI.
#ifndef MLUOP_AMD_CORE_CORE_H_
#define MLUOP_AMD_CORE_CORE_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <sstream>
#include <string>
#include <vector>

#include "core/launch.h"
#include "mlu_op.h"

// reference core/logging.h:37, get_indice_pairs_structs.h:36
#define LARGE_TENSOR_NUM ((uint64_t)2147483648ULL)
#define INDICE_IN_LARGE_TENSOR_NUM 1000000

// ---------------------------------------------------------------------------
// Handle (reference core/context.h:71-147).  The reference keeps MLU cluster
// and NRAM sizes; the fields that matter on this platform are the HIP device,
// the stream and the CU count used to size launches.
// ---------------------------------------------------------------------------
struct mluOpContext {
  int device = -1;            // HIP device ordinal; -1 for a host-only handle
  hipStream_t queue = nullptr;
  int arch = 0;               // numeric part of the gfx name, e.g. 950
  int cu_count = 0;
  int lds_bytes = 0;
  mluOpQuantizeRoundMode_t round_mode = MLUOP_ROUND_HALF_TO_EVEN;
  mluOpAtomicsMode_t atomics_mode = MLUOP_ATOMICS_NOT_ALLOWED;
  int32_t *pinned_scalar = nullptr;  // 64-byte pinned host slot for read-backs
  hipEvent_t readback_event = nullptr;  // recorded behind a kernel that stores into the slot
  mluop::KernelTimer timer;          // per-kernel event timing, off by default
  // Modes the reference rejects (inverse convolution, filters_grad written in its
  // tagged layout): off unless mluOpExtSetSparseConvExtendedModes switched them on.
  bool sparse_conv_extended = false;
  // The caller's promise that no offset of a rulebook names a result row twice
  // (mluOpExtSetDistinctPairsPromise): forward and backward data then skip the
  // check that finds and adds such pairs.
  bool distinct_pairs_promised = false;
  // Row maps built by mluOpExtBuildRowMap with no pair lost, and the one announced for the
  // next forward / backward-data call (mluOpExtUseRowMap).
  struct RowMapRecord {
    const void *map;
    const void *pairs;
    int K, L, rows, source_rows, row_column;
  };
  std::vector<RowMapRecord> row_maps;
  const void *pending_row_map = nullptr;
  // Rulebooks mluOpGetIndicePairs built on this handle, by the address of their pair tensor.
  // The last kernel of a rulebook reports into a slot of pinned host memory whether the
  // input rows were in cell order (then both pair columns ascend inside every offset); the
  // convolution operators read the slot, without waiting for anything, to choose their way
  // through the pair lists.  A note is a hint about speed only: what the kernels rely on is
  // checked on the device in every call.
  struct RulebookReport {       // pinned host memory, written by the device
    unsigned long long stamp;   // the note's stamp, stored after the flag
    unsigned int rows_in_order;
    unsigned int unused;
  };
  struct RulebookNote {
    const void *pairs = nullptr;
    int K = 0, L = 0;
    unsigned long long stamp = 0;
  };
  static constexpr int kRulebookNotes = 32;
  RulebookNote rulebook_notes[kRulebookNotes];
  RulebookReport *rulebook_reports = nullptr;  // kRulebookNotes slots behind pinned_scalar
  int next_rulebook_note = 0;
  unsigned long long next_stamp = 1;   // also the source of per-call tickets

  // What the kernel launchers need: the stream, and the timer while it is on.
  mluop::KernelChoices kernel_choices;
  mluop::LaunchCtx launchCtx() {
    return mluop::LaunchCtx(queue, timer.enabled ? &timer : nullptr, &kernel_choices);
  }
};

// ---------------------------------------------------------------------------
// Tensor descriptor (reference core/tensor.h:41-235).
// ---------------------------------------------------------------------------
struct mluOpTensorStruct {
  int dim = 0;
  int64_t normal_dims[MLUOP_DIM_MAX] = {0};
  int64_t normal_strides[MLUOP_DIM_MAX] = {0};
  int64_t *dims = normal_dims;
  int64_t *strides = normal_strides;
  mluOpDataType_t dtype = MLUOP_DTYPE_FLOAT;
  mluOpDataType_t onchip_dtype = MLUOP_DTYPE_INVALID;
  mluOpTensorLayout_t layout = MLUOP_LAYOUT_ARRAY;
  mluOpPointerMode_t pointer_mode = MLUOP_POINTER_MODE_DEVICE;
  uint64_t total_element_num = 0;
  uint64_t total_tensor_size = 0;

  ~mluOpTensorStruct() { releaseDims(); }
  void releaseDims() {
    if (dims != normal_dims) delete[] dims;
    if (strides != normal_strides) delete[] strides;
    dims = normal_dims;
    strides = normal_strides;
  }
  int getDim() const { return dim; }
  int64_t getDimIndex(int i) const { return dims[i]; }
  mluOpDataType_t getDtype() const { return dtype; }
  mluOpDataType_t getOnchipDtype() const { return onchip_dtype; }
  mluOpTensorLayout_t getLayout() const { return layout; }
  uint64_t getTotalElementNum() const { return total_element_num; }
};

// ---------------------------------------------------------------------------
// Sparse convolution descriptor (reference get_indice_pairs_structs.h:85-98).
// ---------------------------------------------------------------------------
struct mluOpSparseConvolutionStruct {
  int dimNb = 0;
  int batch = 0;
  int pad[6] = {0};
  int stride[6] = {0};
  int dilation[6] = {0};
  int input_space[3] = {0};
  int filter_space[3] = {0};
  int output_space[3] = {0};
  int sub_m = 0;
  int transpose = 0;
  int inverse = 0;
  int num_act_out = 0;
};

namespace mluop {

size_t getSizeOfDataType(mluOpDataType_t dtype);
const char *getNameOfDataType(mluOpDataType_t dtype);
const char *getNameOfTensorLayout(mluOpTensorLayout_t layout);
bool isStrideTensor(int dim, const int64_t *dims, const int64_t *strides);

// Dimension getters by layout (reference core/tensor.h:387-478); 0 when the
// layout has no such dimension.
int64_t dimN(const mluOpTensorStruct *d);
int64_t dimC(const mluOpTensorStruct *d);
int64_t dimD(const mluOpTensorStruct *d);
int64_t dimH(const mluOpTensorStruct *d);
int64_t dimW(const mluOpTensorStruct *d);

// Error lines go to stderr unless MLUOP_LOG_PRINT=0 is set in the environment.
bool logEnabled();
void logLine(const char *level, const std::string &msg);

class LogMessage {
 public:
  explicit LogMessage(const char *level) : level_(level) {}
  ~LogMessage() { logLine(level_, ss_.str()); }
  std::ostringstream &stream() { return ss_; }

 private:
  const char *level_;
  std::ostringstream ss_;
};

}  // namespace mluop

#define MLUOP_LOG(level) ::mluop::LogMessage(#level).stream()

// Check macros with the status conventions of reference core/logging.h:93-230.
#define PARAM_CHECK(api, condition)                                  \
  if (!(condition)) {                                                \
    MLUOP_LOG(ERROR) << api << " Check failed: " #condition ". ";    \
    return MLUOP_STATUS_BAD_PARAM;                                   \
  }

#define PARAM_CHECK_V2(api, condition, extra)                              \
  if (!(condition)) {                                                      \
    MLUOP_LOG(ERROR) << api << " Check failed: " #condition ". " << extra; \
    return MLUOP_STATUS_BAD_PARAM;                                         \
  }

#define PARAM_CHECK_EQ(api, a, b) PARAM_CHECK(api, (a) == (b))
#define PARAM_CHECK_LE(api, a, b) PARAM_CHECK(api, (a) <= (b))

#define STRIDE_TENSOR_CHECK(api, desc, reason)                                   \
  if ((desc) != NULL && (desc)->total_element_num != 0 &&                        \
      ::mluop::isStrideTensor((desc)->dim, (desc)->dims, (desc)->strides)) {     \
    MLUOP_LOG(ERROR) << api << " stride tensor is not supported. " << reason;    \
    return MLUOP_STATUS_NOT_SUPPORTED;                                           \
  }

#define TENSOR_NUM_CHECK(api, num, max_num, reason)                                  \
  if (!((num) < (max_num))) {                                                        \
    MLUOP_LOG(ERROR) << api << " overflow max supported tensor num " << (max_num)-1  \
                     << ", now tensor's total num is " << (num) << ". " << reason;   \
    return MLUOP_STATUS_NOT_SUPPORTED;                                               \
  }

#define CHECK_RETURN(api, status)                                              \
  {                                                                            \
    mluOpStatus_t __status__ = (status);                                       \
    if (__status__ != MLUOP_STATUS_SUCCESS) {                                  \
      MLUOP_LOG(ERROR) << api << " BAD return status: " #status " returns "    \
                       << (int)__status__;                                     \
      return __status__;                                                       \
    }                                                                          \
  }

// A failed HIP runtime call or launch maps to EXECUTION_FAILED, the status the
// reference's KERNEL_CHECK gives for a failed kernel invocation.
#define HIP_CHECK_RETURN(api, call)                                            \
  {                                                                            \
    hipError_t __e__ = (call);                                                 \
    if (__e__ != hipSuccess) {                                                 \
      MLUOP_LOG(ERROR) << api << " " #call " failed: "                         \
                       << hipGetErrorString(__e__);                            \
      return MLUOP_STATUS_EXECUTION_FAILED;                                    \
    }                                                                          \
  }

// Every operator refuses to launch on a handle that has no device behind it.
#define DEVICE_HANDLE_CHECK(api, handle)                                            \
  if ((handle)->device < 0) {                                                       \
    MLUOP_LOG(ERROR) << api << " the handle was created without a HIP device "      \
                     << "(host-only handle): no kernel can be launched.";           \
    return MLUOP_STATUS_EXECUTION_FAILED;                                           \
  }

#endif  // MLUOP_AMD_CORE_CORE_H_
