// Handle management: mluOpCreate / Destroy / SetQueue / GetQueue and the
// small per-handle switches.  Behaviour follows reference
// core/context.cpp:158-470; the MLU attribute reads become a read of the HIP
// device properties and the queue is a hipStream_t.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <new>

#include "core/core.h"
#include "mlu_op_ext.h"
#include "sparse_conv/no_alloc_scratch.h"

namespace {

int parseGfxNumber(const char *name) {
  // "gfx950:sramecc+:xnack-" -> 950 ; "gfx90a" -> 0x90a is not needed here,
  // only gfx950 is a supported target, so a decimal parse is enough.
  const char *p = strstr(name, "gfx");
  if (p == nullptr) return 0;
  return atoi(p + 3);
}

bool hostOnlyHandleRequested() {
  const char *v = getenv("MLUOP_HOST_ONLY_HANDLE");
  return v != nullptr && v[0] == '1';
}

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpCreate(mluOpHandle_t *handle) {
  PARAM_CHECK("[mluOpCreate]", handle != NULL);
  mluOpContext *ctx = new (std::nothrow) mluOpContext();
  if (ctx == nullptr) return MLUOP_STATUS_ALLOC_FAILED;

  if (hostOnlyHandleRequested()) {
    // A handle for exercising descriptor logic and parameter checks: no device is looked
    // for, whether the machine has one or not (the tests that ask for it pass made-up
    // pointers, which must never reach a kernel).  It reports the supported architecture
    // so the checks behind the architecture gate can be reached; every operator returns
    // EXECUTION_FAILED before it would launch anything.
    ctx->device = -1;
    ctx->arch = 950;
    *handle = ctx;
    return MLUOP_STATUS_SUCCESS;
  }
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    MLUOP_LOG(ERROR) << "[mluOpCreate] no usable HIP device: " << hipGetErrorString(err);
    delete ctx;
    return MLUOP_STATUS_INTERNAL_ERROR;
  }
  hipDeviceProp_t prop;
  err = hipGetDeviceProperties(&prop, dev);
  if (err != hipSuccess) {
    MLUOP_LOG(ERROR) << "[mluOpCreate] hipGetDeviceProperties failed: " << hipGetErrorString(err);
    delete ctx;
    return MLUOP_STATUS_INTERNAL_ERROR;
  }
  ctx->device = dev;
  ctx->arch = parseGfxNumber(prop.gcnArchName);
  ctx->cu_count = prop.multiProcessorCount;
  ctx->lds_bytes = (int)prop.sharedMemPerBlock;
  void *pinned = nullptr;
  const size_t pinned_bytes = 64 + sizeof(mluOpContext::RulebookReport) * mluOpContext::kRulebookNotes;
  err = hipHostMalloc(&pinned, pinned_bytes, hipHostMallocDefault);
  if (err != hipSuccess) {
    MLUOP_LOG(ERROR) << "[mluOpCreate] hipHostMalloc failed: " << hipGetErrorString(err);
    delete ctx;
    return MLUOP_STATUS_ALLOC_FAILED;
  }
  ctx->pinned_scalar = static_cast<int32_t *>(pinned);
  memset(pinned, 0, pinned_bytes);
  err = hipEventCreateWithFlags(&ctx->readback_event, hipEventDisableTiming | hipEventReleaseToSystem);
  if (err != hipSuccess) {
    MLUOP_LOG(ERROR) << "[mluOpCreate] hipEventCreateWithFlags failed: " << hipGetErrorString(err);
    (void)hipHostFree(pinned);
    delete ctx;
    return MLUOP_STATUS_INTERNAL_ERROR;
  }
  ctx->rulebook_reports =
      reinterpret_cast<mluOpContext::RulebookReport *>(static_cast<char *>(pinned) + 64);
  // Stamps and tickets only have to differ from what earlier calls, of this handle or of
  // another, left in memory: start somewhere no other handle starts.
  ctx->next_stamp = ((unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count()
                     << 20) ^ (unsigned long long)reinterpret_cast<uintptr_t>(ctx) ^ 0x9E3779B97F4A7C15ull;
  // `dev` is the current device: the address of the library's scratch array on it is looked
  // up here, once, so that the entry point that uses it has nothing to set up.
  err = mluop::sparse_conv::lookUpNoAllocScratch(dev);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    MLUOP_LOG(WARNING) << "[mluOpCreate] hipGetSymbolAddress for the scratch array failed: "
                       << hipGetErrorString(err)
                       << "; mluOpExtIndiceConvolutionBackwardFilterNoAlloc will refuse to run.";
  }
  *handle = ctx;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpDestroy(mluOpHandle_t handle) {
  PARAM_CHECK("[mluOpDestroy]", handle != NULL);
  if (handle->device >= 0) {
    // Kernels of this handle's rulebooks store into the handle's report slots: nothing of
    // them may be in flight when the slots go away.  (A queue that is being captured cannot
    // be waited for; a graph captured from it must not be replayed after this call.)
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(handle->queue, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing == hipStreamCaptureStatusNone && hipStreamSynchronize(handle->queue) != hipSuccess)
      (void)hipGetLastError();
  }
  if (handle->pinned_scalar != nullptr) (void)hipHostFree(handle->pinned_scalar);
  if (handle->readback_event != nullptr) (void)hipEventDestroy(handle->readback_event);
  handle->timer.destroy();
  delete handle;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetQueue(mluOpHandle_t handle, mluOpQueue_t queue) {
  PARAM_CHECK("[mluOpSetQueue]", handle != NULL);
  handle->queue = reinterpret_cast<hipStream_t>(queue);  // NULL is allowed
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetQueue(mluOpHandle_t handle, mluOpQueue_t *queue) {
  PARAM_CHECK("[mluOpGetQueue]", handle != NULL);
  PARAM_CHECK("[mluOpGetQueue]", queue != NULL);
  *queue = reinterpret_cast<mluOpQueue_t>(handle->queue);
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetQuantizeRoundMode(mluOpHandle_t handle,
                                                      mluOpQuantizeRoundMode_t round_mode) {
  PARAM_CHECK("[mluOpSetQuantizeRoundMode]", handle != NULL);
  // A C caller can pass any integer here; it is looked at as one before it is used as the
  // enumeration.
  int as_int = 0;
  static_assert(sizeof(as_int) == sizeof(round_mode), "enumeration passed as an int");
  std::memcpy(&as_int, &round_mode, sizeof(as_int));
  PARAM_CHECK("[mluOpSetQuantizeRoundMode]", as_int == MLUOP_ROUND_HALF_TO_EVEN ||
                                                 as_int == MLUOP_ROUND_HALF_OFF_ZERO ||
                                                 as_int == MLUOP_ROUND_HALF_UP);
  handle->round_mode = round_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetQuantizeRoundMode(mluOpHandle_t handle,
                                                      mluOpQuantizeRoundMode_t *round_mode) {
  PARAM_CHECK("[mluOpGetQuantizeRoundMode]", handle != NULL);
  PARAM_CHECK("[mluOpGetQuantizeRoundMode]", round_mode != NULL);
  *round_mode = handle->round_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetAtomicsMode(mluOpHandle_t handle,
                                                mluOpAtomicsMode_t atomics_mode) {
  PARAM_CHECK("[mluOpSetAtomicsMode]", handle != NULL);
  handle->atomics_mode = atomics_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetAtomicsMode(mluOpHandle_t handle,
                                                mluOpAtomicsMode_t *atomics_mode) {
  PARAM_CHECK("[mluOpGetAtomicsMode]", handle != NULL);
  PARAM_CHECK("[mluOpGetAtomicsMode]", atomics_mode != NULL);
  *atomics_mode = handle->atomics_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtSetKernelTiming(mluOpHandle_t handle, int enable) {
  PARAM_CHECK("[mluOpExtSetKernelTiming]", handle != NULL);
  if (handle->device >= 0) (void)hipStreamSynchronize(handle->queue);
  handle->timer.clear();
  handle->timer.enabled = enable != 0 && handle->device >= 0;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtSetKernelChoice(mluOpHandle_t handle,
                                                    mluOpExtKernelChoice_t which, int value) {
  PARAM_CHECK("[mluOpExtSetKernelChoice]", handle != NULL);
  PARAM_CHECK("[mluOpExtSetKernelChoice]", value >= -1 && value <= 1);
  int as_int = 0;
  static_assert(sizeof(as_int) == sizeof(which), "enumeration passed as an int");
  std::memcpy(&as_int, &which, sizeof(as_int));
  mluop::KernelChoices &c = handle->kernel_choices;
  switch (as_int) {
    case MLUOP_EXT_KERNEL_GATHER_SIMT: c.gather_simt = value; break;
    case MLUOP_EXT_KERNEL_DENSE_TILES: c.dense_tiles = value; break;
    case MLUOP_EXT_KERNEL_WAVE_PER_TILE: c.wave_per_tile = value; break;
    case MLUOP_EXT_KERNEL_FLAT_SLICE_SUM: c.flat_slice_sum = value; break;
    case MLUOP_EXT_KERNEL_FLAT_SCATTER: c.flat_scatter = value; break;
    case MLUOP_EXT_KERNEL_SMALL_MAP_CHUNKS: c.small_map_chunks = value; break;
    case MLUOP_EXT_KERNEL_FILTER_STORES: c.filter_stores = value; break;
    case MLUOP_EXT_KERNEL_LISTS_ON_TRUST: c.lists_on_trust = value; break;
    default:
      MLUOP_LOG(ERROR) << "[mluOpExtSetKernelChoice] unknown kernel choice " << as_int;
      return MLUOP_STATUS_BAD_PARAM;
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtSetSparseConvExtendedModes(mluOpHandle_t handle,
                                                               int enable) {
  PARAM_CHECK("[mluOpExtSetSparseConvExtendedModes]", handle != NULL);
  handle->sparse_conv_extended = enable != 0;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtSetDistinctPairsPromise(mluOpHandle_t handle, int promised) {
  PARAM_CHECK("[mluOpExtSetDistinctPairsPromise]", handle != NULL);
  handle->distinct_pairs_promised = promised != 0;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTimingCount(mluOpHandle_t handle, int *count) {
  PARAM_CHECK("[mluOpExtGetKernelTimingCount]", handle != NULL);
  PARAM_CHECK("[mluOpExtGetKernelTimingCount]", count != NULL);
  if (handle->device >= 0) {
    HIP_CHECK_RETURN("[mluOpExtGetKernelTimingCount]", hipStreamSynchronize(handle->queue));
  }
  *count = (int)handle->timer.records.size();
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpExtGetKernelTiming(mluOpHandle_t handle, int index,
                                                    const char **name, float *milliseconds) {
  const char *api = "[mluOpExtGetKernelTiming]";
  PARAM_CHECK(api, handle != NULL);
  PARAM_CHECK(api, name != NULL);
  PARAM_CHECK(api, milliseconds != NULL);
  PARAM_CHECK(api, index >= 0 && index < (int)handle->timer.records.size());
  const mluop::KernelTimingRecord &r = handle->timer.records[index];
  *name = r.name;
  HIP_CHECK_RETURN(api, hipEventElapsedTime(milliseconds, r.start, r.stop));
  return MLUOP_STATUS_SUCCESS;
}

void MLUOP_WIN_API mluOpGetLibVersion(int *major, int *minor, int *patch) {
  if (major) *major = MLUOP_MAJOR;
  if (minor) *minor = MLUOP_MINOR;
  if (patch) *patch = MLUOP_PATCHLEVEL;
}

const char *MLUOP_WIN_API mluOpGetErrorString(mluOpStatus_t status) {
  switch (status) {
    case MLUOP_STATUS_SUCCESS: return "MLUOP_STATUS_SUCCESS";
    case MLUOP_STATUS_NOT_INITIALIZED: return "MLUOP_STATUS_NOT_INITIALIZED";
    case MLUOP_STATUS_ALLOC_FAILED: return "MLUOP_STATUS_ALLOC_FAILED";
    case MLUOP_STATUS_BAD_PARAM: return "MLUOP_STATUS_BAD_PARAM";
    case MLUOP_STATUS_INTERNAL_ERROR: return "MLUOP_STATUS_INTERNAL_ERROR";
    case MLUOP_STATUS_ARCH_MISMATCH: return "MLUOP_STATUS_ARCH_MISMATCH";
    case MLUOP_STATUS_EXECUTION_FAILED: return "MLUOP_STATUS_EXECUTION_FAILED";
    case MLUOP_STATUS_NOT_SUPPORTED: return "MLUOP_STATUS_NOT_SUPPORTED";
    case MLUOP_STATUS_NUMERICAL_OVERFLOW: return "MLUOP_STATUS_NUMERICAL_OVERFLOW";
  }
  return "MLUOP_STATUS_UNKNOWN";
}

}  // extern "C"

namespace mluop {

bool logEnabled() {
  static const bool enabled = [] {
    const char *v = getenv("MLUOP_LOG_PRINT");
    return !(v != nullptr && v[0] == '0');
  }();
  return enabled;
}

void logLine(const char *level, const std::string &msg) {
  if (!logEnabled()) return;
  fprintf(stderr, "[mluop][%s] %s\n", level, msg.c_str());
}

}  // namespace mluop
