// Launch context handed from the API layer to the kernel launchers: the HIP
// stream plus an optional per-kernel event timer.
#ifndef MLUOP_AMD_CORE_LAUNCH_H_
#define MLUOP_AMD_CORE_LAUNCH_H_

#include <hip/hip_runtime_api.h>

#include <vector>

namespace mluop {

struct KernelTimingRecord {
  const char *name;
  hipEvent_t start;
  hipEvent_t stop;
};

struct KernelTimer {
  bool enabled = false;
  std::vector<KernelTimingRecord> records;  // launches since timing was enabled
  std::vector<hipEvent_t> spare;            // events kept for reuse
  static constexpr size_t kMaxRecords = 1 << 16;

  hipEvent_t takeEvent() {
    if (!spare.empty()) {
      hipEvent_t e = spare.back();
      spare.pop_back();
      return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
  }
  void clear() {
    for (auto &r : records) {
      if (r.start) spare.push_back(r.start);
      if (r.stop) spare.push_back(r.stop);
    }
    records.clear();
  }
  void destroy() {
    clear();
    for (hipEvent_t e : spare) (void)hipEventDestroy(e);
    spare.clear();
  }
};

// Which kernel the sparse convolution launchers take where more than one computes the same
// result: -1 lets the shape decide, 0 / 1 switch a kernel off / on for every shape it can
// run.  A handle holds one set (mluOpExtSetKernelChoice); the parity tests use it to run
// both kernels of a pair on one shape.
struct KernelChoices {
  int gather_simt = -1;     // 1: the plain SIMT gather and filter-gradient kernels instead of MFMA
  int dense_tiles = -1;     // the register-accumulating gather kernel
  int wave_per_tile = -1;   // the one-wavefront-per-tile gather kernel
  int flat_slice_sum = -1;  // backward filter: partial tiles summed on the flat grid
  int flat_scatter = -1;    // 1: row maps built on the flat grid
  int small_map_chunks = -1;  // 1: row maps cover 2048 result rows at a time (the chunked path, on small inputs)
  int filter_stores = -1;   // 1: backward filter transposes with element-sized LDS stores also where transposing reads serve
  int lists_on_trust = -1;  // pair lists of unreported order: -1 lists with the row-map kernels behind, 0 row map, 1 lists only
};

class LaunchCtx {
 public:
  LaunchCtx(hipStream_t s, KernelTimer *t, const KernelChoices *c = nullptr)
      : stream(s), choices(c ? *c : KernelChoices()), timer_(t) {}
  hipStream_t stream;
  KernelChoices choices;

  // Call right before / right after enqueueing kernel `name`.
  void begin(const char *name) const {
    if (timer_ == nullptr || timer_->records.size() >= KernelTimer::kMaxRecords) return;
    KernelTimingRecord r{name, timer_->takeEvent(), timer_->takeEvent()};
    if (r.start == nullptr || r.stop == nullptr) return;
    (void)hipEventRecord(r.start, stream);
    timer_->records.push_back(r);
    open_ = true;
  }
  void end() const {
    if (!open_) return;
    (void)hipEventRecord(timer_->records.back().stop, stream);
    open_ = false;
  }

 private:
  KernelTimer *timer_;
  mutable bool open_ = false;
};

}  // namespace mluop

#endif  // MLUOP_AMD_CORE_LAUNCH_H_
