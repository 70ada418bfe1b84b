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

class LaunchCtx {
 public:
  LaunchCtx(hipStream_t s, KernelTimer *t) : stream(s), timer_(t) {}
  hipStream_t stream;

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
