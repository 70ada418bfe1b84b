#include "core/gen_case.h"

#include <sys/stat.h>
#include <sys/types.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

namespace mluop {
namespace gen_case {

namespace {

struct Settings {
  int mode = 0;
  std::string dir = "gen_case";
};

const Settings &settings() {
  static const Settings s = [] {
    Settings v;
    if (const char *m = getenv("MLUOP_GEN_CASE")) v.mode = atoi(m);
    if (v.mode < 0 || v.mode > 3) v.mode = 0;
    if (const char *d = getenv("MLUOP_GEN_CASE_DIR")) {
      if (d[0] != '\0') v.dir = d;
    }
    return v;
  }();
  return s;
}

const char *protoDtype(mluOpDataType_t t) {
  switch (t) {
    case MLUOP_DTYPE_HALF: return "DTYPE_HALF";
    case MLUOP_DTYPE_FLOAT: return "DTYPE_FLOAT";
    case MLUOP_DTYPE_BFLOAT16: return "DTYPE_BFLOAT16";
    case MLUOP_DTYPE_INT32: return "DTYPE_INT32";
    case MLUOP_DTYPE_INT64: return "DTYPE_INT64";
    case MLUOP_DTYPE_INT8: return "DTYPE_INT8";
    case MLUOP_DTYPE_INT16: return "DTYPE_INT16";
    case MLUOP_DTYPE_DOUBLE: return "DTYPE_DOUBLE";
    default: return "DTYPE_INVALID";
  }
}

const char *protoLayout(mluOpTensorLayout_t l) {
  switch (l) {
    case MLUOP_LAYOUT_NCHW: return "LAYOUT_NCHW";
    case MLUOP_LAYOUT_NHWC: return "LAYOUT_NHWC";
    case MLUOP_LAYOUT_HWCN: return "LAYOUT_HWCN";
    case MLUOP_LAYOUT_NDHWC: return "LAYOUT_NDHWC";
    case MLUOP_LAYOUT_NCDHW: return "LAYOUT_NCDHW";
    default: return "LAYOUT_ARRAY";
  }
}

void makeDirs(const std::string &path) {
  std::string part;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!part.empty()) (void)mkdir(part.c_str(), 0777);  // existing directories are fine
    }
    if (i < path.size()) part += path[i];
  }
}

std::atomic<unsigned> g_serial{0};

}  // namespace

int mode() { return settings().mode; }

CaseWriter::CaseWriter(mluOpHandle_t handle, const char *op_name, const char *param_name)
    : mode_(settings().mode), handle_(handle), op_(op_name), param_name_(param_name) {}

void CaseWriter::tensor(const char *kind, const char *id, const mluOpTensorDescriptor_t desc,
                        const void *device_values) {
  if (mode_ == 0 || desc == nullptr) return;
  std::string shape;
  for (int i = 0; i < desc->dim; ++i) shape += "    dims: " + std::to_string(desc->dims[i]) + "\n";
  summary_ += std::string(" ") + id + "[";
  for (int i = 0; i < desc->dim; ++i) summary_ += (i ? "," : "") + std::to_string(desc->dims[i]);
  summary_ += "]";
  if (mode_ == 3) return;
  tensors_ += std::string(kind) + " {\n  id: \"" + id + "\"\n  shape {\n" + shape + "  }\n  layout: " +
              protoLayout(desc->layout) + "\n  dtype: " + protoDtype(desc->dtype) + "\n";
  if (desc->onchip_dtype != MLUOP_DTYPE_INVALID)
    tensors_ += std::string("  onchip_dtype: ") + protoDtype(desc->onchip_dtype) + "\n";
  const size_t elem = mluop::getSizeOfDataType(desc->dtype);
  const size_t n = (size_t)desc->total_element_num;
  if (mode_ == 2 && device_values != nullptr && n > 0 && elem > 0 && handle_ != nullptr &&
      handle_->device >= 0) {
    std::vector<unsigned char> host(n * elem);
    if (hipStreamSynchronize(handle_->queue) == hipSuccess &&
        hipMemcpy(host.data(), device_values, n * elem, hipMemcpyDeviceToHost) == hipSuccess) {
      char buf[48];
      for (size_t i = 0; i < n; ++i) {
        if (desc->dtype == MLUOP_DTYPE_INT32) {
          int32_t v;
          memcpy(&v, &host[i * 4], 4);
          snprintf(buf, sizeof(buf), "  value_i: %d\n", v);
        } else if (elem == 2) {
          uint16_t v;
          memcpy(&v, &host[i * 2], 2);
          snprintf(buf, sizeof(buf), "  value_h: \"%04x\"\n", (unsigned)v);
        } else if (elem == 4) {
          uint32_t v;
          memcpy(&v, &host[i * 4], 4);
          snprintf(buf, sizeof(buf), "  value_h: \"%08x\"\n", (unsigned)v);
        } else {
          break;  // other types are dumped without values
        }
        tensors_ += buf;
      }
    }
  }
  tensors_ += "}\n";
}

void CaseWriter::input(const char *id, const mluOpTensorDescriptor_t desc, const void *device_values) {
  tensor("input", id, desc, device_values);
}

void CaseWriter::output(const char *id, const mluOpTensorDescriptor_t desc) {
  tensor("output", id, desc, nullptr);
}

void CaseWriter::param(const char *name, int64_t value) {
  if (mode_ == 0) return;
  params_ += std::string("  ") + name + ": " + std::to_string(value) + "\n";
}

void CaseWriter::paramName(const char *name, const char *enumerator) {
  if (mode_ == 0) return;
  params_ += std::string("  ") + name + ": " + enumerator + "\n";
}

void CaseWriter::params(const char *name, const int *values, int n) {
  for (int i = 0; i < n; ++i) param(name, values[i]);
}

void CaseWriter::params(const char *name, const int64_t *values, int n) {
  for (int i = 0; i < n; ++i) param(name, values[i]);
}

void CaseWriter::finish(double threshold) {
  if (mode_ == 0) return;
  if (mode_ == 3) {
    fprintf(stderr, "[MLUOP_GEN_CASE] %s:%s\n", op_.c_str(), summary_.c_str());
    return;
  }
  char thr[64];
  snprintf(thr, sizeof(thr), "%g", threshold);
  std::string text = "op_name: \"" + op_ + "\"\n" + tensors_ + param_name_ + " {\n" + params_ + "}\n" +
                     "test_param {\n  error_func: DIFF1\n  error_func: DIFF2\n  error_threshold: " + thr +
                     "\n  error_threshold: " + thr + "\n  baseline_device: CPU\n}\n";
  const std::string dir = settings().dir + "/" + op_;
  static std::mutex dir_mutex;
  {
    std::lock_guard<std::mutex> guard(dir_mutex);
    makeDirs(dir);
  }
  const auto now = std::chrono::system_clock::now().time_since_epoch();
  const long long us = std::chrono::duration_cast<std::chrono::microseconds>(now).count();
  const std::string path = dir + "/" + op_ + "_" + std::to_string(us) + "_pid" + std::to_string((long)getpid()) +
                           "_" + std::to_string(g_serial.fetch_add(1)) + ".prototxt";
  FILE *f = fopen(path.c_str(), "w");
  if (f == nullptr) {
    MLUOP_LOG(ERROR) << "[MLUOP_GEN_CASE] cannot write " << path;
    return;
  }
  fwrite(text.data(), 1, text.size(), f);
  fclose(f);
}

}  // namespace gen_case
}  // namespace mluop
