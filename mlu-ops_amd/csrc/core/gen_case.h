// Case dump inside the library: with MLUOP_GEN_CASE set, every operator call that passed its
// parameter checks writes a prototxt case file in the reference test runner's format
// (reference core/gen_case.{h,cpp}; call sites such as
// kernels/sparse_conv/get_indice_pairs/get_indice_pairs.cpp:47-75), which
// mluop_hip.casefile and the reference's gtest can replay.
//   MLUOP_GEN_CASE=1  shapes, types and operator parameters
//   MLUOP_GEN_CASE=2  also the values of the input tensors (the call waits for the queue and
//                     copies them to the host: a debugging aid, not for timed runs)
//   MLUOP_GEN_CASE=3  one line per call on stderr, no file
//   MLUOP_GEN_CASE_DIR  where the files go (default ./gen_case); one directory per operator
// The variables are read once, when the library first needs them.
#ifndef MLUOP_AMD_CORE_GEN_CASE_H_
#define MLUOP_AMD_CORE_GEN_CASE_H_

#include <cstdint>
#include <string>

#include "core/core.h"

namespace mluop {
namespace gen_case {

int mode();  // 0 when off

class CaseWriter {
 public:
  // op_name as in the case file ("get_indice_pairs"); param_name the name of its parameter
  // message ("get_indice_pairs_param").  Does nothing when mode() is 0.
  CaseWriter(mluOpHandle_t handle, const char *op_name, const char *param_name);
  bool on() const { return mode_ != 0; }
  void input(const char *id, const mluOpTensorDescriptor_t desc, const void *device_values);
  void output(const char *id, const mluOpTensorDescriptor_t desc);
  void param(const char *name, int64_t value);
  void paramName(const char *name, const char *enumerator);  // an enumeration written by name
  void params(const char *name, const int *values, int n);
  void params(const char *name, const int64_t *values, int n);
  // error functions DIFF1 and DIFF2 at `threshold`, CPU baseline; writes the file
  void finish(double threshold);

 private:
  void tensor(const char *kind, const char *id, const mluOpTensorDescriptor_t desc,
              const void *device_values);
  int mode_ = 0;
  mluOpHandle_t handle_ = nullptr;
  std::string op_, param_name_, tensors_, params_, summary_;
};

}  // namespace gen_case
}  // namespace mluop

#endif  // MLUOP_AMD_CORE_GEN_CASE_H_
