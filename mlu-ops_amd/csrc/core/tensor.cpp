// Tensor descriptor API.  Behaviour and status codes follow reference
// core/tensor.cpp:245-857 (set/get/reset), core/type.h:55-86 (element sizes),
// core/util.cpp:42-55 (contiguity test) and core/tensor.h:387-478 (dimension
// getters by layout).
#include <algorithm>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "core/core.h"

namespace mluop {

size_t getSizeOfDataType(mluOpDataType_t dtype) {
  switch (dtype) {
    case MLUOP_DTYPE_BOOL:
    case MLUOP_DTYPE_INT8:
    case MLUOP_DTYPE_UINT8:
      return 1;
    case MLUOP_DTYPE_INT16:
    case MLUOP_DTYPE_UINT16:
    case MLUOP_DTYPE_HALF:
    case MLUOP_DTYPE_BFLOAT16:
      return 2;
    case MLUOP_DTYPE_INT31:
    case MLUOP_DTYPE_INT32:
    case MLUOP_DTYPE_UINT32:
    case MLUOP_DTYPE_FLOAT:
    case MLUOP_DTYPE_COMPLEX_HALF:
      return 4;
    case MLUOP_DTYPE_UINT64:
    case MLUOP_DTYPE_INT64:
    case MLUOP_DTYPE_DOUBLE:
    case MLUOP_DTYPE_COMPLEX_FLOAT:
      return 8;
    default:
      return 0;
  }
}

const char *getNameOfDataType(mluOpDataType_t dtype) {
  switch (dtype) {
    case MLUOP_DTYPE_INVALID: return "DTYPE_INVALID";
    case MLUOP_DTYPE_HALF: return "DTYPE_HALF";
    case MLUOP_DTYPE_FLOAT: return "DTYPE_FLOAT";
    case MLUOP_DTYPE_DOUBLE: return "DTYPE_DOUBLE";
    case MLUOP_DTYPE_INT8: return "DTYPE_INT8";
    case MLUOP_DTYPE_INT16: return "DTYPE_INT16";
    case MLUOP_DTYPE_INT31: return "DTYPE_INT31";
    case MLUOP_DTYPE_INT32: return "DTYPE_INT32";
    case MLUOP_DTYPE_INT64: return "DTYPE_INT64";
    case MLUOP_DTYPE_UINT8: return "DTYPE_UINT8";
    case MLUOP_DTYPE_UINT16: return "DTYPE_UINT16";
    case MLUOP_DTYPE_UINT32: return "DTYPE_UINT32";
    case MLUOP_DTYPE_UINT64: return "DTYPE_UINT64";
    case MLUOP_DTYPE_BOOL: return "DTYPE_BOOL";
    case MLUOP_DTYPE_COMPLEX_HALF: return "DTYPE_COMPLEX_HALF";
    case MLUOP_DTYPE_COMPLEX_FLOAT: return "DTYPE_COMPLEX_FLOAT";
    case MLUOP_DTYPE_BFLOAT16: return "DTYPE_BFLOAT16";
  }
  return "DTYPE_INVALID";
}

const char *getNameOfTensorLayout(mluOpTensorLayout_t layout) {
  switch (layout) {
    case MLUOP_LAYOUT_NCHW: return "LAYOUT_NCHW";
    case MLUOP_LAYOUT_NHWC: return "LAYOUT_NHWC";
    case MLUOP_LAYOUT_HWCN: return "LAYOUT_HWCN";
    case MLUOP_LAYOUT_NDHWC: return "LAYOUT_NDHWC";
    case MLUOP_LAYOUT_ARRAY: return "LAYOUT_ARRAY";
    case MLUOP_LAYOUT_NCDHW: return "LAYOUT_NCDHW";
    case MLUOP_LAYOUT_TNC: return "LAYOUT_TNC";
    case MLUOP_LAYOUT_NTC: return "LAYOUT_NTC";
    case MLUOP_LAYOUT_NC: return "LAYOUT_NC";
    case MLUOP_LAYOUT_NLC: return "LAYOUT_NLC";
    case MLUOP_LAYOUT_NCL: return "LAYOUT_NCL";
  }
  return "LAYOUT_ARRAY";
}

bool isStrideTensor(int dim, const int64_t *dims, const int64_t *strides) {
  int64_t stride_base = 1;
  for (int i = dim - 1; i >= 0; --i) {
    if (dims[i] != 1 && strides[i] != stride_base) return true;
    stride_base *= dims[i];
  }
  return false;
}

int64_t dimN(const mluOpTensorStruct *d) {
  switch (d->layout) {
    case MLUOP_LAYOUT_NCHW:
    case MLUOP_LAYOUT_NHWC:
    case MLUOP_LAYOUT_NDHWC:
    case MLUOP_LAYOUT_NLC:
    case MLUOP_LAYOUT_NC:
    case MLUOP_LAYOUT_NCL:
    case MLUOP_LAYOUT_NCDHW:
      return d->dims[0];
    case MLUOP_LAYOUT_TNC:
      return d->dims[1];
    case MLUOP_LAYOUT_HWCN:
      return d->dims[3];
    default:
      return 0;
  }
}

int64_t dimD(const mluOpTensorStruct *d) {
  switch (d->layout) {
    case MLUOP_LAYOUT_NDHWC: return d->dims[1];
    case MLUOP_LAYOUT_NCDHW: return d->dims[2];
    default: return 0;
  }
}

int64_t dimC(const mluOpTensorStruct *d) {
  switch (d->layout) {
    case MLUOP_LAYOUT_NCHW:
    case MLUOP_LAYOUT_NCDHW:
    case MLUOP_LAYOUT_NC:
    case MLUOP_LAYOUT_NCL:
      return d->dims[1];
    case MLUOP_LAYOUT_HWCN:
    case MLUOP_LAYOUT_NLC:
    case MLUOP_LAYOUT_NTC:
    case MLUOP_LAYOUT_TNC:
      return d->dims[2];
    case MLUOP_LAYOUT_NHWC:
      return d->dims[3];
    case MLUOP_LAYOUT_NDHWC:
      return d->dims[4];
    default:
      return 0;
  }
}

int64_t dimH(const mluOpTensorStruct *d) {
  switch (d->layout) {
    case MLUOP_LAYOUT_HWCN: return d->dims[0];
    case MLUOP_LAYOUT_NHWC: return d->dims[1];
    case MLUOP_LAYOUT_NCHW:
    case MLUOP_LAYOUT_NDHWC: return d->dims[2];
    case MLUOP_LAYOUT_NCDHW: return d->dims[3];
    default: return 0;
  }
}

int64_t dimW(const mluOpTensorStruct *d) {
  switch (d->layout) {
    case MLUOP_LAYOUT_HWCN: return d->dims[1];
    case MLUOP_LAYOUT_NHWC: return d->dims[2];
    case MLUOP_LAYOUT_NCHW:
    case MLUOP_LAYOUT_NDHWC: return d->dims[3];
    case MLUOP_LAYOUT_NCDHW: return d->dims[4];
    default: return 0;
  }
}

}  // namespace mluop

namespace {

// Descriptors are created and destroyed around every operator call by typical
// callers, so released ones are kept on a free list (the reference recycles
// them through a locked queue as well, core/tensor.cpp:205-241).
class DescriptorPool {
 public:
  mluOpTensorStruct *acquire() {
    {
      std::lock_guard<std::mutex> g(mu_);
      if (!free_.empty()) {
        void *mem = free_.back();
        free_.pop_back();
        return ::new (mem) mluOpTensorStruct();
      }
    }
    void *mem = ::operator new(sizeof(mluOpTensorStruct), std::nothrow);
    if (mem == nullptr) return nullptr;
    return ::new (mem) mluOpTensorStruct();
  }
  void release(mluOpTensorStruct *d) {
    d->~mluOpTensorStruct();
    std::lock_guard<std::mutex> g(mu_);
    if (free_.size() < kMaxCached) {
      free_.push_back(d);
    } else {
      ::operator delete(static_cast<void *>(d));
    }
  }
  ~DescriptorPool() {
    for (void *p : free_) ::operator delete(p);
  }

 private:
  static constexpr size_t kMaxCached = 4096;
  std::mutex mu_;
  std::vector<void *> free_;
};

DescriptorPool &pool() {
  static DescriptorPool *p = new DescriptorPool();  // never destroyed: safe at exit
  return *p;
}

void setDimBase(mluOpTensorStruct *t, int dimNb) {
  if (dimNb != t->dim) {
    t->releaseDims();
    if (dimNb > MLUOP_DIM_MAX) {
      t->dims = new int64_t[dimNb];
      t->strides = new int64_t[dimNb];
    }
    t->dim = dimNb;
  }
}

mluOpStatus_t setZeroDim(mluOpTensorStruct *t) {
  if (t->pointer_mode == MLUOP_POINTER_MODE_HOST) {
    t->releaseDims();
    t->dim = 0;
    t->total_element_num = 1;
    t->total_tensor_size = mluop::getSizeOfDataType(t->dtype);
    return MLUOP_STATUS_SUCCESS;
  }
  MLUOP_LOG(ERROR) << "[mluOpSetTensorDescriptorDim]: the dim can be set to 0 only when the "
                   << "pointer mode of desc is MLUOP_POINTER_MODE_HOST.";
  return MLUOP_STATUS_BAD_PARAM;
}

template <typename IntT>
mluOpStatus_t setContiguous(mluOpTensorStruct *t, int dimNb, const IntT *dimSize) {
  setDimBase(t, dimNb);
  for (int i = 0; i < dimNb; ++i) t->dims[i] = static_cast<int64_t>(dimSize[i]);
  uint64_t stride_base = 1;
  for (int i = dimNb - 1; i >= 0; --i) {
    t->strides[i] = static_cast<int64_t>(stride_base);
    stride_base *= static_cast<uint64_t>(dimSize[i]);
  }
  t->total_element_num = stride_base;
  t->total_tensor_size = stride_base * mluop::getSizeOfDataType(t->dtype);
  return MLUOP_STATUS_SUCCESS;
}

template <typename IntT>
mluOpStatus_t setDescriptor(const char *api, mluOpTensorStruct *t, mluOpTensorLayout_t layout,
                            mluOpDataType_t dtype, int dimNb, const IntT *dimSize) {
  PARAM_CHECK(api, layout >= 0);
  PARAM_CHECK(api, dtype >= 0);
  t->dtype = dtype;
  t->layout = layout;
  if (dimNb == 0) return setZeroDim(t);
  PARAM_CHECK(api, dimNb > 0);
  PARAM_CHECK(api, dimSize != NULL);
  return setContiguous(t, dimNb, dimSize);
}

template <typename IntT>
mluOpStatus_t setDescriptorEx(const char *api, mluOpTensorStruct *t, mluOpTensorLayout_t layout,
                              mluOpDataType_t dtype, int dimNb, const IntT *dimSize,
                              const IntT *dimStride) {
  PARAM_CHECK(api, layout >= 0);
  PARAM_CHECK(api, dtype >= 0);
  t->dtype = dtype;
  t->layout = layout;
  if (dimNb == 0) return setZeroDim(t);
  PARAM_CHECK(api, dimSize != NULL);
  PARAM_CHECK(api, dimStride != NULL);
  PARAM_CHECK(api, dimNb > 0);
  setDimBase(t, dimNb);
  uint64_t total = 1;
  for (int i = 0; i < dimNb; ++i) {
    t->dims[i] = static_cast<int64_t>(dimSize[i]);
    t->strides[i] = static_cast<int64_t>(dimStride[i]);
    total *= static_cast<uint64_t>(dimSize[i]);
  }
  t->total_element_num = total;
  t->total_tensor_size = total * mluop::getSizeOfDataType(dtype);
  return MLUOP_STATUS_SUCCESS;
}

}  // namespace

extern "C" {

mluOpStatus_t MLUOP_WIN_API mluOpGetSizeOfDataType(mluOpDataType_t data_type, size_t *size) {
  PARAM_CHECK("[mluOpGetSizeOfDataType]", size != NULL);
  if (data_type != MLUOP_DTYPE_INVALID) {
    *size = mluop::getSizeOfDataType(data_type);
    return MLUOP_STATUS_SUCCESS;
  }
  MLUOP_LOG(ERROR) << "[mluOpGetSizeOfDataType]: data_type should not be MLUOP_DTYPE_INVALID.";
  return MLUOP_STATUS_BAD_PARAM;
}

mluOpStatus_t MLUOP_WIN_API mluOpCreateTensorDescriptor(mluOpTensorDescriptor_t *desc) {
  PARAM_CHECK("[mluOpCreateTensorDescriptor]", desc != NULL);
  mluOpTensorStruct *t = pool().acquire();
  if (t == nullptr) return MLUOP_STATUS_ALLOC_FAILED;
  *desc = t;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptor(mluOpTensorDescriptor_t desc,
                                                     mluOpTensorLayout_t layout,
                                                     mluOpDataType_t dtype, int dimNb,
                                                     const int dimSize[]) {
  PARAM_CHECK("[mluOpSetTensorDescriptor]", desc != NULL);
  return setDescriptor("[mluOpSetTensorDescriptor]", desc, layout, dtype, dimNb, dimSize);
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptor_v2(mluOpTensorDescriptor_t desc,
                                                        mluOpTensorLayout_t layout,
                                                        mluOpDataType_t dtype, int dimNb,
                                                        const int64_t dimSize[]) {
  PARAM_CHECK("[mluOpSetTensorDescriptor]", desc != NULL);
  return setDescriptor("[mluOpSetTensorDescriptor]", desc, layout, dtype, dimNb, dimSize);
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorEx(mluOpTensorDescriptor_t desc,
                                                       mluOpTensorLayout_t layout,
                                                       mluOpDataType_t dtype, int dimNb,
                                                       const int dimSize[],
                                                       const int dimStride[]) {
  PARAM_CHECK("[mluOpSetTensorDescriptorEx]", desc != NULL);
  return setDescriptorEx("[mluOpSetTensorDescriptorEx]", desc, layout, dtype, dimNb, dimSize,
                         dimStride);
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorEx_v2(mluOpTensorDescriptor_t desc,
                                                          mluOpTensorLayout_t layout,
                                                          mluOpDataType_t dtype, int dimNb,
                                                          const int64_t dimSize[],
                                                          const int64_t dimStride[]) {
  PARAM_CHECK("[mluOpSetTensorDescriptorEx]", desc != NULL);
  return setDescriptorEx("[mluOpSetTensorDescriptorEx]", desc, layout, dtype, dimNb, dimSize,
                         dimStride);
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorPointerMode(mluOpTensorDescriptor_t desc,
                                                                mluOpPointerMode_t pointer_mode) {
  PARAM_CHECK("[mluOpSetTensorDescriptorPointerMode]", desc != NULL);
  PARAM_CHECK("[mluOpSetTensorDescriptorPointerMode]", pointer_mode >= 0);
  desc->pointer_mode = pointer_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorPointerMode(mluOpTensorDescriptor_t desc,
                                                                mluOpPointerMode_t *pointer_mode) {
  PARAM_CHECK("[mluOpGetTensorDescriptorPointerMode]", desc != NULL);
  PARAM_CHECK("[mluOpGetTensorDescriptorPointerMode]", pointer_mode != NULL);
  *pointer_mode = desc->pointer_mode;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpSetTensorDescriptorOnchipDataType(mluOpTensorDescriptor_t desc,
                                                                   mluOpDataType_t onchip_dtype) {
  PARAM_CHECK("[mluOpSetTensorDescriptorOnchipDataType]", desc != NULL);
  desc->onchip_dtype = onchip_dtype;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorOnchipDataType(
    const mluOpTensorDescriptor_t desc, mluOpDataType_t *onchip_dtype) {
  PARAM_CHECK("[mluOpGetTensorDescriptorOnchipDataType]", desc != NULL);
  PARAM_CHECK("[mluOpGetTensorDescriptorOnchipDataType]", onchip_dtype != NULL);
  *onchip_dtype = desc->onchip_dtype;
  return MLUOP_STATUS_SUCCESS;
}

// The plain getters tolerate NULL output pointers and skip them (reference
// SET_PARAM_FOR_POINTER); the Ex getters require every pointer.
mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptor(const mluOpTensorDescriptor_t desc,
                                                     mluOpTensorLayout_t *layout,
                                                     mluOpDataType_t *dtype, int *dimNb,
                                                     int dimSize[]) {
  PARAM_CHECK("[mluOpGetTensorDescriptor]", desc != NULL);
  if (layout) *layout = desc->layout;
  if (dtype) *dtype = desc->dtype;
  if (dimNb) *dimNb = desc->dim;
  if (dimSize) {
    for (int i = 0; i < desc->dim; ++i) dimSize[i] = static_cast<int>(desc->dims[i]);
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptor_v2(const mluOpTensorDescriptor_t desc,
                                                        mluOpTensorLayout_t *layout,
                                                        mluOpDataType_t *dtype, int *dimNb,
                                                        int64_t dimSize[]) {
  PARAM_CHECK("[mluOpGetTensorDescriptor]", desc != NULL);
  if (layout) *layout = desc->layout;
  if (dtype) *dtype = desc->dtype;
  if (dimNb) *dimNb = desc->dim;
  if (dimSize) {
    for (int i = 0; i < desc->dim; ++i) dimSize[i] = desc->dims[i];
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorEx(const mluOpTensorDescriptor_t desc,
                                                       mluOpTensorLayout_t *layout,
                                                       mluOpDataType_t *dtype, int *dimNb,
                                                       int dimSize[], int dimStride[]) {
  const char *api = "[mluOpGetTensorDescriptorEx]";
  PARAM_CHECK(api, desc != NULL);
  PARAM_CHECK(api, layout != NULL);
  PARAM_CHECK(api, dtype != NULL);
  PARAM_CHECK(api, dimNb != NULL);
  PARAM_CHECK(api, dimSize != NULL);
  PARAM_CHECK(api, dimStride != NULL);
  *layout = desc->layout;
  *dtype = desc->dtype;
  *dimNb = desc->dim;
  for (int i = 0; i < desc->dim; ++i) {
    dimSize[i] = static_cast<int>(desc->dims[i]);
    dimStride[i] = static_cast<int>(desc->strides[i]);
  }
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpGetTensorDescriptorEx_v2(const mluOpTensorDescriptor_t desc,
                                                          mluOpTensorLayout_t *layout,
                                                          mluOpDataType_t *dtype, int *dimNb,
                                                          int64_t dimSize[],
                                                          int64_t dimStride[]) {
  const char *api = "[mluOpGetTensorDescriptorEx]";
  PARAM_CHECK(api, desc != NULL);
  PARAM_CHECK(api, layout != NULL);
  PARAM_CHECK(api, dtype != NULL);
  PARAM_CHECK(api, dimNb != NULL);
  PARAM_CHECK(api, dimSize != NULL);
  PARAM_CHECK(api, dimStride != NULL);
  *layout = desc->layout;
  *dtype = desc->dtype;
  *dimNb = desc->dim;
  for (int i = 0; i < desc->dim; ++i) {
    dimSize[i] = desc->dims[i];
    dimStride[i] = desc->strides[i];
  }
  return MLUOP_STATUS_SUCCESS;
}

size_t MLUOP_WIN_API mluOpGetTensorElementNum(const mluOpTensorDescriptor_t desc) {
  // The reference aborts on NULL here (CHECK); returning 0 keeps the process alive.
  if (desc == NULL) {
    MLUOP_LOG(ERROR) << "[mluOpGetTensorElementNum] desc is NULL.";
    return 0;
  }
  return static_cast<size_t>(desc->total_element_num);
}

mluOpStatus_t MLUOP_WIN_API mluOpResetTensorDescriptor(mluOpTensorDescriptor_t desc) {
  PARAM_CHECK("[mluOpResetTensorDescriptor]", desc != NULL);
  desc->releaseDims();
  desc->dim = 0;
  desc->dtype = MLUOP_DTYPE_FLOAT;
  desc->onchip_dtype = MLUOP_DTYPE_INVALID;
  desc->layout = MLUOP_LAYOUT_ARRAY;
  desc->pointer_mode = MLUOP_POINTER_MODE_DEVICE;
  desc->total_element_num = 0;
  desc->total_tensor_size = 0;
  return MLUOP_STATUS_SUCCESS;
}

mluOpStatus_t MLUOP_WIN_API mluOpDestroyTensorDescriptor(mluOpTensorDescriptor_t desc) {
  PARAM_CHECK("[mluOpDestroyTensorDescriptor]", desc != NULL);
  pool().release(desc);
  return MLUOP_STATUS_SUCCESS;
}

}  // extern "C"
