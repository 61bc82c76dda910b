// Glue between TensorFlow tensors and the C ABI of libatex_norms_hip.so (include/atex_norms.h),
// shared by the OpKernels of norm_kernels_rocm.cc and the functor specialisations of
// fused_norm_functors_rocm.cc.  Header-only.
#ifndef ATEXN_TF_GLUE_H_
#define ATEXN_TF_GLUE_H_

#include <cstdint>

#include "atex_norms.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/tensor.h"
#include "tensorflow/core/framework/tensor_shape.h"
#include "tensorflow/core/framework/types.h"

namespace tensorflow {
namespace atexn_glue {

template <typename T> struct DtypeCode;
template <> struct DtypeCode<float> { static constexpr int value = ATEXN_F32; };
template <> struct DtypeCode<Eigen::half> { static constexpr int value = ATEXN_F16; };
template <> struct DtypeCode<bfloat16> { static constexpr int value = ATEXN_BF16; };

inline int DtypeOf(const Tensor& t) {
  switch (t.dtype()) {
    case DT_HALF: return ATEXN_F16;
    case DT_BFLOAT16: return ATEXN_BF16;
    default: return ATEXN_F32;
  }
}

// The library's status codes as TensorFlow statuses: an argument error keeps the library's
// message (the texts of the reference's OP_REQUIRES checks), anything else is Internal.
inline Status ToStatus(int st) {
  if (st == ATEXN_OK) return OkStatus();
  if (st == ATEXN_INVALID_ARGUMENT) return errors::InvalidArgument(atexn_last_error());
  return errors::Internal(atexn_last_error());
}

// Descriptor of a tensor as the op-level entry points take it.  `device`: ATEXN_DEVICE_GPU or
// ATEXN_DEVICE_CPU, from the kernel's registration.
inline Status Describe(const Tensor& t, int device, atexn_tensor* out) {
  if (t.dims() > ATEXN_MAX_RANK) {
    return errors::InvalidArgument("tensors of rank ", t.dims(), " are not supported (limit ",
                                   ATEXN_MAX_RANK, ")");
  }
  out->dtype = DtypeOf(t);
  out->rank = t.dims();
  for (int i = 0; i < t.dims(); ++i) out->dims[i] = t.dim_size(i);
  out->data = t.NumElements() == 0 ? nullptr : const_cast<char*>(t.tensor_data().data());
  out->device = device;
  return OkStatus();
}

// Scratch for one call, from the framework's allocator (the counterpart of the reference's
// allocate_temp calls, fused_layer_norm_op.cu:853-867).  The library wants 256-byte alignment,
// so the buffer is over-allocated and the pointer rounded up.
class Workspace {
 public:
  Status Allocate(OpKernelContext* ctx, size_t need) {
    bytes_ = need;
    if (need == 0) return OkStatus();
    TF_RETURN_IF_ERROR(
        ctx->allocate_temp(DT_UINT8, TensorShape({static_cast<int64_t>(need + 255)}), &buffer_));
    const uintptr_t p = reinterpret_cast<uintptr_t>(buffer_.tensor_data().data());
    ptr_ = reinterpret_cast<void*>((p + 255) & ~static_cast<uintptr_t>(255));
    return OkStatus();
  }
  void* ptr() const { return ptr_; }
  size_t bytes() const { return bytes_; }

 private:
  Tensor buffer_;
  void* ptr_ = nullptr;
  size_t bytes_ = 0;
};

}  // namespace atexn_glue
}  // namespace tensorflow

#endif  // ATEXN_TF_GLUE_H_
