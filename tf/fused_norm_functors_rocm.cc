// Second way of putting the library under the reference's ops: keep the reference's own
// OpKernels (fused_layer_norm_op.cc, fused_instance_norm_op.cc) and op registrations, drop its
// two .cu files from the build, and compile this file instead.  It defines the four GPU functor
// specialisations those OpKernels call -- the symbols declared there by DECLARE_GPU_SPEC
// (fused_layer_norm_op.cc:227-246, fused_instance_norm_op.cc:286-305) -- as calls into the
// kernel-level C ABI.  Not used together with norm_kernels_rocm.cc, which replaces the
// OpKernels as well.
//
// The primary templates are only forward-declared here; their definitions live in the
// reference's headers (fused_layer_norm_op.h:12-29, fused_instance_norm_op.h:12-29), which the
// OpKernel translation units include.  Argument meaning, taken from the call sites:
//   LayerNorm     x arrives flattened to [N, D]; batch_dim / feature_dim are the INDICES 0 and 1
//                 of those dimensions (fused_layer_norm_op.cc:333-334), sizes come from
//                 dim_size(...) (fused_layer_norm_op.cu:814-815);
//   InstanceNorm  x arrives as [N, C, D] (is_channel_first) or [N, D, C]
//                 (fused_instance_norm_op.cc:363-373).
// With -DATEXN_TF_CPU_FUNCTORS the CPU specialisations are defined too (host kernels of the
// library, atexn_*_cpu); the reference's Eigen functors (fused_layer_norm_op.cc:27-223,
// fused_instance_norm_op.cc:39-284) must then be taken out of its .cc files.
#include "atex_norms.h"
#include "atexn_tf_glue.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/tensor.h"

namespace tensorflow {

typedef Eigen::ThreadPoolDevice CPUDevice;
typedef Eigen::GpuDevice GPUDevice;

namespace functor {

template <typename Device, typename T, typename U> struct FusedLayerNorm;
template <typename Device, typename T, typename U> struct FusedLayerNormGrad;
template <typename Device, typename T, typename U> struct FusedInstanceNorm;
template <typename Device, typename T, typename U> struct FusedInstanceNormGrad;

using atexn_glue::DtypeCode;
using atexn_glue::ToStatus;
using atexn_glue::Workspace;

namespace {
inline void* StreamOf(OpKernelContext* ctx) {
  return reinterpret_cast<void*>(ctx->eigen_device<GPUDevice>().stream());
}
struct InstanceView {
  int layout;
  int64_t N, C, D;
  InstanceView(const Tensor& x, bool channel_first)
      : layout(channel_first ? ATEXN_LAYOUT_NC_ : ATEXN_LAYOUT_N_C),
        N(x.dim_size(0)),
        C(x.dim_size(channel_first ? 1 : 2)),
        D(x.dim_size(channel_first ? 2 : 1)) {}
};
}  // namespace

template <typename T, typename U>
struct FusedLayerNorm<GPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& x, const Tensor& scale, const Tensor& offset,
                  U epsilon, int batch_dim, int feature_dim, Tensor* y, Tensor* saved_mean,
                  Tensor* saved_inv_var) {
    if (x.NumElements() == 0) return;
    const int64_t N = x.dim_size(batch_dim);
    const int64_t D = x.dim_size(feature_dim);
    const int dt = DtypeCode<T>::value;
    Workspace ws;  // 0 bytes for rows that fit in registers
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_layer_norm_fwd_workspace_bytes(dt, N, D)));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_layer_norm_fwd(
                            dt, x.flat<T>().data(), scale.flat<U>().data(), offset.flat<U>().data(), N, D,
                            epsilon, y->flat<T>().data(), saved_mean->flat<U>().data(),
                            saved_inv_var->flat<U>().data(), ws.ptr(), ws.bytes(), StreamOf(ctx))));
  }
};

template <typename T, typename U>
struct FusedLayerNormGrad<GPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& y_backprop, const Tensor& x, const Tensor& scale,
                  const Tensor& saved_mean, const Tensor& saved_inv_var, U /*epsilon*/, int batch_dim,
                  int feature_dim, Tensor* x_backprop, Tensor* scale_backprop, Tensor* offset_backprop) {
    const int64_t N = x.dim_size(batch_dim);
    const int64_t D = x.dim_size(feature_dim);
    const int dt = DtypeCode<T>::value;
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_layer_norm_bwd_workspace_bytes(dt, N, D)));
    // an empty x: the library zero-fills scale_backprop / offset_backprop and launches nothing else
    OP_REQUIRES_OK(ctx, ToStatus(atexn_layer_norm_bwd(
                            dt, y_backprop.flat<T>().data(), x.flat<T>().data(), scale.flat<U>().data(),
                            saved_mean.flat<U>().data(), saved_inv_var.flat<U>().data(), N, D,
                            x_backprop->flat<T>().data(), scale_backprop->flat<U>().data(),
                            offset_backprop->flat<U>().data(), ws.ptr(), ws.bytes(), StreamOf(ctx))));
  }
};

template <typename T, typename U>
struct FusedInstanceNorm<GPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& x, const Tensor& scale, const Tensor& offset,
                  U epsilon, bool is_channel_first, Tensor* y, Tensor* saved_mean,
                  Tensor* saved_inv_var) {
    if (x.NumElements() == 0) return;
    const InstanceView v(x, is_channel_first);
    const int dt = DtypeCode<T>::value;
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_instance_norm_fwd_workspace_bytes(dt, v.layout, v.N, v.C, v.D)));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_instance_norm_fwd(
                            dt, v.layout, x.flat<T>().data(), scale.flat<U>().data(), offset.flat<U>().data(),
                            v.N, v.C, v.D, epsilon, y->flat<T>().data(), saved_mean->flat<U>().data(),
                            saved_inv_var->flat<U>().data(), ws.ptr(), ws.bytes(), StreamOf(ctx))));
  }
};

template <typename T, typename U>
struct FusedInstanceNormGrad<GPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& y_backprop, const Tensor& x, const Tensor& scale,
                  const Tensor& saved_mean, const Tensor& saved_inv_var, U /*epsilon*/, bool is_channel_first,
                  Tensor* x_backprop, Tensor* scale_backprop, Tensor* offset_backprop) {
    const InstanceView v(x, is_channel_first);
    const int dt = DtypeCode<T>::value;
    // one workspace stands for the functor's two [N * C] temporaries
    // (fused_instance_norm_op.cu:1546-1554) and every allocate_temp of the drivers it calls
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_instance_norm_bwd_workspace_bytes(dt, v.layout, v.N, v.C, v.D)));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_instance_norm_bwd(
                            dt, v.layout, y_backprop.flat<T>().data(), x.flat<T>().data(), scale.flat<U>().data(),
                            saved_mean.flat<U>().data(), saved_inv_var.flat<U>().data(), v.N, v.C, v.D,
                            x_backprop->flat<T>().data(), scale_backprop->flat<U>().data(),
                            offset_backprop->flat<U>().data(), ws.ptr(), ws.bytes(), StreamOf(ctx))));
  }
};

#define ATEXN_INSTANTIATE(D, T)                          \
  template struct FusedLayerNorm<D, T, float>;           \
  template struct FusedLayerNormGrad<D, T, float>;       \
  template struct FusedInstanceNorm<D, T, float>;        \
  template struct FusedInstanceNormGrad<D, T, float>;
ATEXN_INSTANTIATE(GPUDevice, float)
ATEXN_INSTANTIATE(GPUDevice, Eigen::half)
ATEXN_INSTANTIATE(GPUDevice, bfloat16)  // with bfloat16 added to T in the op and kernel registrations

#ifdef ATEXN_TF_CPU_FUNCTORS
template <typename T, typename U>
struct FusedLayerNorm<CPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& x, const Tensor& scale, const Tensor& offset,
                  U epsilon, int batch_dim, int feature_dim, Tensor* y, Tensor* saved_mean,
                  Tensor* saved_inv_var) {
    OP_REQUIRES_OK(ctx, ToStatus(atexn_layer_norm_fwd_cpu(
                            DtypeCode<T>::value, x.flat<T>().data(), scale.flat<U>().data(),
                            offset.flat<U>().data(), x.dim_size(batch_dim), x.dim_size(feature_dim), epsilon,
                            y->flat<T>().data(), saved_mean->flat<U>().data(),
                            saved_inv_var->flat<U>().data())));
  }
};

template <typename T, typename U>
struct FusedLayerNormGrad<CPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& y_backprop, const Tensor& x, const Tensor& scale,
                  const Tensor& saved_mean, const Tensor& saved_inv_var, U /*epsilon*/, int batch_dim,
                  int feature_dim, Tensor* x_backprop, Tensor* scale_backprop, Tensor* offset_backprop) {
    OP_REQUIRES_OK(ctx, ToStatus(atexn_layer_norm_bwd_cpu(
                            DtypeCode<T>::value, y_backprop.flat<T>().data(), x.flat<T>().data(),
                            scale.flat<U>().data(), saved_mean.flat<U>().data(), saved_inv_var.flat<U>().data(),
                            x.dim_size(batch_dim), x.dim_size(feature_dim), x_backprop->flat<T>().data(),
                            scale_backprop->flat<U>().data(), offset_backprop->flat<U>().data())));
  }
};

template <typename T, typename U>
struct FusedInstanceNorm<CPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& x, const Tensor& scale, const Tensor& offset,
                  U epsilon, bool is_channel_first, Tensor* y, Tensor* saved_mean,
                  Tensor* saved_inv_var) {
    const InstanceView v(x, is_channel_first);
    OP_REQUIRES_OK(ctx, ToStatus(atexn_instance_norm_fwd_cpu(
                            DtypeCode<T>::value, v.layout, x.flat<T>().data(), scale.flat<U>().data(),
                            offset.flat<U>().data(), v.N, v.C, v.D, epsilon, y->flat<T>().data(),
                            saved_mean->flat<U>().data(), saved_inv_var->flat<U>().data())));
  }
};

template <typename T, typename U>
struct FusedInstanceNormGrad<CPUDevice, T, U> {
  void operator()(OpKernelContext* ctx, const Tensor& y_backprop, const Tensor& x, const Tensor& scale,
                  const Tensor& saved_mean, const Tensor& saved_inv_var, U /*epsilon*/, bool is_channel_first,
                  Tensor* x_backprop, Tensor* scale_backprop, Tensor* offset_backprop) {
    const InstanceView v(x, is_channel_first);
    OP_REQUIRES_OK(ctx, ToStatus(atexn_instance_norm_bwd_cpu(
                            DtypeCode<T>::value, v.layout, y_backprop.flat<T>().data(), x.flat<T>().data(),
                            scale.flat<U>().data(), saved_mean.flat<U>().data(), saved_inv_var.flat<U>().data(),
                            v.N, v.C, v.D, x_backprop->flat<T>().data(), scale_backprop->flat<U>().data(),
                            offset_backprop->flat<U>().data())));
  }
};

ATEXN_INSTANTIATE(CPUDevice, float)
ATEXN_INSTANTIATE(CPUDevice, Eigen::half)
ATEXN_INSTANTIATE(CPUDevice, bfloat16)
#endif  // ATEXN_TF_CPU_FUNCTORS
#undef ATEXN_INSTANTIATE

}  // namespace functor
}  // namespace tensorflow
