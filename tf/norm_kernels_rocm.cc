// OpKernels of FusedLayerNorm[Grad] / FusedInstanceNorm[Grad] for TensorFlow-ROCm on top of
// libatex_norms_hip.so.  They take the place of the reference's OpKernels and device functors
// (atex/nv_norms/cc/kernels/fused_layer_norm_op.cc:285-484, fused_instance_norm_op.cc:311-560,
// and the .cu files behind them).
//
// A Compute body only does what needs the framework: it allocates the outputs (forwarding x
// onto y where the reference does, fused_layer_norm_op.cc:337, fused_instance_norm_op.cc:390),
// asks the library for its scratch size and allocates that, describes every tensor and calls
// the op-level entry point.  Axis packing, data-format parsing, flattening and every shape
// check happen inside atexn_fused_*, which reports them as INVALID_ARGUMENT with the
// reference's message texts before anything is launched.
//
// One class serves the CPU and the GPU registration: the descriptors carry the device, the
// library picks its host or its HIP kernels by it.
#include <string>
#include <vector>

#include "atex_norms.h"
#include "atexn_tf_glue.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/register_types.h"
#include "tensorflow/core/framework/tensor.h"

namespace tensorflow {

typedef Eigen::ThreadPoolDevice CPUDevice;
typedef Eigen::GpuDevice GPUDevice;

namespace {

using atexn_glue::Describe;
using atexn_glue::ToStatus;
using atexn_glue::Workspace;

template <typename Device> struct DeviceTraits;
template <> struct DeviceTraits<CPUDevice> {
  static constexpr int kind = ATEXN_DEVICE_CPU;
  static void* Stream(OpKernelContext*) { return nullptr; }
};
template <> struct DeviceTraits<GPUDevice> {
  static constexpr int kind = ATEXN_DEVICE_GPU;
  // gpuStream_t is hipStream_t under TensorFlow-ROCm; the library takes it as void*
  static void* Stream(OpKernelContext* ctx) {
    return reinterpret_cast<void*>(ctx->eigen_device<GPUDevice>().stream());
  }
};

// N and D of x under the op's axis list, for sizing the statistics outputs.
Status LayerNormSizes(const Tensor& x, const std::vector<int>& axis, int64_t* n, int64_t* d) {
  if (x.dims() < 1 || x.dims() > ATEXN_MAX_RANK) {
    return errors::InvalidArgument("input must be at least 1-dimensional", x.shape().DebugString());
  }
  int64_t dims[ATEXN_MAX_RANK];
  for (int i = 0; i < x.dims(); ++i) dims[i] = x.dim_size(i);
  return ToStatus(atexn_layer_norm_resolve_axes(x.dims(), dims, axis.data(),
                                                static_cast<int>(axis.size()), n, d));
}

Status InstanceNormSizes(const Tensor& x, const std::string& data_format, int64_t* n, int64_t* c) {
  if (x.dims() < 4 || x.dims() > ATEXN_MAX_RANK) {
    return errors::InvalidArgument("input must be at least 4-dimensional", x.shape().DebugString());
  }
  int64_t dims[ATEXN_MAX_RANK];
  for (int i = 0; i < x.dims(); ++i) dims[i] = x.dim_size(i);
  int layout = 0;
  int64_t d = 0;
  return ToStatus(atexn_instance_norm_resolve_format(x.dims(), dims, data_format.c_str(), &layout, n, c, &d));
}

}  // namespace

template <typename Device, typename T>
class FusedLayerNormOp : public OpKernel {
 public:
  explicit FusedLayerNormOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("epsilon", &epsilon_));
    OP_REQUIRES_OK(ctx, ctx->GetAttr("axis", &axis_));
  }

  void Compute(OpKernelContext* ctx) override {
    const Tensor& x = ctx->input(0);
    const Tensor& scale = ctx->input(1);
    const Tensor& offset = ctx->input(2);
    int64_t n = 0, d = 0;
    OP_REQUIRES_OK(ctx, LayerNormSizes(x, axis_, &n, &d));
    Tensor* y = nullptr;
    OP_REQUIRES_OK(ctx, ctx->forward_input_or_allocate_output({0}, 0, x.shape(), &y));
    Tensor* mean = nullptr;
    Tensor* inv_std = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, TensorShape({n}), &mean));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, TensorShape({n}), &inv_std));

    constexpr int dev = DeviceTraits<Device>::kind;
    atexn_tensor tx, ts, to, ty, tm, tr;
    OP_REQUIRES_OK(ctx, Describe(x, dev, &tx));
    OP_REQUIRES_OK(ctx, Describe(scale, dev, &ts));
    OP_REQUIRES_OK(ctx, Describe(offset, dev, &to));
    OP_REQUIRES_OK(ctx, Describe(*y, dev, &ty));
    OP_REQUIRES_OK(ctx, Describe(*mean, dev, &tm));
    OP_REQUIRES_OK(ctx, Describe(*inv_std, dev, &tr));
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_fused_layer_norm_workspace_bytes(
                                             &tx, axis_.data(), static_cast<int>(axis_.size()))));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_fused_layer_norm(
                            &tx, &ts, &to, epsilon_, axis_.data(), static_cast<int>(axis_.size()), &ty,
                            &tm, &tr, ws.ptr(), ws.bytes(), DeviceTraits<Device>::Stream(ctx))));
  }

 private:
  float epsilon_;
  std::vector<int> axis_;
};

template <typename Device, typename T>
class FusedLayerNormGradOp : public OpKernel {
 public:
  explicit FusedLayerNormGradOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("axis", &axis_));  // epsilon plays no part in the gradient
  }

  void Compute(OpKernelContext* ctx) override {
    const Tensor& dy = ctx->input(0);
    const Tensor& x = ctx->input(1);
    const Tensor& scale = ctx->input(2);
    const Tensor& mean = ctx->input(3);
    const Tensor& inv_std = ctx->input(4);
    int64_t n = 0, d = 0;
    OP_REQUIRES_OK(ctx, LayerNormSizes(x, axis_, &n, &d));
    // dgamma / dbeta leave in the shape gamma came in (fused_layer_norm_op.cc:451-457)
    Tensor* dx = nullptr;
    Tensor* dscale = nullptr;
    Tensor* doffset = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, x.shape(), &dx));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, scale.shape(), &dscale));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, scale.shape(), &doffset));

    constexpr int dev = DeviceTraits<Device>::kind;
    atexn_tensor tdy, tx, ts, tm, tr, tdx, tds, tdo;
    OP_REQUIRES_OK(ctx, Describe(dy, dev, &tdy));
    OP_REQUIRES_OK(ctx, Describe(x, dev, &tx));
    OP_REQUIRES_OK(ctx, Describe(scale, dev, &ts));
    OP_REQUIRES_OK(ctx, Describe(mean, dev, &tm));
    OP_REQUIRES_OK(ctx, Describe(inv_std, dev, &tr));
    OP_REQUIRES_OK(ctx, Describe(*dx, dev, &tdx));
    OP_REQUIRES_OK(ctx, Describe(*dscale, dev, &tds));
    OP_REQUIRES_OK(ctx, Describe(*doffset, dev, &tdo));
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_fused_layer_norm_grad_workspace_bytes(
                                             &tx, axis_.data(), static_cast<int>(axis_.size()))));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_fused_layer_norm_grad(
                            &tdy, &tx, &ts, &tm, &tr, axis_.data(), static_cast<int>(axis_.size()), &tdx,
                            &tds, &tdo, ws.ptr(), ws.bytes(), DeviceTraits<Device>::Stream(ctx))));
  }

 private:
  std::vector<int> axis_;
};

template <typename Device, typename T>
class FusedInstanceNormOp : public OpKernel {
 public:
  explicit FusedInstanceNormOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("epsilon", &epsilon_));
    OP_REQUIRES_OK(ctx, ctx->GetAttr("data_format", &data_format_));
  }

  void Compute(OpKernelContext* ctx) override {
    const Tensor& x = ctx->input(0);
    const Tensor& scale = ctx->input(1);
    const Tensor& offset = ctx->input(2);
    int64_t n = 0, c = 0;
    OP_REQUIRES_OK(ctx, InstanceNormSizes(x, data_format_, &n, &c));
    Tensor* y = nullptr;
    OP_REQUIRES_OK(ctx, ctx->forward_input_or_allocate_output({0}, 0, x.shape(), &y));
    Tensor* mean = nullptr;
    Tensor* inv_std = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, TensorShape({n, c}), &mean));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, TensorShape({n, c}), &inv_std));

    constexpr int dev = DeviceTraits<Device>::kind;
    atexn_tensor tx, ts, to, ty, tm, tr;
    OP_REQUIRES_OK(ctx, Describe(x, dev, &tx));
    OP_REQUIRES_OK(ctx, Describe(scale, dev, &ts));
    OP_REQUIRES_OK(ctx, Describe(offset, dev, &to));
    OP_REQUIRES_OK(ctx, Describe(*y, dev, &ty));
    OP_REQUIRES_OK(ctx, Describe(*mean, dev, &tm));
    OP_REQUIRES_OK(ctx, Describe(*inv_std, dev, &tr));
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_fused_instance_norm_workspace_bytes(&tx, data_format_.c_str())));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_fused_instance_norm(&tx, &ts, &to, epsilon_, data_format_.c_str(), &ty,
                                                           &tm, &tr, ws.ptr(), ws.bytes(),
                                                           DeviceTraits<Device>::Stream(ctx))));
  }

 private:
  float epsilon_;
  std::string data_format_;
};

template <typename Device, typename T>
class FusedInstanceNormGradOp : public OpKernel {
 public:
  explicit FusedInstanceNormGradOp(OpKernelConstruction* ctx) : OpKernel(ctx) {
    OP_REQUIRES_OK(ctx, ctx->GetAttr("data_format", &data_format_));
  }

  void Compute(OpKernelContext* ctx) override {
    const Tensor& dy = ctx->input(0);
    const Tensor& x = ctx->input(1);
    const Tensor& scale = ctx->input(2);
    const Tensor& mean = ctx->input(3);
    const Tensor& inv_std = ctx->input(4);
    int64_t n = 0, c = 0;
    OP_REQUIRES_OK(ctx, InstanceNormSizes(x, data_format_, &n, &c));
    Tensor* dx = nullptr;
    Tensor* dscale = nullptr;
    Tensor* doffset = nullptr;
    OP_REQUIRES_OK(ctx, ctx->allocate_output(0, x.shape(), &dx));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(1, TensorShape({c}), &dscale));
    OP_REQUIRES_OK(ctx, ctx->allocate_output(2, TensorShape({c}), &doffset));

    constexpr int dev = DeviceTraits<Device>::kind;
    atexn_tensor tdy, tx, ts, tm, tr, tdx, tds, tdo;
    OP_REQUIRES_OK(ctx, Describe(dy, dev, &tdy));
    OP_REQUIRES_OK(ctx, Describe(x, dev, &tx));
    OP_REQUIRES_OK(ctx, Describe(scale, dev, &ts));
    OP_REQUIRES_OK(ctx, Describe(mean, dev, &tm));
    OP_REQUIRES_OK(ctx, Describe(inv_std, dev, &tr));
    OP_REQUIRES_OK(ctx, Describe(*dx, dev, &tdx));
    OP_REQUIRES_OK(ctx, Describe(*dscale, dev, &tds));
    OP_REQUIRES_OK(ctx, Describe(*doffset, dev, &tdo));
    Workspace ws;
    OP_REQUIRES_OK(ctx, ws.Allocate(ctx, atexn_fused_instance_norm_grad_workspace_bytes(&tx, data_format_.c_str())));
    OP_REQUIRES_OK(ctx, ToStatus(atexn_fused_instance_norm_grad(&tdy, &tx, &ts, &tm, &tr, data_format_.c_str(),
                                                                &tdx, &tds, &tdo, ws.ptr(), ws.bytes(),
                                                                DeviceTraits<Device>::Stream(ctx))));
  }

 private:
  std::string data_format_;
};

#define ATEXN_REGISTER(D, T)                                                                       \
  REGISTER_KERNEL_BUILDER(                                                                         \
      Name("FusedLayerNorm").Device(DEVICE_##D).TypeConstraint<T>("T").TypeConstraint<float>("U"), \
      FusedLayerNormOp<D##Device, T>);                                                             \
  REGISTER_KERNEL_BUILDER(Name("FusedLayerNormGrad")                                               \
                              .Device(DEVICE_##D)                                                  \
                              .TypeConstraint<T>("T")                                              \
                              .TypeConstraint<float>("U"),                                         \
                          FusedLayerNormGradOp<D##Device, T>);                                     \
  REGISTER_KERNEL_BUILDER(Name("FusedInstanceNorm")                                                \
                              .Device(DEVICE_##D)                                                  \
                              .TypeConstraint<T>("T")                                              \
                              .TypeConstraint<float>("U"),                                         \
                          FusedInstanceNormOp<D##Device, T>);                                      \
  REGISTER_KERNEL_BUILDER(Name("FusedInstanceNormGrad")                                            \
                              .Device(DEVICE_##D)                                                  \
                              .TypeConstraint<T>("T")                                              \
                              .TypeConstraint<float>("U"),                                         \
                          FusedInstanceNormGradOp<D##Device, T>);

ATEXN_REGISTER(CPU, float)
ATEXN_REGISTER(CPU, Eigen::half)
ATEXN_REGISTER(CPU, bfloat16)
ATEXN_REGISTER(GPU, float)
ATEXN_REGISTER(GPU, Eigen::half)
ATEXN_REGISTER(GPU, bfloat16)
#undef ATEXN_REGISTER

}  // namespace tensorflow
