// NOT TensorFlow: see mock_core.h.  OpKernel, its two contexts and the kernel registration macro.
#ifndef ATEXN_TF_MOCK_OP_KERNEL_H_
#define ATEXN_TF_MOCK_OP_KERNEL_H_

#include "tensorflow/core/framework/mock_core.h"

namespace tensorflow {

class OpKernelConstruction {
 public:
  template <typename T> Status GetAttr(StringPiece name, T* value) const;
  void CtxFailure(const char* file, int line, const Status& s);
};

class OpKernelContext {
 public:
  const Tensor& input(int index) const;
  Status allocate_output(int index, const TensorShape& shape, Tensor** tensor);
  Status forward_input_or_allocate_output(std::initializer_list<int> candidate_input_indices, int output_index,
                                          const TensorShape& output_shape, Tensor** output,
                                          int* forwarded_input = nullptr);
  Status allocate_temp(DataType type, const TensorShape& shape, Tensor* out_temp);
  template <typename Device> const Device& eigen_device() const;
  void CtxFailure(const char* file, int line, const Status& s);
};

class OpKernel {
 public:
  explicit OpKernel(OpKernelConstruction* context);
  virtual ~OpKernel();
  virtual void Compute(OpKernelContext* context) = 0;
};

#define OP_REQUIRES_OK(CTX, ...)                          \
  do {                                                    \
    ::tensorflow::Status s_(__VA_ARGS__);                 \
    if (!s_.ok()) {                                       \
      (CTX)->CtxFailure(__FILE__, __LINE__, s_);          \
      return;                                             \
    }                                                     \
  } while (0)

#define OP_REQUIRES(CTX, EXP, STATUS)                     \
  do {                                                    \
    if (!(EXP)) {                                         \
      (CTX)->CtxFailure(__FILE__, __LINE__, (STATUS));    \
      return;                                             \
    }                                                     \
  } while (0)

class KernelDefBuilder {
 public:
  explicit KernelDefBuilder(const char* op_name);
  KernelDefBuilder& Device(const char* device_type);
  template <typename T> KernelDefBuilder& TypeConstraint(const char* attr_name);
};
typedef KernelDefBuilder Name;

namespace mock_registration {
template <typename K>
struct KernelRegistrar {
  explicit KernelRegistrar(const KernelDefBuilder&) { static_assert(sizeof(K) > 0, "kernel class must be complete"); (void)sizeof(&K::Compute); }
};
}  // namespace mock_registration

#define ATEXN_MOCK_CONCAT_(a, b) a##b
#define ATEXN_MOCK_CONCAT(a, b) ATEXN_MOCK_CONCAT_(a, b)
// (instantiates the kernel class, so its Compute body is type-checked)
#define REGISTER_KERNEL_BUILDER(kernel_builder, ...)                                                     \
  template class __VA_ARGS__;                                                                            \
  static ::tensorflow::mock_registration::KernelRegistrar<__VA_ARGS__> ATEXN_MOCK_CONCAT(mock_kernel_, __COUNTER__)( \
      ::tensorflow::kernel_builder)

}  // namespace tensorflow

#endif  // ATEXN_TF_MOCK_OP_KERNEL_H_
