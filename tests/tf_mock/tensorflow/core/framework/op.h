// NOT TensorFlow: see mock_core.h.  REGISTER_OP and its builder.
#ifndef ATEXN_TF_MOCK_OP_H_
#define ATEXN_TF_MOCK_OP_H_

#include "tensorflow/core/framework/mock_core.h"

namespace tensorflow {
namespace shape_inference {
class InferenceContext;
}
class OpDefBuilderWrapper {
 public:
  explicit OpDefBuilderWrapper(const char* name);
  OpDefBuilderWrapper& Input(std::string spec);
  OpDefBuilderWrapper& Output(std::string spec);
  OpDefBuilderWrapper& Attr(std::string spec);
  OpDefBuilderWrapper& SetShapeFn(Status (*fn)(shape_inference::InferenceContext*));
};
#define ATEXN_MOCK_OP_CONCAT_(a, b) a##b
#define ATEXN_MOCK_OP_CONCAT(a, b) ATEXN_MOCK_OP_CONCAT_(a, b)
#define REGISTER_OP(name) \
  static ::tensorflow::OpDefBuilderWrapper& ATEXN_MOCK_OP_CONCAT(mock_op_, __COUNTER__) = ::tensorflow::OpDefBuilderWrapper(name)
}  // namespace tensorflow

#endif  // ATEXN_TF_MOCK_OP_H_
