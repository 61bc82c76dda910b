// NOT TensorFlow: see mock_core.h.  The part of shape_inference::InferenceContext that shape
// functions use.
#ifndef ATEXN_TF_MOCK_SHAPE_INFERENCE_H_
#define ATEXN_TF_MOCK_SHAPE_INFERENCE_H_

#include "tensorflow/core/framework/mock_core.h"

namespace tensorflow {
namespace shape_inference {

class DimensionHandle {};
class ShapeHandle {};
struct DimensionOrConstant {
  DimensionOrConstant(DimensionHandle dim);
  DimensionOrConstant(int64_t val);
};

class InferenceContext {
 public:
  ShapeHandle input(int64_t idx) const;
  void set_output(int idx, ShapeHandle shape);
  bool RankKnown(ShapeHandle s) const;
  int32_t Rank(ShapeHandle s) const;
  DimensionHandle Dim(ShapeHandle s, int64_t idx);
  bool ValueKnown(DimensionOrConstant d) const;
  int64_t Value(DimensionOrConstant d) const;
  DimensionHandle MakeDim(DimensionOrConstant d);
  DimensionHandle UnknownDim();
  ShapeHandle Vector(DimensionOrConstant dim);
  ShapeHandle MakeShape(std::initializer_list<DimensionOrConstant> dims);
  Status WithRankAtLeast(ShapeHandle shape, int64_t rank, ShapeHandle* out);
  template <typename T> Status GetAttr(StringPiece attr_name, T* value) const;
};

}  // namespace shape_inference
}  // namespace tensorflow

#endif  // ATEXN_TF_MOCK_SHAPE_INFERENCE_H_
