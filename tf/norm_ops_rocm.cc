// Op registrations of the four fused normalisation ops for the ROCm build: same op names,
// inputs, outputs, attributes and defaults as the reference registers
// (atex/nv_norms/cc/ops/norm_ops.cc:148-202), with bfloat16 added to T.
//
// The shape functions do not repeat the axis / data-format rules: they hand the known
// dimensions to the library's own resolvers (atexn_layer_norm_resolve_axes,
// atexn_instance_norm_resolve_format), the same code the kernels run, so graph-construction
// errors and kernel errors cannot drift apart.  With a dimension still unknown the dependent
// output dimensions stay unknown.
#include <string>
#include <vector>

#include "atex_norms.h"
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/shape_inference.h"

namespace tensorflow {
namespace {

using shape_inference::DimensionHandle;
using shape_inference::InferenceContext;
using shape_inference::ShapeHandle;

// Dimensions of a shape of known rank; unknown ones are reported through *all_known and
// entered as 1 so that the resolvers can still validate the axis list.
std::vector<int64_t> KnownDims(InferenceContext* c, ShapeHandle s, bool* all_known) {
  std::vector<int64_t> dims;
  *all_known = true;
  for (int i = 0; i < c->Rank(s); ++i) {
    const DimensionHandle d = c->Dim(s, i);
    if (c->ValueKnown(d)) {
      dims.push_back(c->Value(d));
    } else {
      dims.push_back(1);
      *all_known = false;
    }
  }
  return dims;
}

// N (product of the leading dims) and D (product of the normalised dims) of a LayerNorm input.
Status LayerNormSizes(InferenceContext* c, ShapeHandle x, DimensionHandle* n, DimensionHandle* d) {
  std::vector<int> axis;
  TF_RETURN_IF_ERROR(c->GetAttr("axis", &axis));
  if (!c->RankKnown(x)) {
    *n = c->UnknownDim();
    *d = c->UnknownDim();
    return OkStatus();
  }
  if (c->Rank(x) > ATEXN_MAX_RANK) {
    return errors::InvalidArgument("inputs of rank ", c->Rank(x), " are not supported");
  }
  bool known = false;
  const std::vector<int64_t> dims = KnownDims(c, x, &known);
  int64_t nn = 0, dd = 0;
  if (atexn_layer_norm_resolve_axes(c->Rank(x), dims.data(), axis.data(),
                                    static_cast<int>(axis.size()), &nn, &dd) != ATEXN_OK) {
    return errors::InvalidArgument(atexn_last_error());
  }
  *n = known ? c->MakeDim(nn) : c->UnknownDim();
  *d = known ? c->MakeDim(dd) : c->UnknownDim();
  return OkStatus();
}

Status LayerNormShape(InferenceContext* c) {
  ShapeHandle x;
  TF_RETURN_IF_ERROR(c->WithRankAtLeast(c->input(0), 1, &x));
  DimensionHandle n, d;
  TF_RETURN_IF_ERROR(LayerNormSizes(c, x, &n, &d));
  c->set_output(0, x);
  c->set_output(1, c->Vector(n));
  c->set_output(2, c->Vector(n));
  return OkStatus();
}

// The kernel hands dgamma / dbeta back in the shape gamma came in
// (fused_layer_norm_op.cc:451-457), so that is what the graph is told.
Status LayerNormGradShape(InferenceContext* c) {
  ShapeHandle x;
  TF_RETURN_IF_ERROR(c->WithRankAtLeast(c->input(1), 1, &x));
  DimensionHandle n, d;
  TF_RETURN_IF_ERROR(LayerNormSizes(c, x, &n, &d));
  c->set_output(0, x);
  c->set_output(1, c->input(2));
  c->set_output(2, c->input(2));
  return OkStatus();
}

// Index of the channel dimension of an InstanceNorm input of known rank.
Status ChannelIndex(InferenceContext* c, ShapeHandle x, int* index) {
  std::string data_format;
  TF_RETURN_IF_ERROR(c->GetAttr("data_format", &data_format));
  bool known = false;
  const std::vector<int64_t> dims = KnownDims(c, x, &known);
  int layout = 0;
  int64_t n = 0, ch = 0, d = 0;
  if (atexn_instance_norm_resolve_format(c->Rank(x), dims.data(), data_format.c_str(), &layout,
                                         &n, &ch, &d) != ATEXN_OK) {
    return errors::InvalidArgument(atexn_last_error());
  }
  *index = layout == ATEXN_LAYOUT_NC_ ? 1 : c->Rank(x) - 1;
  return OkStatus();
}

Status InstanceNormShape(InferenceContext* c) {
  ShapeHandle x;
  TF_RETURN_IF_ERROR(c->WithRankAtLeast(c->input(0), 4, &x));
  c->set_output(0, x);
  if (!c->RankKnown(x)) {
    c->set_output(1, c->MakeShape({c->UnknownDim(), c->UnknownDim()}));
    c->set_output(2, c->MakeShape({c->UnknownDim(), c->UnknownDim()}));
    return OkStatus();
  }
  int ci = 0;
  TF_RETURN_IF_ERROR(ChannelIndex(c, x, &ci));
  const ShapeHandle stats = c->MakeShape({c->Dim(x, 0), c->Dim(x, ci)});
  c->set_output(1, stats);
  c->set_output(2, stats);
  return OkStatus();
}

Status InstanceNormGradShape(InferenceContext* c) {
  ShapeHandle x;
  TF_RETURN_IF_ERROR(c->WithRankAtLeast(c->input(1), 4, &x));
  c->set_output(0, x);
  if (!c->RankKnown(x)) {
    c->set_output(1, c->Vector(c->UnknownDim()));
    c->set_output(2, c->Vector(c->UnknownDim()));
    return OkStatus();
  }
  int ci = 0;
  TF_RETURN_IF_ERROR(ChannelIndex(c, x, &ci));
  c->set_output(1, c->Vector(c->Dim(x, ci)));
  c->set_output(2, c->Vector(c->Dim(x, ci)));
  return OkStatus();
}

}  // namespace

REGISTER_OP("FusedLayerNorm")
    .Input("x: T")
    .Input("scale: U")
    .Input("offset: U")
    .Output("y: T")
    .Output("reserve_space_1: U")
    .Output("reserve_space_2: U")
    .Attr("T: {half, bfloat16, float}")
    .Attr("U: {float}")
    .Attr("epsilon: float = 0.001")
    .Attr("axis: list(int) = [-1]")
    .SetShapeFn(LayerNormShape);

REGISTER_OP("FusedLayerNormGrad")
    .Input("y_backprop: T")
    .Input("x: T")
    .Input("scale: U")
    .Input("reserve_space_1: U")
    .Input("reserve_space_2: U")
    .Output("x_backprop: T")
    .Output("scale_backprop: U")
    .Output("offset_backprop: U")
    .Attr("T: {half, bfloat16, float}")
    .Attr("U: {float}")
    .Attr("epsilon: float = 0.001")
    .Attr("axis: list(int) = [-1]")
    .SetShapeFn(LayerNormGradShape);

REGISTER_OP("FusedInstanceNorm")
    .Input("x: T")
    .Input("scale: U")
    .Input("offset: U")
    .Output("y: T")
    .Output("reserve_space_1: U")
    .Output("reserve_space_2: U")
    .Attr("T: {half, bfloat16, float}")
    .Attr("U: {float}")
    .Attr("data_format: string = 'N...C'")
    .Attr("epsilon: float = 0.001")
    .SetShapeFn(InstanceNormShape);

REGISTER_OP("FusedInstanceNormGrad")
    .Input("y_backprop: T")
    .Input("x: T")
    .Input("scale: U")
    .Input("reserve_space_1: U")
    .Input("reserve_space_2: U")
    .Output("x_backprop: T")
    .Output("scale_backprop: U")
    .Output("offset_backprop: U")
    .Attr("T: {half, bfloat16, float}")
    .Attr("U: {float}")
    .Attr("data_format: string = 'N...C'")
    .Attr("epsilon: float = 0.001")
    .SetShapeFn(InstanceNormGradShape);

}  // namespace tensorflow
