// Operators that change only how a buffer is viewed: Input, Reshape, Flatten,
// Squeeze, Unsqueeze.  The output blob aliases the input's memory
// (Blob::share_data); nothing is launched.  In-place use is refused, as in the
// reference.
#include "shadow/operator.hpp"

namespace Shadow {

// The network inputs are filled by Backend::Run before the operator loop.
// shadow/operators/input_op.cpp:7-15
class InputOp : public Operator {
 public:
  InputOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {}
  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {}
};

REGISTER_OPERATOR(Input, InputOp);

// Caffe-style reshape of the axes [axis, axis + num_axes): `shape` entries are
// extents, 0 = copy the input's extent at that position, -1 = infer (at most
// one).  shadow/operators/reshape_op.cpp:7-84
class ReshapeOp : public Operator {
 public:
  ReshapeOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 0);
    num_axes_ = get_single_argument<int>("num_axes", -1);
    CHECK_GE(num_axes_, -1);
    shape_ = get_repeated_argument<int>("shape");
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);

    const int rank = input->num_axes();
    const int start_axis = input->canonical_index(axis_);
    const int end_axis = num_axes_ == -1 ? rank : start_axis + num_axes_;
    CHECK_LE(end_axis, rank);

    VecInt out_shape(input->shape().begin(), input->shape().begin() + start_axis);
    out_shape.insert(out_shape.end(), shape_.begin(), shape_.end());
    out_shape.insert(out_shape.end(), input->shape().begin() + end_axis, input->shape().end());

    int inferred = -1, known = input->count(0, start_axis) * input->count(end_axis);
    for (int d = 0; d < static_cast<int>(shape_.size()); ++d) {
      int& dim = out_shape[start_axis + d];
      if (dim == 0) {
        CHECK_GT(rank, start_axis + d);
        dim = input->shape(start_axis + d);
      }
      if (dim == -1) {
        CHECK_EQ(inferred, -1);
        inferred = start_axis + d;
      } else {
        known *= dim;
      }
    }
    if (inferred >= 0) {
      CHECK_EQ(0, input->count() % known);
      out_shape[inferred] = input->count() / known;
    }
    output->share_data(input->data<void>(), out_shape);
    CHECK_EQ(output->count(), input->count());
  }

 private:
  int axis_ = 0, num_axes_ = -1;
  VecInt shape_;
};

REGISTER_OPERATOR(Reshape, ReshapeOp);

// Axes [axis, end_axis] become one (defaults 1 and -1 = last).
// shadow/operators/flatten_op.cpp:7-44
class FlattenOp : public Operator {
 public:
  FlattenOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 1);
    CHECK_GE(axis_, 0);
    end_axis_ = get_single_argument<int>("end_axis", -1);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    const int rank = input->num_axes();
    // -1 is resolved on the first run and then kept, as in the reference.
    if (end_axis_ == -1) end_axis_ = rank - 1;
    CHECK_LT(end_axis_, rank);
    CHECK_LE(axis_, end_axis_);
    VecInt out_shape(input->shape().begin(), input->shape().begin() + axis_);
    out_shape.push_back(input->count(axis_, end_axis_ + 1));
    out_shape.insert(out_shape.end(), input->shape().begin() + end_axis_ + 1, input->shape().end());
    output->share_data(input->data<void>(), out_shape);
    CHECK_EQ(output->count(), input->count());
  }

 private:
  int axis_ = 1, end_axis_ = -1;
};

REGISTER_OPERATOR(Flatten, FlattenOp);

// Drops the listed axes (each must have extent 1), or every extent-1 axis when
// none is listed.  shadow/operators/squeeze_op.cpp:7-56
class SqueezeOp : public Operator {
 public:
  SqueezeOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axes_ = get_repeated_argument<int>("axes");
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    VecInt out_shape;
    for (int n = 0; n < input->num_axes(); ++n) {
      const int dim = input->shape(n);
      bool drop = axes_.empty() && dim <= 1;
      for (int axis : axes_) drop = drop || axis == n;
      if (drop) {
        CHECK_EQ(dim, 1);
      } else {
        out_shape.push_back(dim);
      }
    }
    output->share_data(input->data<void>(), out_shape);
    CHECK_EQ(output->count(), input->count());
  }

 private:
  VecInt axes_;
};

REGISTER_OPERATOR(Squeeze, SqueezeOp);

// Inserts extent-1 axes at the listed OUTPUT positions (negative: from the end
// of the output rank).  shadow/operators/unsqueeze_op.cpp:7-49
class UnsqueezeOp : public Operator {
 public:
  UnsqueezeOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axes_ = get_repeated_argument<int>("axes");
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    const int rank = input->num_axes();
    const int out_rank = rank + static_cast<int>(axes_.size());
    VecInt out_shape(out_rank, 0);
    for (int axis : axes_) {
      if (axis < 0) axis += rank + 1;
      CHECK_GE(axis, 0);
      CHECK_LT(axis, out_rank);
      out_shape[axis] = 1;
    }
    int d = 0;
    for (auto& dim : out_shape) {
      if (dim == 0) {
        CHECK_LT(d, rank);
        dim = input->shape(d++);
      }
    }
    CHECK_EQ(d, rank);
    output->share_data(input->data<void>(), out_shape);
    CHECK_EQ(output->count(), input->count());
  }

 private:
  VecInt axes_;
};

REGISTER_OPERATOR(Unsqueeze, UnsqueezeOp);

}  // namespace Shadow
