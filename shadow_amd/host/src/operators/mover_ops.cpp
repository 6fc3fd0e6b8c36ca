// Concat, Slice, Stack, Gather, Pad, Permute, Reorg, ShuffleChannel, Resize:
// argument handling and output shapes of the reference's operators
// (shadow/operators/{concat,slice,stack,gather,pad,permute,reorg,
// shuffle_channel,resize}_op.cpp); the data movement is in the kernels.
#include "shadow/kernels/movers.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

namespace {

template <class K>
std::shared_ptr<K> kernel_of(const shadow::OpParam& op_param, Workspace* ws) {
  auto kernel = std::dynamic_pointer_cast<K>(CreateKernel(op_param.type(), ws->Ctx()->device_type()));
  CHECK_NOTNULL(kernel);
  return kernel;
}

}  // namespace

// All inputs agree except along `axis` (default 1).  concat_op.cpp:9-50
class ConcatOp : public Operator {
 public:
  ConcatOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 1);
    kernel_ = kernel_of<ConcatKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_GE(inputs.size(), 2);
    const auto& first = inputs[0];
    auto& output = outputs[0];
    axis_ = first->canonical_index(axis_);
    auto out_shape = first->shape();
    const int num_axes = first->num_axes();
    for (size_t n = 1; n < inputs.size(); ++n) {
      const auto& input = inputs[n];
      CHECK_EQ(num_axes, input->num_axes()) << "Inputs must have the same axes!";
      for (int d = 0; d < num_axes; ++d) {
        if (d != axis_) {
          CHECK_EQ(out_shape[d], input->shape(d))
              << "Inputs must have the same shape, except at concat_axis!";
        }
      }
      out_shape[axis_] += input->shape(axis_);
    }
    for (const auto& input : inputs) CHECK_NE(input, output);
    output->reshape(out_shape);
    kernel_->Run(inputs, output, ws_, axis_);
  }

 private:
  int axis_ = 1;
  std::shared_ptr<ConcatKernel> kernel_;
};
REGISTER_OPERATOR(Concat, ConcatOp);

// Splits `axis` (default 1) over the outputs: equal parts, or at `slice_point`.
// slice_op.cpp:9-66
class SliceOp : public Operator {
 public:
  SliceOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 1);
    slice_point_ = get_repeated_argument<int>("slice_point");
    kernel_ = kernel_of<SliceKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_GE(outputs.size(), 2);
    const auto& input = inputs[0];
    axis_ = input->canonical_index(axis_);
    const int num_outputs = static_cast<int>(outputs.size());
    const int in_slice_axis = input->shape(axis_);
    VecInt slices;
    if (slice_point_.empty()) {
      CHECK_EQ(in_slice_axis % num_outputs, 0);
      slices.assign(num_outputs, in_slice_axis / num_outputs);
    } else {
      CHECK_EQ(slice_point_.size(), num_outputs - 1);
      int prev = 0;
      for (int point : slice_point_) {
        CHECK_GT(point, prev);
        slices.push_back(point - prev);
        prev = point;
      }
      CHECK_GT(in_slice_axis, prev);
      slices.push_back(in_slice_axis - prev);
    }
    int count = 0;
    auto out_shape = input->shape();
    for (int n = 0; n < num_outputs; ++n) {
      CHECK_NE(input, outputs[n]);
      out_shape[axis_] = slices[n];
      outputs[n]->reshape(out_shape);
      count += outputs[n]->count();
    }
    CHECK_EQ(count, input->count());
    kernel_->Run(input, outputs, ws_, axis_);
  }

 private:
  int axis_ = 1;
  VecInt slice_point_;
  std::shared_ptr<SliceKernel> kernel_;
};
REGISTER_OPERATOR(Slice, SliceOp);

// A new axis of extent inputs.size() at `axis` (default 0, negative from the
// end of the output rank).  stack_op.cpp:9-47
class StackOp : public Operator {
 public:
  StackOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 0);
    kernel_ = kernel_of<StackKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_GE(inputs.size(), 2);
    const auto& first = inputs[0];
    auto& output = outputs[0];
    const int num_axes = first->num_axes();
    CHECK(axis_ >= -(num_axes + 1) && axis_ < num_axes + 1) << "axis out of bound.";
    if (axis_ < 0) axis_ += num_axes + 1;
    auto out_shape = first->shape();
    out_shape.insert(out_shape.begin() + axis_, static_cast<int>(inputs.size()));
    for (const auto& input : inputs) CHECK_NE(input, output);
    output->reshape(out_shape);
    kernel_->Run(inputs, output, ws_, axis_);
  }

 private:
  int axis_ = 0;
  std::shared_ptr<StackKernel> kernel_;
};
REGISTER_OPERATOR(Stack, StackOp);

// Picks entries along `axis` (default 0) by the `indexes` argument or, without
// it, by a second 1-D int32 input.  gather_op.cpp:9-59
class GatherOp : public Operator {
 public:
  GatherOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 0);
    indexes_value_ = get_repeated_argument<int>("indexes");
    kernel_ = kernel_of<GatherKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    axis_ = input->canonical_index(axis_);
    std::shared_ptr<Blob> indexes;
    if (indexes_value_.empty()) {
      CHECK_EQ(inputs.size(), 2);
      indexes = inputs[1];
      CHECK_EQ(indexes->num_axes(), 1);
      CHECK(indexes->data_type() == DataType::kI32) << "indexes must be an int blob";
    } else {
      // Host values can be checked here; the reference would read out of bounds.
      for (int index : indexes_value_) {
        CHECK_GE(index, 0);
        CHECK_LT(index, input->shape(axis_));
      }
      const int num_indexes = static_cast<int>(indexes_value_.size());
      ws_->GrowTempBuffer(num_indexes * sizeof(int));
      indexes = ws_->CreateTempBlob({num_indexes}, DataType::kI32);
      indexes->set_data<std::int32_t>(indexes_value_.data(), indexes->count());
    }
    const int num_indexes = indexes->count();
    CHECK_GT(num_indexes, 0);
    auto out_shape = input->shape();
    out_shape[axis_] = num_indexes;
    output->reshape(out_shape);
    kernel_->Run(input, indexes, output, ws_, axis_);
  }

 private:
  int axis_ = 0;
  VecInt indexes_value_;
  std::shared_ptr<GatherKernel> kernel_;
};
REGISTER_OPERATOR(Gather, GatherOp);

// `paddings` = top, bottom, left, right on the two trailing axes of a 4-D
// input (negative crops), `value` fills.  pad_op.cpp:9-46
class PadOp : public Operator {
 public:
  PadOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    paddings_ = get_repeated_argument<int>("paddings");
    CHECK_EQ(paddings_.size(), 4);
    value_ = get_single_argument<float>("value", 0);
    kernel_ = kernel_of<PadKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    CHECK_EQ(input->num_axes(), 4);
    auto out_shape = input->shape();
    out_shape[2] = input->shape(2) + paddings_[0] + paddings_[1];
    out_shape[3] = input->shape(3) + paddings_[2] + paddings_[3];
    CHECK_GT(out_shape[2], 0);
    CHECK_GT(out_shape[3], 0);
    output->reshape(out_shape);
    kernel_->Run(input, output, ws_, paddings_, value_);
  }

 private:
  float value_ = 0;
  VecInt paddings_;
  std::shared_ptr<PadKernel> kernel_;
};
REGISTER_OPERATOR(Pad, PadOp);

// Output axis j is input axis order[j].  permute_op.cpp:9-43
class PermuteOp : public Operator {
 public:
  PermuteOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    order_value_ = get_repeated_argument<int>("order");
    kernel_ = kernel_of<PermuteKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    CHECK_EQ(input->num_axes(), order_value_.size());
    VecInt out_shape;
    for (int axis : order_value_) out_shape.push_back(input->shape(axis));
    output->reshape(out_shape);
    CHECK_EQ(output->count(), input->count()) << "order must name every axis once";
    kernel_->Run(input, output, ws_, order_value_);
  }

 private:
  VecInt order_value_;
  std::shared_ptr<PermuteKernel> kernel_;
};
REGISTER_OPERATOR(Permute, PermuteOp);

// Space-to-depth by `stride` (default 2); `type` 0 = Darknet order, 1 = natural.
// reorg_op.cpp:9-51
class ReorgOp : public Operator {
 public:
  ReorgOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    type_ = get_single_argument<int>("type", 0);
    stride_ = get_single_argument<int>("stride", 2);
    kernel_ = kernel_of<ReorgKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    CHECK_EQ(input->num_axes(), 4);
    CHECK_GT(stride_, 0);
    const int in_c = input->shape(1), in_h = input->shape(2), in_w = input->shape(3);
    if (type_ == kDarknet) CHECK_EQ(in_c % (stride_ * stride_), 0);
    CHECK_EQ(in_h % stride_, 0);
    CHECK_EQ(in_w % stride_, 0);
    auto out_shape = input->shape();
    out_shape[1] = in_c * stride_ * stride_;
    out_shape[2] = in_h / stride_;
    out_shape[3] = in_w / stride_;
    output->reshape(out_shape);
    kernel_->Run(input, output, ws_, type_, stride_);
  }

 private:
  int type_ = 0, stride_ = 2;
  std::shared_ptr<ReorgKernel> kernel_;
};
REGISTER_OPERATOR(Reorg, ReorgOp);

// ShuffleNet channel shuffle with `group` groups (mandatory, > 0).
// shuffle_channel_op.cpp:9-42
class ShuffleChannelOp : public Operator {
 public:
  ShuffleChannelOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    group_ = get_single_argument<int>("group", 0);
    CHECK_GT(group_, 0) << "group must be larger than 0";
    kernel_ = kernel_of<ShuffleChannelKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    CHECK_EQ(input->shape(1) % group_, 0);
    output->reshape(input->shape());
    kernel_->Run(input, output, ws_, group_);
  }

 private:
  int group_ = 0;
  std::shared_ptr<ShuffleChannelKernel> kernel_;
};
REGISTER_OPERATOR(ShuffleChannel, ShuffleChannelOp);

// 2-D resize to `size` (when > 0) or by `scale`; `type` 0 nearest, 1 bilinear
// (default); `align_corners` default false.  resize_op.cpp:9-76
class ResizeOp : public Operator {
 public:
  ResizeOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    size_ = get_repeated_argument<int>("size", 0);
    scale_ = get_repeated_argument<float>("scale", 1);
    type_ = get_single_argument<int>("type", 1);
    CHECK_GE(type_, 0);
    CHECK_LE(type_, 1);
    align_corners_ = get_single_argument<bool>("align_corners", false);
    kernel_ = kernel_of<ResizeKernel>(op_param, ws_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);
    const int num_spatial_axes = input->num_axes() - 2;
    CHECK_EQ(num_spatial_axes, 2) << "Only support 2D Resize";
    const auto size = expand(size_, num_spatial_axes);
    const auto scale = expand(scale_, num_spatial_axes);
    auto out_shape = input->shape();
    for (int n = 0; n < num_spatial_axes; ++n) {
      out_shape[n + 2] =
          size[n] > 0 ? size[n] : static_cast<int>(input->shape(n + 2) * scale[n]);
      CHECK_GT(out_shape[n + 2], 0);
    }
    output->reshape(out_shape);
    kernel_->Run(input, output, ws_, type_, align_corners_);
  }

 private:
  // One value stands for both axes.
  template <typename T>
  static std::vector<T> expand(const std::vector<T>& param, int num) {
    if (param.size() == 1) return std::vector<T>(num, param[0]);
    CHECK_EQ(param.size(), num);
    return param;
  }

  int type_ = 1;
  bool align_corners_ = false;
  VecInt size_;
  VecFloat scale_;
  std::shared_ptr<ResizeKernel> kernel_;
};
REGISTER_OPERATOR(Resize, ResizeOp);

}  // namespace Shadow
