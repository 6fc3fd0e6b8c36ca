// Scale: y = x * s[c] + b[c] along `axis` (default 1).  Parameters are either
// input blobs (`has_scale` / `has_bias`) or the host arguments `scale_value` /
// `bias_value`, where a single value is replicated over the axis.  Behaviour of
// shadow/operators/scale_op.cpp:9-52.
#include "shadow/kernels/scale.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class ScaleOp : public Operator {
 public:
  ScaleOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    axis_ = get_single_argument<int>("axis", 1);
    has_scale_ = get_single_argument<bool>("has_scale", false);
    has_bias_ = get_single_argument<bool>("has_bias", false);
    scale_value_ = get_repeated_argument<float>("scale_value");
    bias_value_ = get_repeated_argument<float>("bias_value");
    kernel_ = std::dynamic_pointer_cast<ScaleKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    output->reshape(input->shape());

    if (has_scale_ || has_bias_) {
      CHECK_EQ(inputs.size(), has_scale_ && has_bias_ ? 3 : 2);
      const std::shared_ptr<Blob> none;
      kernel_->Run(input, has_scale_ ? inputs[1] : none,
                   has_bias_ ? inputs[has_scale_ ? 2 : 1] : none, output, ws_, axis_);
      return;
    }
    const int dim = input->shape(axis_);
    spread(&scale_value_, dim);
    spread(&bias_value_, dim);
    kernel_->Run(input, output, ws_, axis_, scale_value_, bias_value_);
  }

 private:
  // One value stands for the whole axis; several must match its extent.
  static void spread(VecFloat* values, int dim) {
    if (values->size() > 1) {
      CHECK_EQ(values->size(), dim);
    } else if (values->size() == 1) {
      values->assign(dim, (*values)[0]);
    }
  }

  int axis_ = 1;
  bool has_scale_ = false, has_bias_ = false;
  VecFloat scale_value_, bias_value_;
  std::shared_ptr<ScaleKernel> kernel_;
};

REGISTER_OPERATOR(Scale, ScaleOp);

}  // namespace Shadow
