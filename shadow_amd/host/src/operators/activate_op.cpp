// Activate: `type` 0 PRelu (second input = slopes) .. 8 Gelu, default 1 (ReLU);
// `slope` (default 0.1) for Leaky.  Behaviour of
// shadow/operators/activate_op.cpp:9-34.
#include "shadow/kernels/activate.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class ActivateOp : public Operator {
 public:
  ActivateOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    activate_type_ = get_single_argument<int>("type", 1);
    slope_ = get_single_argument<float>("slope", 0.1f);
    CHECK_GE(activate_type_, 0);
    CHECK_LE(activate_type_, 8);
    kernel_ = std::dynamic_pointer_cast<ActivateKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const bool prelu = activate_type_ == kPRelu;
    CHECK_EQ(inputs.size(), prelu ? 2 : 1);
    outputs[0]->reshape(inputs[0]->shape());
    kernel_->Run(inputs[0], prelu ? inputs[1] : std::shared_ptr<Blob>(), outputs[0], ws_,
                 activate_type_, slope_);
  }

 private:
  int activate_type_ = 1;
  float slope_ = 0.1f;
  std::shared_ptr<ActivateKernel> kernel_;
};

REGISTER_OPERATOR(Activate, ActivateOp);

}  // namespace Shadow
