// Eltwise: K >= 2 inputs of one shape combined by Prod(0) / Sum(1) / Max(2) /
// Min(3); `coeff` (one per input) only with Sum.  Behaviour of
// shadow/operators/eltwise_op.cpp:9-47.
#include "shadow/kernels/eltwise.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class EltwiseOp : public Operator {
 public:
  EltwiseOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    operation_ = get_single_argument<int>("operation", -1);
    CHECK_GE(operation_, 0);
    CHECK_LE(operation_, 3);
    coeff_ = get_repeated_argument<float>("coeff");
    kernel_ = std::dynamic_pointer_cast<EltwiseKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_GE(inputs.size(), 2);
    const auto& first = inputs[0];
    for (size_t n = 1; n < inputs.size(); ++n) CHECK(inputs[n]->shape() == first->shape());
    outputs[0]->reshape(first->shape());

    CHECK(coeff_.empty() || coeff_.size() == inputs.size())
        << "Eltwise op takes one coefficient per input blob.";
    CHECK(operation_ == kSum || coeff_.empty())
        << "Eltwise op only takes coefficients for summation.";

    VecFloat coeff(inputs.size(), 1.f);
    std::copy(coeff_.begin(), coeff_.end(), coeff.begin());
    kernel_->Run(inputs, outputs[0], ws_, operation_, coeff);
  }

 private:
  int operation_ = -1;
  VecFloat coeff_;
  std::shared_ptr<EltwiseKernel> kernel_;
};

REGISTER_OPERATOR(Eltwise, EltwiseOp);

}  // namespace Shadow
