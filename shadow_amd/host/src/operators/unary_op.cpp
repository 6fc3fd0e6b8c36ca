// Unary: y = f(x) for one of 15 functions.  Behaviour of
// shadow/operators/unary_op.cpp:9-28: argument `operation` (s_i, 0..14,
// mandatory), output takes the input's shape.
#include "shadow/kernels/unary.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class UnaryOp : public Operator {
 public:
  UnaryOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    operation_ = get_single_argument<int>("operation", -1);
    CHECK_GE(operation_, 0);
    CHECK_LE(operation_, 14);
    kernel_ = std::dynamic_pointer_cast<UnaryKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    outputs[0]->reshape(inputs[0]->shape());
    kernel_->Run(inputs[0], outputs[0], ws_, operation_);
  }

 private:
  int operation_ = -1;
  std::shared_ptr<UnaryKernel> kernel_;
};

REGISTER_OPERATOR(Unary, UnaryOp);

}  // namespace Shadow
