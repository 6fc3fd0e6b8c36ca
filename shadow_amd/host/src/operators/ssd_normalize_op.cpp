// SSDNormalize: L2 normalisation across the whole item or across channels at
// every position, with an optional second input holding the scale (defaults
// across_spatial = true, channel_shared = true, eps = 1e-5).  Behaviour of
// shadow/operators/ssd_normalize_op.cpp:7-45.
#include "shadow/kernels/ssd_normalize.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class SSDNormalizeOp : public Operator {
 public:
  SSDNormalizeOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    across_spatial_ = get_single_argument<bool>("across_spatial", true);
    channel_shared_ = get_single_argument<bool>("channel_shared", true);
    eps_ = get_single_argument<float>("eps", 1e-5);
    kernel_ = std::dynamic_pointer_cast<SSDNormalizeKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    output->reshape(input->shape());
    if (inputs.size() == 1) {
      kernel_->Run(input, nullptr, output, ws_, across_spatial_, channel_shared_, eps_);
    } else {
      CHECK_EQ(inputs.size(), 2);
      kernel_->Run(input, inputs[1], output, ws_, across_spatial_, channel_shared_, eps_);
    }
  }

 private:
  float eps_ = 1e-5f;
  bool across_spatial_ = true, channel_shared_ = true;
  std::shared_ptr<SSDNormalizeKernel> kernel_;
};

REGISTER_OPERATOR(SSDNormalize, SSDNormalizeOp);

}  // namespace Shadow
