// GroupNorm (`group`, default 1; `eps`, default 1e-5) and InstanceNorm (one
// group per channel): inputs are x alone or x, scale, bias (per channel).
// Behaviour of shadow/operators/group_norm_op.cpp:7-47 and
// instance_norm_op.cpp:7-44; both use the "GroupNorm" kernel.
#include "shadow/kernels/group_norm.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

namespace {

void run_group_norm(GroupNormKernel* kernel, const std::vector<std::shared_ptr<Blob>>& inputs,
                    std::shared_ptr<Blob>& output, Workspace* ws, int group, float eps) {
  const std::shared_ptr<Blob> none;
  if (inputs.size() == 1) {
    kernel->Run(inputs[0], none, none, output, ws, group, eps);
  } else {
    CHECK_EQ(inputs.size(), 3);
    kernel->Run(inputs[0], inputs[1], inputs[2], output, ws, group, eps);
  }
}

}  // namespace

class GroupNormOp : public Operator {
 public:
  GroupNormOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    group_ = get_single_argument<int>("group", 1);
    eps_ = get_single_argument<float>("eps", 1e-5);
    kernel_ = std::dynamic_pointer_cast<GroupNormKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    output->reshape(input->shape());
    CHECK_GT(group_, 0);
    CHECK_EQ(input->shape(1) % group_, 0);
    run_group_norm(kernel_.get(), inputs, output, ws_, group_, eps_);
  }

 private:
  int group_ = 1;
  float eps_ = 1e-5f;
  std::shared_ptr<GroupNormKernel> kernel_;
};

REGISTER_OPERATOR(GroupNorm, GroupNormOp);

class InstanceNormOp : public Operator {
 public:
  InstanceNormOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    eps_ = get_single_argument<float>("eps", 1e-5);
    kernel_ = std::dynamic_pointer_cast<GroupNormKernel>(
        CreateKernel("GroupNorm", ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    output->reshape(input->shape());
    run_group_norm(kernel_.get(), inputs, output, ws_, input->shape(1), eps_);
  }

 private:
  float eps_ = 1e-5f;
  std::shared_ptr<GroupNormKernel> kernel_;
};

REGISTER_OPERATOR(InstanceNorm, InstanceNormOp);

}  // namespace Shadow
