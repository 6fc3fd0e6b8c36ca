// LayerNorm over the trailing dims named by `normalized_shape` (mandatory),
// `eps` default 1e-5; inputs are x alone or x, scale, bias of that shape.
// Behaviour of shadow/operators/layer_norm_op.cpp:7-53.
#include "shadow/kernels/layer_norm.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class LayerNormOp : public Operator {
 public:
  LayerNormOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    normalized_shape_ = get_repeated_argument<int>("normalized_shape");
    CHECK(!normalized_shape_.empty());
    eps_ = get_single_argument<float>("eps", 1e-5);
    kernel_ = std::dynamic_pointer_cast<LayerNormKernel>(
        CreateKernel("LayerNorm", ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    output->reshape(input->shape());

    const int rank = static_cast<int>(normalized_shape_.size());
    CHECK_LE(rank, input->num_axes());
    for (int n = 0; n < rank; ++n) CHECK_EQ(input->shape(n - rank), normalized_shape_[n]);

    const std::shared_ptr<Blob> none;
    if (inputs.size() == 1) {
      kernel_->Run(input, none, none, output, ws_, normalized_shape_, eps_);
    } else {
      CHECK_EQ(inputs.size(), 3);
      kernel_->Run(input, inputs[1], inputs[2], output, ws_, normalized_shape_, eps_);
    }
  }

 private:
  float eps_ = 1e-5f;
  VecInt normalized_shape_;
  std::shared_ptr<LayerNormKernel> kernel_;
};

REGISTER_OPERATOR(LayerNorm, LayerNormOp);

}  // namespace Shadow
