// LRN: local response normalisation.  Arguments and checks of
// shadow/operators/lrn_op.cpp:7-44: `local_size` (odd, default 5), `alpha` (1),
// `beta` (0.75), `k` (1) and `norm_region`, of which only 0, across channels,
// exists.  The output takes the input's shape.
#include "shadow/kernels/lrn.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

namespace {

struct LRNArgs {
  int local_size;
  float alpha, beta, k;
};

}  // namespace

class LRNOp : public Operator {
 public:
  LRNOp(const shadow::OpParam& op_param, Workspace* ws)
      : Operator(op_param, ws),
        args_{get_single_argument<int>("local_size", 5), get_single_argument<float>("alpha", 1),
              get_single_argument<float>("beta", 0.75), get_single_argument<float>("k", 1)} {
    CHECK_EQ(args_.local_size % 2, 1) << "LRN only supports odd values for local_size";
    CHECK_EQ(get_single_argument<int>("norm_region", 0), 0)
        << "Currently only support norm region method: Across Channels!";
    kernel_ = std::dynamic_pointer_cast<LRNKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& x = inputs[0];
    // Two things the reference leaves to the caller: its kernel reads in_shape[0..3],
    // and with fewer channels than lie behind a window's centre its last loop writes
    // in front of the scale blob.
    CHECK_EQ(x->num_axes(), 4) << "LRN works on [batch, channels, height, width]";
    CHECK_GE(x->shape(1), (args_.local_size - 1) / 2) << "LRN window reaches past every channel";
    outputs[0]->reshape(x->shape());
    kernel_->Run(x, outputs[0], ws_, args_.local_size, args_.alpha, args_.beta, args_.k);
  }

 private:
  LRNArgs args_;
  std::shared_ptr<LRNKernel> kernel_;
};

REGISTER_OPERATOR(LRN, LRNOp);

}  // namespace Shadow
