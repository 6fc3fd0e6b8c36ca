// Pooling over the 2 or 3 trailing axes: `pool` 0 = max, 1 = average;
// `global_pooling` takes the whole plane; `full_pooling` (default true) rounds
// the output extent up instead of down.  Sizes are computed in fp32 exactly as
// shadow/operators/pooling_op.cpp:7-26; behaviour of :28-95.
#include <cmath>

#include "shadow/kernels/pooling.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

inline int pooling_out_size(int dim, int kernel_size, int stride, int pad, bool full_pooling) {
  const float span = (dim + 2.f * pad - kernel_size) / stride;
  return static_cast<int>((full_pooling ? std::ceil(span) : std::floor(span)) + 1);
}

// One value stands for every spatial axis.
inline VecInt expand_param(const VecInt& param, int num) {
  if (param.size() == 1) return VecInt(num, param[0]);
  CHECK_EQ(param.size(), num);
  return param;
}

class PoolingOp : public Operator {
 public:
  PoolingOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    pool_type_ = get_single_argument<int>("pool", 0);
    CHECK_GE(pool_type_, 0);
    CHECK_LE(pool_type_, 1);
    global_pooling_ = get_single_argument<bool>("global_pooling", false);
    if (global_pooling_) {
      stride_ = VecInt(1, 1), pad_ = VecInt(1, 0);
    } else {
      kernel_size_ = get_repeated_argument<int>("kernel_size", 0);
      stride_ = get_repeated_argument<int>("stride", 1);
      pad_ = get_repeated_argument<int>("pad", 0);
    }
    full_pooling_ = get_single_argument<bool>("full_pooling", true);
    kernel_ = std::dynamic_pointer_cast<PoolingKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);

    const int num_spatial_axes = input->num_axes() - 2;
    CHECK(num_spatial_axes == 2 || num_spatial_axes == 3) << "Only support 2D or 3D Pooling";

    // The plane extents are captured on the first run only, as in the reference.
    if (global_pooling_ && static_cast<int>(kernel_size_.size()) != num_spatial_axes) {
      for (int n = 0; n < num_spatial_axes; ++n) kernel_size_.push_back(input->shape(n + 2));
    }
    const auto kernel_size = expand_param(kernel_size_, num_spatial_axes);
    const auto stride = expand_param(stride_, num_spatial_axes);
    const auto pad = expand_param(pad_, num_spatial_axes);

    auto out_shape = input->shape();
    for (int n = 0; n < num_spatial_axes; ++n) {
      out_shape[n + 2] =
          pooling_out_size(input->shape(n + 2), kernel_size[n], stride[n], pad[n], full_pooling_);
    }
    output->reshape(out_shape);

    if (num_spatial_axes == 2) {
      kernel_->Run(input, output, ws_, pool_type_, kernel_size[0], kernel_size[1], stride[0],
                   stride[1], pad[0], pad[1], full_pooling_);
    } else {
      kernel_->Run(input, output, ws_, pool_type_, kernel_size[0], kernel_size[1], kernel_size[2],
                   stride[0], stride[1], stride[2], pad[0], pad[1], pad[2], full_pooling_);
    }
  }

 private:
  int pool_type_ = 0;
  bool global_pooling_ = false, full_pooling_ = true;
  VecInt kernel_size_, stride_, pad_;
  std::shared_ptr<PoolingKernel> kernel_;
};

REGISTER_OPERATOR(Pooling, PoolingOp);

}  // namespace Shadow
