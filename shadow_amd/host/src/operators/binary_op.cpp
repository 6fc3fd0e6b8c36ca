// Binary: out = bottom[0] (op) bottom[1] with numpy-style broadcasting, or
// bottom[0] (op) scalar when the argument `scalar` is present.  Behaviour of
// shadow/operators/binary_op.cpp:9-65.
#include <algorithm>

#include "shadow/kernels/binary.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class BinaryOp : public Operator {
 public:
  BinaryOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    operation_ = get_single_argument<int>("operation", -1);
    CHECK_GE(operation_, 0);
    CHECK_LE(operation_, 6);
    // The PRESENCE of `scalar` selects the one-input form.
    has_scalar_ = has_argument("scalar");
    if (has_scalar_) scalar_value_ = get_single_argument<float>("scalar", 0);
    kernel_ = std::dynamic_pointer_cast<BinaryKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_EQ(inputs.size(), has_scalar_ ? 1 : 2);
    const auto& lhs = inputs[0];
    auto& out = outputs[0];

    if (has_scalar_) {
      out->reshape(lhs->shape());
      kernel_->Run(lhs, out, ws_, operation_, scalar_value_);
      return;
    }
    const auto& rhs = inputs[1];
    if (lhs->shape() == rhs->shape()) {
      out->reshape(lhs->shape());
      kernel_->Run(lhs, rhs, out, ws_, operation_, false);
      return;
    }

    // Rank-align by left-padding the shorter shape with 1s.  The kernel reads the
    // shapes from the blobs, so they are swapped in for the call and restored
    // afterwards (also when the call throws).
    const VecInt lhs_shape = lhs->shape(), rhs_shape = rhs->shape();
    const size_t rank = std::max(lhs_shape.size(), rhs_shape.size());
    VecInt lhs_padded(rank - lhs_shape.size(), 1), rhs_padded(rank - rhs_shape.size(), 1);
    lhs_padded.insert(lhs_padded.end(), lhs_shape.begin(), lhs_shape.end());
    rhs_padded.insert(rhs_padded.end(), rhs_shape.begin(), rhs_shape.end());
    VecInt out_shape(rank);
    for (size_t n = 0; n < rank; ++n) {
      const int l = lhs_padded[n], r = rhs_padded[n];
      CHECK(l == r || l == 1 || r == 1);
      out_shape[n] = std::max(l, r);
    }
    out->reshape(out_shape);

    struct Restore {
      const std::shared_ptr<Blob>&a, &b;
      VecInt sa, sb;
      ~Restore() { a->set_shape(sa), b->set_shape(sb); }
    } restore{lhs, rhs, lhs_shape, rhs_shape};
    lhs->set_shape(lhs_padded);
    rhs->set_shape(rhs_padded);
    kernel_->Run(lhs, rhs, out, ws_, operation_, true);
  }

 private:
  int operation_ = -1;
  float scalar_value_ = 0.f;
  bool has_scalar_ = false;
  std::shared_ptr<BinaryKernel> kernel_;
};

REGISTER_OPERATOR(Binary, BinaryOp);

}  // namespace Shadow
