// Reduce: Prod/Sum/Max/Min/Avg/L1/L2 over a set of axes (empty = all).
// Behaviour of shadow/operators/reduce_op.cpp:9-65: the kernel always writes
// the keep-dims layout; keep_dims = false only rewrites the shape vector.
#include <algorithm>

#include "shadow/kernels/reduce.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class ReduceOp : public Operator {
 public:
  ReduceOp(const shadow::OpParam& op_param, Workspace* ws) : Operator(op_param, ws) {
    operation_ = get_single_argument<int>("operation", 0);
    CHECK_GE(operation_, 0);
    CHECK_LE(operation_, 6);
    axes_ = get_repeated_argument<int>("axes");
    keep_dims_ = get_single_argument<bool>("keep_dims", true);
    kernel_ = std::dynamic_pointer_cast<ReduceKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    const auto& input = inputs[0];
    auto& output = outputs[0];
    CHECK_NE(input, output);  // never in place

    const int num_axes = input->num_axes();
    VecInt axes = axes_;
    if (axes.empty()) {
      for (int n = 0; n < num_axes; ++n) axes.push_back(n);
    }
    VecInt out_shape = input->shape();
    for (int axis : axes) out_shape[input->canonical_index(axis)] = 1;
    output->reshape(out_shape);

    kernel_->Run(input, output, ws_, operation_, axes);

    if (!keep_dims_) {
      // Drop exactly the listed axes; all of them -> rank 0, count() == 1.
      VecInt squeezed;
      for (int n = 0; n < num_axes; ++n) {
        const bool listed = std::find(axes.begin(), axes.end(), n) != axes.end();
        if (listed) {
          CHECK_EQ(output->shape(n), 1);
        } else {
          squeezed.push_back(output->shape(n));
        }
      }
      output->set_shape(squeezed);
    }
  }

 private:
  int operation_ = 0;
  bool keep_dims_ = true;
  VecInt axes_;
  std::shared_ptr<ReduceKernel> kernel_;
};

REGISTER_OPERATOR(Reduce, ReduceOp);

}  // namespace Shadow
