// GridSample: the input sampled at the positions a grid blob names.  Arguments and
// checks of shadow/operators/grid_sample_op.cpp:7-52: `mode` (0 nearest, 1 bilinear,
// the default) and `padding_mode` (0 zeros, the default, 1 border); inputs are the
// tensor [b, c, h, w] and the grid [b, out_h, out_w, 2]; the output is
// [b, c, out_h, out_w] and may not be the input.
#include "shadow/kernels/grid_sample.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

class GridSampleOp : public Operator {
 public:
  GridSampleOp(const shadow::OpParam& op_param, Workspace* ws)
      : Operator(op_param, ws),
        mode_(get_single_argument<int>("mode", 1)),
        padding_mode_(get_single_argument<int>("padding_mode", 0)) {
    CHECK(mode_ == 0 || mode_ == 1);
    CHECK(padding_mode_ == 0 || padding_mode_ == 1);
    kernel_ = std::dynamic_pointer_cast<GridSampleKernel>(
        CreateKernel(op_param.type(), ws_->Ctx()->device_type()));
    CHECK_NOTNULL(kernel_);
  }

  void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
           std::vector<std::shared_ptr<Blob>>& outputs) override {
    CHECK_EQ(inputs.size(), 2);
    const auto &x = inputs[0], &grid = inputs[1];
    CHECK_NE(x, outputs[0]);
    // the kernel reads shape[0..3] of both
    CHECK_EQ(x->num_axes(), 4);
    CHECK_EQ(grid->num_axes(), 4);
    CHECK_EQ(x->shape(0), grid->shape(0));
    CHECK_EQ(grid->shape(3), 2);
    outputs[0]->reshape({x->shape(0), x->shape(1), grid->shape(1), grid->shape(2)});
    kernel_->Run(x, grid, outputs[0], ws_, mode_, padding_mode_);
  }

 private:
  int mode_, padding_mode_;
  std::shared_ptr<GridSampleKernel> kernel_;
};

REGISTER_OPERATOR(GridSample, GridSampleOp);

}  // namespace Shadow
