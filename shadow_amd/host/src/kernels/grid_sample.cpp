#include "shadow/kernels/grid_sample.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void GridSample<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                         const float* grid_data, int mode, int padding_mode,
                                         const VecInt& out_shape, float* out_data, Context* context) {
  CHECK_EQ(in_shape.size(), 4u);
  CHECK_EQ(out_shape.size(), 4u);
  CHECK(mode == 0 || mode == 1) << "Unsupported grid sample mode: " << mode;
  SHADOW_HIP_CHECK(shdw_hip_grid_sample(in_shape.data(), out_shape.data(), mode, padding_mode, in_data,
                                        grid_data, out_data, context->stream()));
}

}  // namespace Vision

class GridSampleKernelHip : public GridSampleKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& grid,
           std::shared_ptr<Blob>& output, Workspace* ws, int mode, int padding_mode) override {
    Vision::GridSample<DeviceType::kGPU, float>(input->data<float>(), input->shape(), grid->data<float>(),
                                                mode, padding_mode, output->shape(),
                                                output->mutable_data<float>(), ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(GridSampleGPU, GridSampleKernelHip);

}  // namespace Shadow
