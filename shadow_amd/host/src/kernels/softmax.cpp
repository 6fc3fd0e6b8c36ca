#include "shadow/kernels/softmax.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Softmax<DeviceType::kGPU, float>(const float* in_data, int outer_num, int dim,
                                      int inner_num, float* out_data, Context* context) {
  SHADOW_HIP_CHECK(
      shdw_hip_softmax(outer_num, dim, inner_num, in_data, out_data, context->stream()));
}

}  // namespace Vision

class SoftmaxKernelHip : public SoftmaxKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int axis) override {
    const int outer_num = input->count(0, axis), dim = input->shape(axis),
              inner_num = input->count(axis + 1);
    Vision::Softmax<DeviceType::kGPU, float>(input->data<float>(), outer_num, dim, inner_num,
                                             output->mutable_data<float>(), ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(SoftmaxGPU, SoftmaxKernelHip);

}  // namespace Shadow
