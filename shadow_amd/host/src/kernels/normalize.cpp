#include "shadow/kernels/normalize.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Normalize<DeviceType::kGPU, float>(const float* in_data, int outer_num, int dim,
                                        int inner_num, float p, float eps, float* out_data,
                                        Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_normalize(outer_num, dim, inner_num, p, eps, in_data, out_data,
                                      context->stream()));
}

}  // namespace Vision

class NormalizeKernelHip : public NormalizeKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           float p, int axis, float eps) override {
    const int outer_num = input->count(0, axis), dim = input->shape(axis),
              inner_num = input->count(axis + 1);
    Vision::Normalize<DeviceType::kGPU, float>(input->data<float>(), outer_num, dim, inner_num, p,
                                               eps, output->mutable_data<float>(),
                                               ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(NormalizeGPU, NormalizeKernelHip);

}  // namespace Shadow
