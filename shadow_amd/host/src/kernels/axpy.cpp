#include "shadow/kernels/axpy.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Axpy<DeviceType::kGPU, float>(const float* alpha_data, const float* x_data,
                                   const float* y_data, int outer_num, int inner_num,
                                   float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_axpy_rows(outer_num, inner_num, alpha_data, x_data, y_data, out_data,
                                      context->stream()));
}

}  // namespace Vision

class AxpyKernelHip : public AxpyKernel {
 public:
  void Run(const std::shared_ptr<Blob>& alpha, const std::shared_ptr<Blob>& x,
           const std::shared_ptr<Blob>& y, std::shared_ptr<Blob>& output,
           Workspace* ws) override {
    // one alpha per (n, c) plane of x
    Vision::Axpy<DeviceType::kGPU, float>(alpha->data<float>(), x->data<float>(),
                                          y->data<float>(), alpha->count(), x->count(2),
                                          output->mutable_data<float>(), ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(AxpyGPU, AxpyKernelHip);

}  // namespace Shadow
