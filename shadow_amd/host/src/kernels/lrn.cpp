#include "shadow/kernels/lrn.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void LRN<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape, int size, float alpha,
                                  float beta, float k, float* /*scale_data*/, float* out_data,
                                  Context* context) {
  CHECK_EQ(in_shape.size(), 4u) << "LRN reads in_shape[0..3]";
  SHADOW_HIP_CHECK(shdw_hip_lrn(in_shape.data(), size, alpha, beta, k, in_data, out_data,
                                context->stream()));
}

}  // namespace Vision

// No temp blob: the reference grows the temp buffer by the input's size for the
// scale values (shadow/operators/kernels/lrn.hpp:39-41).
class LRNKernelHip : public LRNKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws, int size,
           float alpha, float beta, float k) override {
    Vision::LRN<DeviceType::kGPU, float>(input->data<float>(), input->shape(), size, alpha, beta, k,
                                         nullptr, output->mutable_data<float>(), ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(LRNGPU, LRNKernelHip);

}  // namespace Shadow
