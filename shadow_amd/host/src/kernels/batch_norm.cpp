#include "shadow/kernels/batch_norm.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void BatchNorm<DeviceType::kGPU, float>(const float* in_data, int count, const float* mean_data,
                                        const float* variance_data, int channel, int inner_num,
                                        float scale_factor, float eps, float* out_data,
                                        Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_batch_norm(count, channel, inner_num, in_data, mean_data,
                                       variance_data, scale_factor, eps, out_data,
                                       context->stream()));
}

}  // namespace Vision

class BatchNormKernelHip : public BatchNormKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& mean,
           const std::shared_ptr<Blob>& variance, std::shared_ptr<Blob>& output, Workspace* ws,
           float scale_factor, float eps) override {
    const int channel = input->shape(1);
    CHECK_EQ(channel, mean->count());
    CHECK_EQ(channel, variance->count());
    Vision::BatchNorm<DeviceType::kGPU, float>(
        input->data<float>(), input->count(), mean->data<float>(), variance->data<float>(),
        channel, input->count(2), scale_factor, eps, output->mutable_data<float>(),
        ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(BatchNormGPU, BatchNormKernelHip);

}  // namespace Shadow
