#include "shadow/kernels/ssd_normalize.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

size_t SSDNormalizeScratchBytes(int outer_num, int channel, int inner_num, bool across_spatial) {
  return shdw_hip_ssd_normalize_workspace_bytes(outer_num, channel, inner_num, across_spatial);
}

template <>
void SSDNormalize<DeviceType::kGPU, float>(const float* in_data, int outer_num, int channel,
                                           int inner_num, bool across_spatial, float eps,
                                           const float* scale_data, bool channel_shared,
                                           void* val_data, float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_ssd_normalize(outer_num, channel, inner_num, across_spatial, eps,
                                          in_data, scale_data, channel_shared, out_data, val_data,
                                          context->stream()));
}

}  // namespace Vision

class SSDNormalizeKernelHip : public SSDNormalizeKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
           std::shared_ptr<Blob>& output, Workspace* ws, bool across_spatial, bool channel_shared,
           float eps) override {
    const int batch = input->shape(0), channel = input->shape(1), spatial_dim = input->count(2);
    const float* scale_data = nullptr;
    if (scale != nullptr) {
      // ssd_normalize.hpp:70 checks the shared form; the per-channel form reads
      // `channel` values (scale.cpp:14), which the blob must hold.
      if (channel_shared) {
        CHECK_EQ(scale->count(), 1);
      } else {
        CHECK_GE(scale->count(), channel);
      }
      scale_data = scale->data<float>();
    }
    void* scratch = nullptr;
    const size_t bytes = Vision::SSDNormalizeScratchBytes(batch, channel, spatial_dim, across_spatial);
    std::shared_ptr<Blob> temp;
    if (bytes > 0) {
      ws->GrowTempBuffer(bytes);
      temp = ws->CreateTempBlob({static_cast<int>((bytes + 3) / 4)}, DataType::kI32);
      scratch = temp->mutable_data<int>();
    }
    Vision::SSDNormalize<DeviceType::kGPU, float>(input->data<float>(), batch, channel, spatial_dim,
                                                  across_spatial, eps, scale_data, channel_shared,
                                                  scratch, output->mutable_data<float>(),
                                                  ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(SSDNormalizeGPU, SSDNormalizeKernelHip);

}  // namespace Shadow
