#include "shadow/kernels/activate.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Activate<DeviceType::kGPU, float>(const float* in_data, float* out_data, int count, int type,
                                       float slope, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_activate(type, slope, count, in_data, out_data, context->stream()));
}

template <>
void PRelu<DeviceType::kGPU, float>(const float* in_data, float* out_data, const VecInt& in_shape,
                                    bool channel_shared, const float* slope_data,
                                    Context* context) {
  const int channels = in_shape[1];
  int dim = 1;
  for (size_t i = 2; i < in_shape.size(); ++i) dim *= in_shape[i];
  const int count = in_shape[0] * channels * dim;
  SHADOW_HIP_CHECK(shdw_hip_prelu(count, channels, dim, channel_shared ? 1 : 0, in_data,
                                  slope_data, out_data, context->stream()));
}

}  // namespace Vision

class ActivateKernelHip : public ActivateKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& slope,
           std::shared_ptr<Blob>& output, Workspace* ws, int activate_type,
           float slope_val) override {
    if (activate_type == kPRelu) {
      CHECK_GE(input->num_axes(), 2);
      CHECK_NOTNULL(slope);
      const bool channel_shared = slope->count() == 1;
      if (!channel_shared) CHECK_EQ(slope->count(), input->shape(1));
      Vision::PRelu<DeviceType::kGPU, float>(input->data<float>(), output->mutable_data<float>(),
                                             output->shape(), channel_shared,
                                             slope->data<float>(), ws->Ctx().get());
    } else if (activate_type >= kRelu && activate_type <= kGelu) {
      Vision::Activate<DeviceType::kGPU, float>(input->data<float>(),
                                                output->mutable_data<float>(), output->count(),
                                                activate_type, slope_val, ws->Ctx().get());
    }
    // Any other value leaves the output untouched, as in
    // shadow/operators/kernels/activate.hpp:51-70.
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(ActivateGPU, ActivateKernelHip);

}  // namespace Shadow
