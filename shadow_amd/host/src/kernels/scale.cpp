#include "shadow/kernels/scale.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void ScaleBias<DeviceType::kGPU, float>(const float* in_data, int count, const float* scale_data,
                                        const float* bias_data, int scale_num, int inner_num,
                                        float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_scale_bias(count, scale_num, inner_num, in_data, scale_data, bias_data,
                                       0, out_data, context->stream()));
}

template <>
void Scale<DeviceType::kGPU, float>(const float* in_data, int count, const float* scale_data,
                                    int scale_num, int inner_num, float* out_data,
                                    Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_scale_bias(count, scale_num, inner_num, in_data, scale_data, nullptr,
                                       0, out_data, context->stream()));
}

template <>
void Bias<DeviceType::kGPU, float>(const float* in_data, int count, const float* bias_data,
                                   int scale_num, int inner_num, float* out_data,
                                   Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_scale_bias(count, scale_num, inner_num, in_data, nullptr, bias_data,
                                       0, out_data, context->stream()));
}

}  // namespace Vision

class ScaleKernelHip : public ScaleKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
           const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output, Workspace* ws,
           int axis) override {
    CHECK(scale != nullptr || bias != nullptr);
    if (scale != nullptr && bias != nullptr) CHECK(scale->shape() == bias->shape());
    const auto& param = scale != nullptr ? scale : bias;
    // The parameter blob covers axes [axis, axis + its rank); what follows is
    // the contiguous run one parameter applies to.
    const int inner_num = input->count(axis + param->num_axes());
    launch(input, scale != nullptr ? scale->data<float>() : nullptr,
           bias != nullptr ? bias->data<float>() : nullptr, param->count(), inner_num, output, ws);
  }

  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int axis, const VecFloat& scale_value, const VecFloat& bias_value) override {
    const int dim = input->shape(axis), inner_num = input->count(axis + 1);
    CHECK(!scale_value.empty() || !bias_value.empty());
    if (!scale_value.empty()) CHECK_EQ(scale_value.size(), dim);
    if (!bias_value.empty()) CHECK_EQ(bias_value.size(), dim);
    // Per-channel values arrive as host vectors; they are staged in the temp
    // buffer on every call, like shadow/operators/kernels/scale.hpp:84-107.
    ws->GrowTempBuffer(2 * dim * sizeof(float));
    const float *scale_ptr = nullptr, *bias_ptr = nullptr;
    if (!scale_value.empty()) {
      auto blob = ws->CreateTempBlob({dim}, DataType::kF32);
      blob->set_data<float>(scale_value.data(), dim);
      scale_ptr = blob->data<float>();
    }
    if (!bias_value.empty()) {
      auto blob = ws->CreateTempBlob({dim}, DataType::kF32);
      blob->set_data<float>(bias_value.data(), dim);
      bias_ptr = blob->data<float>();
    }
    launch(input, scale_ptr, bias_ptr, dim, inner_num, output, ws);
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }

 private:
  static void launch(const std::shared_ptr<Blob>& input, const float* scale, const float* bias,
                     int scale_num, int inner_num, std::shared_ptr<Blob>& output, Workspace* ws) {
    auto* ctx = ws->Ctx().get();
    const float* in = input->data<float>();
    float* out = output->mutable_data<float>();
    const int count = input->count();
    if (scale != nullptr && bias != nullptr) {
      Vision::ScaleBias<DeviceType::kGPU, float>(in, count, scale, bias, scale_num, inner_num, out, ctx);
    } else if (scale != nullptr) {
      Vision::Scale<DeviceType::kGPU, float>(in, count, scale, scale_num, inner_num, out, ctx);
    } else {
      Vision::Bias<DeviceType::kGPU, float>(in, count, bias, scale_num, inner_num, out, ctx);
    }
  }
};

REGISTER_OP_KERNEL_DEFAULT(ScaleGPU, ScaleKernelHip);

}  // namespace Shadow
