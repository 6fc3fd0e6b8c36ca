#include "shadow/kernels/group_norm.hpp"

#include "shadow/kernels/layer_norm.hpp"
#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

size_t NormalizeRowsScratchBytes(int outer_num, int inner_num) {
  return shdw_hip_group_norm_workspace_bytes(outer_num, inner_num);
}

template <>
void NormalizeRows<DeviceType::kGPU, float>(const float* in_data, int outer_num, int inner_num,
                                            float eps, const float* scale_data,
                                            const float* bias_data, int scale_num,
                                            int scale_inner, float* out_data, void* scratch,
                                            size_t scratch_bytes, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_group_norm_ws(outer_num, inner_num, eps, in_data, scale_data, bias_data,
                                          scale_num, scale_inner, out_data, scratch, scratch_bytes,
                                          context->stream()));
}

// Scratch from the workspace's temp buffer, as the reference takes its mean /
// variance / temp blobs (group_norm.hpp:49-54); nullptr when the rows need none.
static void* NormalizeRowsScratch(Workspace* ws, int outer_num, int inner_num, size_t* bytes,
                                  std::shared_ptr<Blob>* hold) {
  *bytes = NormalizeRowsScratchBytes(outer_num, inner_num);
  if (*bytes == 0) return nullptr;
  ws->GrowTempBuffer(*bytes + 8);
  *hold = ws->CreateTempBlob({static_cast<int>((*bytes + 3) / 4)}, DataType::kI32);
  return (*hold)->mutable_data<int>();
}

}  // namespace Vision

// Rows are the (sample, group) slices; the affine step is per channel.
class GroupNormKernelHip : public GroupNormKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
           const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output, Workspace* ws,
           int group, float eps) override {
    const int count = input->count();
    const int outer_num = input->shape(0) * group, inner_num = count / outer_num;
    const float *scale_data = nullptr, *bias_data = nullptr;
    int channel = 1, spatial_dim = 1;
    if (scale != nullptr && bias != nullptr) {
      channel = input->shape(1), spatial_dim = input->count(2);
      CHECK_EQ(scale->count(), channel);
      CHECK_EQ(bias->count(), channel);
      scale_data = scale->data<float>(), bias_data = bias->data<float>();
    }
    size_t scratch_bytes = 0;
    std::shared_ptr<Blob> hold;
    void* scratch = Vision::NormalizeRowsScratch(ws, outer_num, inner_num, &scratch_bytes, &hold);
    Vision::NormalizeRows<DeviceType::kGPU, float>(
        input->data<float>(), outer_num, inner_num, eps, scale_data, bias_data, channel,
        spatial_dim, output->mutable_data<float>(), scratch, scratch_bytes, ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(GroupNormGPU, GroupNormKernelHip);

// Rows are the trailing `normalized_shape` dims; scale and bias have that shape.
class LayerNormKernelHip : public LayerNormKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
           const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output, Workspace* ws,
           const VecInt& normalized_shape, float eps) override {
    const int inner_num =
        input->count(input->num_axes() - static_cast<int>(normalized_shape.size()));
    const int count = input->count(), outer_num = count / inner_num;
    const float *scale_data = nullptr, *bias_data = nullptr;
    if (scale != nullptr && bias != nullptr) {
      CHECK(scale->shape() == normalized_shape);
      CHECK(bias->shape() == normalized_shape);
      scale_data = scale->data<float>(), bias_data = bias->data<float>();
    }
    size_t scratch_bytes = 0;
    std::shared_ptr<Blob> hold;
    void* scratch = Vision::NormalizeRowsScratch(ws, outer_num, inner_num, &scratch_bytes, &hold);
    Vision::NormalizeRows<DeviceType::kGPU, float>(
        input->data<float>(), outer_num, inner_num, eps, scale_data, bias_data, inner_num, 1,
        output->mutable_data<float>(), scratch, scratch_bytes, ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(LayerNormGPU, LayerNormKernelHip);

}  // namespace Shadow
