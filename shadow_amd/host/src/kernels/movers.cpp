#include "shadow/kernels/movers.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Concat<DeviceType::kGPU, float>(const float* in_data, int count, int num_concats,
                                     int concat_size, int out_concat_axis, int in_concat_axis,
                                     int offset_concat_axis, float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_copy_chunks(num_concats, in_concat_axis * concat_size, in_data,
                                        in_concat_axis * concat_size, 0, out_data,
                                        out_concat_axis * concat_size,
                                        offset_concat_axis * concat_size, context->stream()));
}

template <>
void Slice<DeviceType::kGPU, float>(const float* in_data, int count, int num_slices,
                                    int slice_size, int in_slice_axis, int out_slice_axis,
                                    int offset_slice_axis, float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_copy_chunks(num_slices, out_slice_axis * slice_size, in_data,
                                        in_slice_axis * slice_size, offset_slice_axis * slice_size,
                                        out_data, out_slice_axis * slice_size, 0,
                                        context->stream()));
}

template <>
void Stack<DeviceType::kGPU, float>(const float* in_data, int count, int num_stacks,
                                    int stack_size, int out_stack_axis, int offset_stack_axis,
                                    float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_copy_chunks(num_stacks, stack_size, in_data, stack_size, 0, out_data,
                                        out_stack_axis * stack_size,
                                        offset_stack_axis * stack_size, context->stream()));
}

template <>
void Gather<DeviceType::kGPU, float>(const float* in_data, const int* indexes_data,
                                     int num_indexes, int gather_dim, int inner_num, int count,
                                     float* out_data, Context* context) {
  const int row = num_indexes * inner_num;
  SHADOW_HIP_CHECK(shdw_hip_gather(row > 0 ? count / row : 0, gather_dim, inner_num, num_indexes,
                                   indexes_data, in_data, out_data, context->stream()));
}

template <>
void Pad<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                  const VecInt& paddings, float value, float* out_data,
                                  Context* context) {
  CHECK_EQ(in_shape.size(), 4);
  CHECK_EQ(paddings.size(), 4);
  SHADOW_HIP_CHECK(shdw_hip_pad(in_shape.data(), paddings.data(), value, in_data, out_data,
                                context->stream()));
}

template <>
void Permute<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                      const VecInt& order, float* out_data, Context* context) {
  CHECK_EQ(in_shape.size(), order.size());
  SHADOW_HIP_CHECK(shdw_hip_permute(static_cast<int>(in_shape.size()), in_shape.data(),
                                    order.data(), in_data, out_data, context->stream()));
}

template <>
void Reorg<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape, int type,
                                    int stride, float* out_data, Context* context) {
  CHECK_EQ(in_shape.size(), 4);
  if (type != kDarknet && type != kNatural) LOG(FATAL) << "Unsupported reorg type: " << type;
  SHADOW_HIP_CHECK(shdw_hip_reorg(in_shape.data(), type, stride, in_data, out_data,
                                  context->stream()));
}

template <>
void ShuffleChannel<DeviceType::kGPU, float>(const float* in_data, int batch, int channel,
                                             int spatial_dim, int group, float* out_data,
                                             Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_shuffle_channel(batch, channel, spatial_dim, group, in_data, out_data,
                                            context->stream()));
}

template <>
void ResizeNearest2D<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                              const VecInt& out_shape, float* out_data,
                                              Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_resize(in_shape.data(), out_shape.data(), 0, 0, in_data, out_data,
                                   context->stream()));
}

template <>
void ResizeBilinear2D<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                               bool align_corners, const VecInt& out_shape,
                                               float* out_data, Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_resize(in_shape.data(), out_shape.data(), 1, align_corners ? 1 : 0,
                                   in_data, out_data, context->stream()));
}

}  // namespace Vision

namespace {
constexpr DeviceType kDev = DeviceType::kGPU;
}

// One pitched copy per input; the running offset along the axis is kept on the host.
class ConcatKernelHip : public ConcatKernel {
 public:
  void Run(const std::vector<std::shared_ptr<Blob>>& inputs, std::shared_ptr<Blob>& output,
           Workspace* ws, int axis) override {
    int offset_concat_axis = 0;
    const int num_concats = output->count(0, axis), concat_size = output->count(axis + 1);
    const int out_concat_axis = output->shape(axis);
    for (const auto& input : inputs) {
      const int in_concat_axis = input->shape(axis);
      Vision::Concat<kDev, float>(input->data<float>(), input->count(), num_concats, concat_size,
                                  out_concat_axis, in_concat_axis, offset_concat_axis,
                                  output->mutable_data<float>(), ws->Ctx().get());
      offset_concat_axis += in_concat_axis;
    }
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(ConcatGPU, ConcatKernelHip);

class SliceKernelHip : public SliceKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::vector<std::shared_ptr<Blob>>& outputs,
           Workspace* ws, int axis) override {
    int offset_slice_axis = 0;
    const int num_slices = input->count(0, axis), slice_size = input->count(axis + 1);
    const int in_slice_axis = input->shape(axis);
    for (auto& output : outputs) {
      const int out_slice_axis = output->shape(axis);
      Vision::Slice<kDev, float>(input->data<float>(), output->count(), num_slices, slice_size,
                                 in_slice_axis, out_slice_axis, offset_slice_axis,
                                 output->mutable_data<float>(), ws->Ctx().get());
      offset_slice_axis += out_slice_axis;
    }
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(SliceGPU, SliceKernelHip);

class StackKernelHip : public StackKernel {
 public:
  void Run(const std::vector<std::shared_ptr<Blob>>& inputs, std::shared_ptr<Blob>& output,
           Workspace* ws, int axis) override {
    const int num_stacks = output->count(0, axis), stack_size = output->count(axis + 1);
    const int out_stack_axis = output->shape(axis);
    for (int n = 0; n < static_cast<int>(inputs.size()); ++n) {
      CHECK(inputs[n]->shape() == inputs[0]->shape()) << "Stacked inputs must have one shape";
      Vision::Stack<kDev, float>(inputs[n]->data<float>(), inputs[n]->count(), num_stacks,
                                 stack_size, out_stack_axis, n, output->mutable_data<float>(),
                                 ws->Ctx().get());
    }
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(StackGPU, StackKernelHip);

class GatherKernelHip : public GatherKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& indexes,
           std::shared_ptr<Blob>& output, Workspace* ws, int axis) override {
    Vision::Gather<kDev, float>(input->data<float>(), indexes->data<int>(), indexes->count(),
                                input->shape(axis), input->count(axis + 1), output->count(),
                                output->mutable_data<float>(), ws->Ctx().get());
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(GatherGPU, GatherKernelHip);

class PadKernelHip : public PadKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           const VecInt& paddings, float value) override {
    if (paddings[0] == 0 && paddings[1] == 0 && paddings[2] == 0 && paddings[3] == 0) {
      Blas::BlasScopy<kDev, float>(input->count(), input->data<float>(), 0,
                                   output->mutable_data<float>(), 0, ws->Ctx().get());
    } else {
      Vision::Pad<kDev, float>(input->data<float>(), input->shape(), paddings, value,
                               output->mutable_data<float>(), ws->Ctx().get());
    }
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(PadGPU, PadKernelHip);

class PermuteKernelHip : public PermuteKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           const VecInt& order_value) override {
    Vision::Permute<kDev, float>(input->data<float>(), input->shape(), order_value,
                                 output->mutable_data<float>(), ws->Ctx().get());
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(PermuteGPU, PermuteKernelHip);

class ReorgKernelHip : public ReorgKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int type, int stride) override {
    Vision::Reorg<kDev, float>(input->data<float>(), input->shape(), type, stride,
                               output->mutable_data<float>(), ws->Ctx().get());
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(ReorgGPU, ReorgKernelHip);

class ShuffleChannelKernelHip : public ShuffleChannelKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int group) override {
    Vision::ShuffleChannel<kDev, float>(input->data<float>(), input->shape(0), input->shape(1),
                                        input->count(2), group, output->mutable_data<float>(),
                                        ws->Ctx().get());
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(ShuffleChannelGPU, ShuffleChannelKernelHip);

class ResizeKernelHip : public ResizeKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int type, bool align_corners) override {
    if (output->shape(2) == input->shape(2) && output->shape(3) == input->shape(3)) {
      Blas::BlasScopy<kDev, float>(input->count(), input->data<float>(), 0,
                                   output->mutable_data<float>(), 0, ws->Ctx().get());
    } else if (type == 0) {
      Vision::ResizeNearest2D<kDev, float>(input->data<float>(), input->shape(), output->shape(),
                                           output->mutable_data<float>(), ws->Ctx().get());
    } else {
      Vision::ResizeBilinear2D<kDev, float>(input->data<float>(), input->shape(), align_corners,
                                            output->shape(), output->mutable_data<float>(),
                                            ws->Ctx().get());
    }
  }
  DeviceType device_type() const override { return kDev; }
  std::string kernel_type() const override { return "Default"; }
};
REGISTER_OP_KERNEL_DEFAULT(ResizeGPU, ResizeKernelHip);

}  // namespace Shadow
