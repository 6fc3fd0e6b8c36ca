#include "shadow/kernels/pooling.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Pooling2D<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                        int pool_type, int kernel_size_h, int kernel_size_w,
                                        int stride_h, int stride_w, int pad_h, int pad_w,
                                        const VecInt& out_shape, float* out_data,
                                        Context* context) {
  CHECK_EQ(in_shape.size(), 4);
  CHECK_EQ(out_shape.size(), 4);
  SHADOW_HIP_CHECK(shdw_hip_pooling2d(in_shape.data(), pool_type, kernel_size_h, kernel_size_w,
                                      stride_h, stride_w, pad_h, pad_w, out_shape.data(), in_data,
                                      out_data, context->stream()));
}

template <>
void Pooling3D<DeviceType::kGPU, float>(const float* in_data, const VecInt& in_shape,
                                        int pool_type, int kernel_size_d, int kernel_size_h,
                                        int kernel_size_w, int stride_d, int stride_h,
                                        int stride_w, int pad_d, int pad_h, int pad_w,
                                        const VecInt& out_shape, float* out_data,
                                        Context* context) {
  CHECK_EQ(in_shape.size(), 5);
  CHECK_EQ(out_shape.size(), 5);
  SHADOW_HIP_CHECK(shdw_hip_pooling3d(in_shape.data(), pool_type, kernel_size_d, kernel_size_h,
                                      kernel_size_w, stride_d, stride_h, stride_w, pad_d, pad_h,
                                      pad_w, out_shape.data(), in_data, out_data,
                                      context->stream()));
}

}  // namespace Vision

class PoolingKernelHip : public PoolingKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int pool_type, int kernel_size_h, int kernel_size_w, int stride_h, int stride_w,
           int pad_h, int pad_w, bool full_pooling) override {
    Vision::Pooling2D<DeviceType::kGPU, float>(
        input->data<float>(), input->shape(), pool_type, kernel_size_h, kernel_size_w, stride_h,
        stride_w, pad_h, pad_w, output->shape(), output->mutable_data<float>(), ws->Ctx().get());
  }

  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int pool_type, int kernel_size_d, int kernel_size_h, int kernel_size_w, int stride_d,
           int stride_h, int stride_w, int pad_d, int pad_h, int pad_w,
           bool full_pooling) override {
    Vision::Pooling3D<DeviceType::kGPU, float>(
        input->data<float>(), input->shape(), pool_type, kernel_size_d, kernel_size_h,
        kernel_size_w, stride_d, stride_h, stride_w, pad_d, pad_h, pad_w, output->shape(),
        output->mutable_data<float>(), ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(PoolingGPU, PoolingKernelHip);

}  // namespace Shadow
