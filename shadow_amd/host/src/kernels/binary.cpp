#include "shadow/kernels/binary.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void BroadcastBinary<DeviceType::kGPU, float>(const float* in_data, const int* in_shape,
                                              const float* scalar_data, const int* scalar_shape,
                                              int operation, int num_axes, int count,
                                              const int* out_shape, float* out_data,
                                              Context* context) {
  (void)count;  // implied by out_shape
  SHADOW_HIP_CHECK(shdw_hip_broadcast_binary(operation, num_axes, in_shape, scalar_shape,
                                             out_shape, in_data, scalar_data, out_data,
                                             context->stream()));
}

}  // namespace Vision

class BinaryKernelHip : public BinaryKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int operation, float scalar_value) override {
    check(operation);
    SHADOW_HIP_CHECK(shdw_hip_binary_scalar(operation, input->count(), input->data<float>(),
                                            scalar_value, output->mutable_data<float>(),
                                            ws->Ctx()->stream()));
  }

  void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scalar,
           std::shared_ptr<Blob>& output, Workspace* ws, int operation,
           bool need_broadcast) override {
    check(operation);
    if (need_broadcast) {
      // The reference uploads three shape arrays into temp blobs on every call
      // (shadow/operators/kernels/binary.hpp:81-92).  The host vectors are
      // enough here, so no temp buffer and no copies.
      Vision::BroadcastBinary<DeviceType::kGPU, float>(
          input->data<float>(), input->shape().data(), scalar->data<float>(),
          scalar->shape().data(), operation, input->num_axes(), output->count(),
          output->shape().data(), output->mutable_data<float>(), ws->Ctx().get());
    } else {
      SHADOW_HIP_CHECK(shdw_hip_binary(operation, input->count(), input->data<float>(),
                                       scalar->data<float>(), output->mutable_data<float>(),
                                       ws->Ctx()->stream()));
    }
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }

 private:
  static void check(int operation) {
    if (operation < kAdd || operation > kMin) LOG(FATAL) << "Unknown binary operation " << operation;
  }
};

REGISTER_OP_KERNEL_DEFAULT(BinaryGPU, BinaryKernelHip);

}  // namespace Shadow
