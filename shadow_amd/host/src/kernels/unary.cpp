#include "shadow/kernels/unary.hpp"

#include "shadow_hip.h"

namespace Shadow {

// All 15 operations share one templated device kernel; the enum values are the
// C ABI's (shadow/operators/kernels/unary.hpp:9-25 == SHDW_UNARY_*).
class UnaryKernelHip : public UnaryKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int operation) override {
    if (operation < kAbs || operation > kReciprocal) {
      LOG(FATAL) << "Unknown unary operation " << operation;
    }
    SHADOW_HIP_CHECK(shdw_hip_unary(operation, input->count(), input->data<float>(),
                                    output->mutable_data<float>(), ws->Ctx()->stream()));
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(UnaryGPU, UnaryKernelHip);

}  // namespace Shadow
