#include "shadow/kernels/eltwise.hpp"

#include "shadow_hip.h"

namespace Shadow {

// One pass over K inputs instead of Set + K x Saxpy (or K-1 chained binary
// kernels): shadow/operators/kernels/eltwise.hpp:28-65 makes 1 + 3K memory
// passes for a sum, this makes K reads and one write.  The evaluation order and
// the behaviour when the output aliases an input are those of the chain.
class EltwiseKernelHip : public EltwiseKernel {
 public:
  void Run(const std::vector<std::shared_ptr<Blob>>& inputs, std::shared_ptr<Blob>& output,
           Workspace* ws, int operation, const VecFloat& coeff) override {
    if (operation < kProd || operation > kMin) {
      LOG(FATAL) << "Unknown eltwise operation " << operation;
    }
    std::vector<const float*> ptrs;
    for (const auto& in : inputs) ptrs.push_back(in->data<float>());
    SHADOW_HIP_CHECK(shdw_hip_eltwise(operation, static_cast<int>(ptrs.size()), ptrs.data(),
                                      operation == kSum ? coeff.data() : nullptr,
                                      inputs[0]->count(), output->mutable_data<float>(),
                                      ws->Ctx()->stream()));
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(EltwiseGPU, EltwiseKernelHip);

}  // namespace Shadow
