#include "shadow/kernels/reduce.hpp"

#include "shadow_hip.h"

namespace Shadow {

namespace Vision {

template <>
void Reduce<DeviceType::kGPU, float>(const float* in_data, const int* in_shape, int num_axes,
                                     const int* axes, int num_reduce, int operation,
                                     float* out_data, void* workspace, size_t workspace_bytes,
                                     Context* context) {
  SHADOW_HIP_CHECK(shdw_hip_reduce(operation, num_axes, in_shape, num_reduce, axes, in_data,
                                   out_data, workspace, workspace_bytes, context->stream()));
}

}  // namespace Vision

// The reference builds one index list per window plus one offset per output on
// the host and uploads both on every call (51 MB for a full-tensor sum,
// shadow/operators/kernels/reduce.hpp:45-82).  Here only the collapsed extents
// travel, as kernel arguments; the temp buffer holds the per-slice partials
// of two-stage reductions and nothing else.
class ReduceKernelHip : public ReduceKernel {
 public:
  void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output, Workspace* ws,
           int operation, const VecInt& axes) override {
    if (operation < kProd || operation > kLpNorm2) {
      LOG(FATAL) << "Unknown reduce operation " << operation;
    }
    const auto& shape = input->shape();
    const int num_axes = input->num_axes(), num_reduce = static_cast<int>(axes.size());
    for (int axis : axes) {
      // The reference indexes its stride table with the raw value, so a negative
      // axis reads out of bounds there; it is refused here.
      CHECK_GE(axis, 0) << "Reduce: negative axes are not supported";
      CHECK_LT(axis, num_axes);
    }
    const size_t bytes = shdw_hip_reduce_workspace_bytes(num_axes, shape.data(), num_reduce, axes.data());
    void* scratch = nullptr;
    if (bytes > 0) {
      ws->GrowTempBuffer(bytes);
      auto temp = ws->CreateTempBlob({static_cast<int>((bytes + 3) / 4)}, DataType::kI32);
      scratch = temp->mutable_data<int>();
    }
    Vision::Reduce<DeviceType::kGPU, float>(input->data<float>(), shape.data(), num_axes,
                                            axes.data(), num_reduce, operation,
                                            output->mutable_data<float>(), scratch, bytes,
                                            ws->Ctx().get());
  }

  DeviceType device_type() const override { return DeviceType::kGPU; }
  std::string kernel_type() const override { return "Default"; }
};

REGISTER_OP_KERNEL_DEFAULT(ReduceGPU, ReduceKernelHip);

}  // namespace Shadow
