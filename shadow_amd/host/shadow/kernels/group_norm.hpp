// GroupNorm kernel interface (also used by InstanceNorm):
// shadow/operators/kernels/group_norm.hpp:8-36.  The reference's inner
// Vision::SubtractMeanAndSquare / Vision::DivideVariance layer and its Sgemv row
// sums are one device call here, so they have no counterpart.
#ifndef SHADOW_AMD_HOST_KERNELS_GROUP_NORM_HPP_
#define SHADOW_AMD_HOST_KERNELS_GROUP_NORM_HPP_

#include <cstddef>

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// x viewed as [outer_num][inner_num]: (x - mean) / sqrt(var + eps) per row, then
// y * scale[c] + bias[c] with c = (i / scale_inner) % scale_num when scale_data
// and bias_data are not null.
// scratch: NormalizeRowsScratchBytes(outer_num, inner_num) bytes of device memory
// (8-byte aligned; nullptr where that is 0), where rows too long and too few for
// a workgroup each leave their partial sums.
size_t NormalizeRowsScratchBytes(int outer_num, int inner_num);
template <DeviceType D, typename T>
void NormalizeRows(const T* in_data, int outer_num, int inner_num, float eps, const T* scale_data,
                   const T* bias_data, int scale_num, int scale_inner, T* out_data, void* scratch,
                   size_t scratch_bytes, Context* context);
}  // namespace Vision

class GroupNormKernel : public Kernel {
 public:
  // scale and bias: both blobs or both nullptr
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
                   const std::shared_ptr<Blob>& bias, std::shared_ptr<Blob>& output,
                   Workspace* ws, int group, float eps) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_GROUP_NORM_HPP_
