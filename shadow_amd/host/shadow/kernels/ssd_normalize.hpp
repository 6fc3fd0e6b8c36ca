// SSDNormalize kernel interface: shadow/operators/kernels/ssd_normalize.hpp:15-33.
// Vision::SSDNormalize here covers both forms and the optional scale in one
// device call, so there is no Square / Sasum / Mul / Sscal / Scale sequence and
// no per-item return to the host.
#ifndef SHADOW_AMD_HOST_KERNELS_SSD_NORMALIZE_HPP_
#define SHADOW_AMD_HOST_KERNELS_SSD_NORMALIZE_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// scale_data: nullptr, one value (channel_shared) or `channel` values.
// val_data: device scratch of SSDNormalizeScratchBytes(...) bytes (may be
// nullptr when that is 0).
template <DeviceType D, typename T>
void SSDNormalize(const T* in_data, int outer_num, int channel, int inner_num, bool across_spatial,
                  float eps, const T* scale_data, bool channel_shared, void* val_data, T* out_data,
                  Context* context);
size_t SSDNormalizeScratchBytes(int outer_num, int channel, int inner_num, bool across_spatial);
}  // namespace Vision

class SSDNormalizeKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& scale,
                   std::shared_ptr<Blob>& output, Workspace* ws, bool across_spatial,
                   bool channel_shared, float eps) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_SSD_NORMALIZE_HPP_
