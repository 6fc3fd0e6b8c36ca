// Pooling kernel interface: shadow/operators/kernels/pooling.hpp:8-70.
#ifndef SHADOW_AMD_HOST_KERNELS_POOLING_HPP_
#define SHADOW_AMD_HOST_KERNELS_POOLING_HPP_

#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {
// pool_type: 0 max, 1 average
template <DeviceType D, typename T>
void Pooling2D(const T* in_data, const VecInt& in_shape, int pool_type, int kernel_size_h,
               int kernel_size_w, int stride_h, int stride_w, int pad_h, int pad_w,
               const VecInt& out_shape, T* out_data, Context* context);
template <DeviceType D, typename T>
void Pooling3D(const T* in_data, const VecInt& in_shape, int pool_type, int kernel_size_d,
               int kernel_size_h, int kernel_size_w, int stride_d, int stride_h, int stride_w,
               int pad_d, int pad_h, int pad_w, const VecInt& out_shape, T* out_data,
               Context* context);
}  // namespace Vision

class PoolingKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int pool_type, int kernel_size_h, int kernel_size_w,
                   int stride_h, int stride_w, int pad_h, int pad_w, bool full_pooling) = 0;
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int pool_type, int kernel_size_d, int kernel_size_h,
                   int kernel_size_w, int stride_d, int stride_h, int stride_w, int pad_d,
                   int pad_h, int pad_w, bool full_pooling) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_POOLING_HPP_
