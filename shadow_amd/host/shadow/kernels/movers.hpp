// Kernel interfaces of the data movers:
//   shadow/operators/kernels/{concat,slice,stack,gather,pad,permute,reorg,
//   shuffle_channel,resize}.hpp
// The inner Vision:: functions keep the reference's signatures except Permute,
// whose order / step tables are host arrays here (nothing is uploaded).
#ifndef SHADOW_AMD_HOST_KERNELS_MOVERS_HPP_
#define SHADOW_AMD_HOST_KERNELS_MOVERS_HPP_

#include "shadow/blas.hpp"
#include "shadow/kernel.hpp"

namespace Shadow {

namespace Vision {

template <DeviceType D, typename T>
void Concat(const T* in_data, int count, int num_concats, int concat_size, int out_concat_axis,
            int in_concat_axis, int offset_concat_axis, T* out_data, Context* context);
template <DeviceType D, typename T>
void Slice(const T* in_data, int count, int num_slices, int slice_size, int in_slice_axis,
           int out_slice_axis, int offset_slice_axis, T* out_data, Context* context);
template <DeviceType D, typename T>
void Stack(const T* in_data, int count, int num_stacks, int stack_size, int out_stack_axis,
           int offset_stack_axis, T* out_data, Context* context);
template <DeviceType D, typename T>
void Gather(const T* in_data, const int* indexes_data, int num_indexes, int gather_dim,
            int inner_num, int count, T* out_data, Context* context);
// Fills the border with `value` as well (the reference does that with Blas::Set first).
template <DeviceType D, typename T>
void Pad(const T* in_data, const VecInt& in_shape, const VecInt& paddings, float value,
         T* out_data, Context* context);
template <DeviceType D, typename T>
void Permute(const T* in_data, const VecInt& in_shape, const VecInt& order, T* out_data,
             Context* context);
template <DeviceType D, typename T>
void Reorg(const T* in_data, const VecInt& in_shape, int type, int stride, T* out_data,
           Context* context);
template <DeviceType D, typename T>
void ShuffleChannel(const T* in_data, int batch, int channel, int spatial_dim, int group,
                    T* out_data, Context* context);
template <DeviceType D, typename T>
void ResizeNearest2D(const T* in_data, const VecInt& in_shape, const VecInt& out_shape,
                     T* out_data, Context* context);
template <DeviceType D, typename T>
void ResizeBilinear2D(const T* in_data, const VecInt& in_shape, bool align_corners,
                      const VecInt& out_shape, T* out_data, Context* context);

}  // namespace Vision

enum { kDarknet = 0, kNatural = 1 };  // Reorg types

class ConcatKernel : public Kernel {
 public:
  virtual void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
                   std::shared_ptr<Blob>& output, Workspace* ws, int axis) = 0;
};

class SliceKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input,
                   std::vector<std::shared_ptr<Blob>>& outputs, Workspace* ws, int axis) = 0;
};

class StackKernel : public Kernel {
 public:
  virtual void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
                   std::shared_ptr<Blob>& output, Workspace* ws, int axis) = 0;
};

class GatherKernel : public Kernel {
 public:
  // indexes: a 1-D int32 blob on the device
  virtual void Run(const std::shared_ptr<Blob>& input, const std::shared_ptr<Blob>& indexes,
                   std::shared_ptr<Blob>& output, Workspace* ws, int axis) = 0;
};

class PadKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, const VecInt& paddings, float value) = 0;
};

class PermuteKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, const VecInt& order_value) = 0;
};

class ReorgKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int type, int stride) = 0;
};

class ShuffleChannelKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int group) = 0;
};

class ResizeKernel : public Kernel {
 public:
  virtual void Run(const std::shared_ptr<Blob>& input, std::shared_ptr<Blob>& output,
                   Workspace* ws, int type, bool align_corners) = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNELS_MOVERS_HPP_
