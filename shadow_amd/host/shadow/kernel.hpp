// Second-level dispatch: every operator owns a Kernel chosen by
// (operator type, device type, implementation flavour).  Surface and key format
// follow shadow/core/kernel.hpp:13-43 and shadow/core/kernel.cpp:5-56:
//   key = <OpType><"CPU"|"GPU">(<flavour>),  e.g. "UnaryGPU(Default)".
// Only "...GPU(Default)" kernels are registered by this build.  No key containing
// "CUDNN" may be registered: that flavour outranks Default on the GPU.
#ifndef SHADOW_AMD_HOST_KERNEL_HPP_
#define SHADOW_AMD_HOST_KERNEL_HPP_

#include <memory>
#include <string>

#include "blob.hpp"
#include "registry.hpp"
#include "workspace.hpp"

namespace Shadow {

class Kernel {
 public:
  virtual ~Kernel() = default;
  virtual DeviceType device_type() const = 0;
  virtual std::string kernel_type() const = 0;
};

// All registered keys that mention the device ("CPU"/"GPU"), optionally
// narrowed to one operator type.  Matching is by substring, as in the reference.
VecString GetKernelKeys(DeviceType device_type);
VecString GetKernelKeys(const std::string& op_type, DeviceType device_type);

// kernel_type "" picks the best registered flavour (GPU: CUDNN, then Default).
// Throws when nothing matches.
std::shared_ptr<Kernel> CreateKernel(const std::string& op_type, DeviceType device_type,
                                     const std::string& kernel_type = "");

SHADOW_DECLARE_REGISTRY(KernelRegistry, Kernel);

#define REGISTER_OP_KERNEL(name, ...) SHADOW_REGISTER_CLASS(KernelRegistry, name, __VA_ARGS__)
#define REGISTER_OP_KERNEL_DEFAULT(name, ...) REGISTER_OP_KERNEL(name(Default), __VA_ARGS__)
#define REGISTER_OP_KERNEL_DNNL(name, ...) REGISTER_OP_KERNEL(name(DNNL), __VA_ARGS__)
#define REGISTER_OP_KERNEL_CUDNN(name, ...) REGISTER_OP_KERNEL(name(CUDNN), __VA_ARGS__)

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_KERNEL_HPP_
