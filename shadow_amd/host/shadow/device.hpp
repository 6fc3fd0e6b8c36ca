// Device runtime seen by Blob / Workspace / operators: the Allocator and Context
// interfaces of shadow/core/allocator.hpp:8-30 and shadow/core/context.hpp:11-32.
// This build provides the DeviceType::kGPU pair only, implemented over the
// shdw_hip_* C ABI (src/device_hip.cpp); there is no CPU compute path.
#ifndef SHADOW_AMD_HOST_DEVICE_HPP_
#define SHADOW_AMD_HOST_DEVICE_HPP_

#include <cstddef>
#include <memory>

#include "params.hpp"

namespace Shadow {

enum class DeviceType { kCPU, kGPU, kNPU };

class Allocator {
 public:
  virtual ~Allocator() = default;

  virtual DeviceType device_type() const = 0;
  // Allocates `size` bytes; when host_ptr is non-null its contents are copied in.
  virtual void* malloc(size_t size, const void* host_ptr) const = 0;
  virtual void read(size_t size, const void* src, void* dst) const = 0;   // device -> host
  virtual void write(size_t size, const void* src, void* dst) const = 0;  // host -> device
  virtual void copy(size_t size, const void* src, void* dst) const = 0;   // device -> device
  virtual void free(void* ptr) const = 0;
  // After this the three copies are enqueued on `stream` instead of blocking.
  virtual void set_stream(void* stream) = 0;
};

template <DeviceType D>
std::shared_ptr<Allocator> GetAllocator();

class Context {
 public:
  virtual ~Context() = default;

  virtual Allocator* allocator() const = 0;
  virtual DeviceType device_type() const = 0;
  virtual int device_id() const = 0;
  virtual void switch_device() = 0;
  virtual void synchronize() = 0;
  virtual void* stream() const { return nullptr; }

  // Vendor-library handles of the reference.  The GPU context of this build answers
  // cublas_handle() with its Level1Handle (src/level1_handle.hpp): the device scratch
  // of the level-1 routines, which is what the cuBLAS handle's own workspace was.
  // Nothing on this path uses the other three.
  virtual void* cublas_handle() const { return nullptr; }
  virtual void* cudnn_handle() const { return nullptr; }
  virtual void* nnpack_handle() const { return nullptr; }
  virtual void* dnnl_handle() const { return nullptr; }
};

// Reads `device_id` (default 0) from the arguments, as
// shadow/core/context.cu:9-16 does.
template <DeviceType D>
std::shared_ptr<Context> GetContext(const ArgumentHelper& arguments);

// CHECK that a shdw_hip_* call returned 0; the message carries the text of
// shdw_hip_error_string, like CUDA_CHECK (shadow/core/external.hpp:39-43).
void hip_check(int rc, const char* what);
#define SHADOW_HIP_CHECK(call) ::Shadow::hip_check((call), #call)

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_DEVICE_HPP_
