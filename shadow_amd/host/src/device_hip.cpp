#include "shadow/device.hpp"

#include "level1_handle.hpp"
#include "shadow_hip.h"

namespace Shadow {

void hip_check(int rc, const char* what) {
  CHECK_EQ(rc, 0) << what << ": " << shdw_hip_error_string(rc);
}

// Declared before HipContext uses it.
template <>
std::shared_ptr<Allocator> GetAllocator<DeviceType::kGPU>();

namespace {

class HipAllocator : public Allocator {
 public:
  DeviceType device_type() const override { return DeviceType::kGPU; }

  void* malloc(size_t size, const void* host_ptr) const override {
    void* ptr = nullptr;
    SHADOW_HIP_CHECK(shdw_hip_malloc(&ptr, size));
    if (host_ptr != nullptr) write(size, host_ptr, ptr);
    return ptr;
  }
  void read(size_t size, const void* src, void* dst) const override {
    SHADOW_HIP_CHECK(shdw_hip_memcpy_d2h(dst, src, size, stream_));
  }
  void write(size_t size, const void* src, void* dst) const override {
    SHADOW_HIP_CHECK(shdw_hip_memcpy_h2d(dst, src, size, stream_));
  }
  void copy(size_t size, const void* src, void* dst) const override {
    SHADOW_HIP_CHECK(shdw_hip_memcpy_d2d(dst, src, size, stream_));
  }
  void free(void* ptr) const override { SHADOW_HIP_CHECK(shdw_hip_free(ptr)); }
  void set_stream(void* stream) override { stream_ = stream; }

 private:
  void* stream_ = nullptr;
};

class HipContext : public Context {
 public:
  explicit HipContext(const ArgumentHelper& arguments) {
    device_id_ = arguments.GetSingleArgument<int>("device_id", 0);
    int count = 0;
    SHADOW_HIP_CHECK(shdw_hip_device_count(&count));
    CHECK_GE(device_id_, 0);
    CHECK_LT(device_id_, count);
    if (arguments.GetSingleArgument<bool>("debug", false)) {
      char info[256] = {0};
      SHADOW_HIP_CHECK(shdw_hip_device_info(device_id_, info, sizeof(info)));
      LOG(INFO) << "GPU ID: " << device_id_ << ", " << info;
    }
    SHADOW_HIP_CHECK(shdw_hip_set_device(device_id_));
    // `default_cuda_stream` asked the reference for the per-thread default
    // stream; here it selects the null stream.
    own_stream_ = !arguments.GetSingleArgument<bool>("default_cuda_stream", false);
    if (own_stream_) {
      SHADOW_HIP_CHECK(shdw_hip_stream_create(&stream_));
      CHECK_NOTNULL(stream_);
    }
    allocator_ = GetAllocator<DeviceType::kGPU>();
    allocator_->set_stream(stream_);
    SHADOW_HIP_CHECK(shdw_hip_malloc(&level1_.scratch, kLevel1Scratch));
    level1_.bytes = kLevel1Scratch;
  }
  ~HipContext() override {
    if (level1_.scratch != nullptr) shdw_hip_free(level1_.scratch);
    if (own_stream_ && stream_ != nullptr) shdw_hip_stream_destroy(stream_);
  }

  Allocator* allocator() const override { return allocator_.get(); }
  DeviceType device_type() const override { return DeviceType::kGPU; }
  int device_id() const override { return device_id_; }
  void switch_device() override { SHADOW_HIP_CHECK(shdw_hip_set_device(device_id_)); }
  void synchronize() override { SHADOW_HIP_CHECK(shdw_hip_stream_sync(stream_)); }
  void* stream() const override { return stream_; }
  void* cublas_handle() const override { return const_cast<Level1Handle*>(&level1_); }

 private:
  int device_id_ = 0;
  bool own_stream_ = true;
  void* stream_ = nullptr;
  std::shared_ptr<Allocator> allocator_;
  // 4096 partial sums of 8 bytes and the result: what BlasSasum needs for any n
  static constexpr size_t kLevel1Scratch = 64 * 1024;
  Level1Handle level1_;
};

}  // namespace

template <>
std::shared_ptr<Allocator> GetAllocator<DeviceType::kGPU>() {
  return std::make_shared<HipAllocator>();
}

template <>
std::shared_ptr<Context> GetContext<DeviceType::kGPU>(const ArgumentHelper& arguments) {
  return std::make_shared<HipContext>(arguments);
}

}  // namespace Shadow
