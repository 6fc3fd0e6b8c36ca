// Blob: a named, typed, dense row-major tensor handle over an Allocator, with the
// public surface of shadow/core/blob.hpp:28-223.  There is no stride field:
// "NCHW" is only the order of the shape vector.  Element counts are int32.
#ifndef SHADOW_AMD_HOST_BLOB_HPP_
#define SHADOW_AMD_HOST_BLOB_HPP_

#include <cstdint>
#include <string>
#include <type_traits>
#include <typeinfo>
#include <vector>

#include "device.hpp"
#include "log.hpp"

namespace Shadow {

using VecInt = std::vector<int>;
using VecFloat = std::vector<float>;
using VecString = std::vector<std::string>;

// Same enumerators, same order as shadow/core/blob.hpp:15-26.
enum class DataType { kI64, kI32, kI16, kI8, kU64, kU32, kU16, kU8, kF32, kBool };

namespace detail {
template <typename T> struct dtype_of;
template <> struct dtype_of<std::int64_t> { static constexpr DataType value = DataType::kI64; };
template <> struct dtype_of<std::int32_t> { static constexpr DataType value = DataType::kI32; };
template <> struct dtype_of<std::int16_t> { static constexpr DataType value = DataType::kI16; };
template <> struct dtype_of<std::int8_t> { static constexpr DataType value = DataType::kI8; };
template <> struct dtype_of<std::uint64_t> { static constexpr DataType value = DataType::kU64; };
template <> struct dtype_of<std::uint32_t> { static constexpr DataType value = DataType::kU32; };
template <> struct dtype_of<std::uint16_t> { static constexpr DataType value = DataType::kU16; };
template <> struct dtype_of<std::uint8_t> { static constexpr DataType value = DataType::kU8; };
template <> struct dtype_of<float> { static constexpr DataType value = DataType::kF32; };
template <> struct dtype_of<bool> { static constexpr DataType value = DataType::kBool; };

inline size_t dtype_size(DataType t) {
  switch (t) {
    case DataType::kI64: case DataType::kU64: return 8;
    case DataType::kI32: case DataType::kU32: case DataType::kF32: return 4;
    case DataType::kI16: case DataType::kU16: return 2;
    case DataType::kI8: case DataType::kU8: return 1;
    case DataType::kBool: return sizeof(bool);
  }
  return 0;
}
}  // namespace detail

class Blob {
 public:
  Blob(std::string name, DataType data_type, Allocator* allocator)
      : name_(std::move(name)), data_type_(data_type), allocator_(allocator) {
    CHECK_NOTNULL(allocator_);
  }
  Blob(const Blob&) = delete;
  Blob& operator=(const Blob&) = delete;
  ~Blob() { release(); }

  // Raw typed views of the device buffer; no type check, as in the reference.
  template <typename T>
  const T* data() const { return static_cast<const T*>(data_); }
  template <typename T>
  T* mutable_data() { return static_cast<T*>(data_); }

  // Host copy of the contents (kept inside the blob until the next call).
  template <typename T>
  const T* cpu_data() {
    require_type<T>();
    if (allocator_->device_type() == DeviceType::kCPU) return data<T>();
    host_copy_.resize(raw_size(), 0);
    get_data<T>(host_copy_.data(), count());
    return reinterpret_cast<const T*>(host_copy_.data());
  }

  template <typename T>
  void set_data(const void* cpu_data, int set_count, int offset = 0) {
    require_type<T>();
    CHECK_NOTNULL(cpu_data);
    CHECK_LE(set_count + offset, count());
    CHECK_NOTNULL(data_);
    allocator_->write(set_count * elem_size(), cpu_data, mutable_data<T>() + offset);
  }

  template <typename T>
  void get_data(void* cpu_data, int get_count, int offset = 0) const {
    require_type<T>();
    CHECK_NOTNULL(cpu_data);
    CHECK_LE(get_count + offset, count());
    CHECK_NOTNULL(data_);
    allocator_->read(get_count * elem_size(), data<T>() + offset, cpu_data);
  }

  // set_data for callers that do not know the element type statically: copies
  // raw_size() bytes from the host.
  void set_raw_data(const void* cpu_data) {
    CHECK_NOTNULL(cpu_data);
    CHECK_NOTNULL(data_);
    allocator_->write(raw_size(), cpu_data, data_);
  }

  // Alias memory owned by someone else; this blob will never free it.
  void share_data(const void* data, const VecInt& shape) {
    CHECK_NOTNULL(data);
    release();
    data_ = const_cast<void*>(data);
    shape_ = shape;
    capacity_ = 0;
    shared_ = true;
    CHECK_GT(count(), 0);
  }

  // Grow-only: memory is reallocated only when the new element count exceeds
  // the capacity (shadow/core/blob.hpp:96-111).
  void reshape(const VecInt& shape) {
    size_t wanted = 1;
    for (int d : shape) wanted *= static_cast<size_t>(d);
    CHECK_GT(wanted, 0);
    if (shared_ || data_ == nullptr || wanted > capacity_) {
      release();
      data_ = allocator_->malloc(wanted * elem_size(), nullptr);
      capacity_ = wanted;
    }
    shape_ = shape;
    shared_ = false;
  }

  const std::string& name() const { return name_; }
  const DataType& data_type() const { return data_type_; }
  size_t capacity() const { return capacity_; }
  bool shared() const { return shared_; }
  void set_name(const std::string& name) { name_ = name; }
  void set_data_type(const DataType& data_type) { data_type_ = data_type; }
  void set_capacity(size_t capacity) { capacity_ = capacity; }
  void set_shared(bool shared) { shared_ = shared; }

  const VecInt& shape() const { return shape_; }
  int shape(int index) const { return shape_[canonical_index(index)]; }
  void set_shape(int index, int value) { shape_[canonical_index(index)] = value; }
  void set_shape(const VecInt& shape) { shape_ = shape; }
  void add_shape(int value) { shape_.push_back(value); }

  int num_axes() const { return static_cast<int>(shape_.size()); }
  int num() const { return count() / shape(0); }
  int count() const { return count(0); }
  int count(int start_axis) const { return count(start_axis, num_axes()); }
  int count(int start_axis, int end_axis) const {
    CHECK_LE(start_axis, end_axis);
    CHECK_GE(start_axis, 0);
    CHECK_GE(end_axis, 0);
    CHECK_LE(start_axis, num_axes());
    CHECK_LE(end_axis, num_axes());
    int total = 1;
    for (int i = start_axis; i < end_axis; ++i) total *= shape_[i];
    return total;
  }

  size_t raw_size() const { return count() * elem_size(); }
  size_t max_size() const { return capacity_ * elem_size(); }
  size_t elem_size() const { return detail::dtype_size(data_type_); }

  int canonical_index(int index) const {
    CHECK_GE(index, -num_axes());
    CHECK_LT(index, num_axes());
    return index < 0 ? index + num_axes() : index;
  }

 private:
  template <typename T>
  void require_type() const {
    CHECK(data_type_ == detail::dtype_of<T>::value)
        << "blob " << name_ << " does not hold " << typeid(T).name();
  }
  void release() {
    if (data_ != nullptr && !shared_) allocator_->free(data_);
    data_ = nullptr;
  }

  std::string name_;
  DataType data_type_;
  Allocator* allocator_;
  void* data_ = nullptr;
  VecInt shape_;
  size_t capacity_ = 0;
  bool shared_ = false;
  std::vector<unsigned char> host_copy_;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_BLOB_HPP_
