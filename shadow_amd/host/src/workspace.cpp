#include "shadow/workspace.hpp"

#include <limits>

namespace Shadow {

namespace {
const char kTempBlobName[] = "temp_blob";  // shadow/core/workspace.cpp:96

// Keeps every temp blob 256-byte aligned so kernels can use 128-bit accesses on
// them.  (The reference packs them back to back; nothing observes the gap.)
size_t align_up(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }
}  // namespace

Workspace::Workspace(const ArgumentHelper& arguments) {
  const auto backend_type = arguments.GetSingleArgument<std::string>("backend_type", "");
  CHECK(backend_type == "Native" || backend_type == "TensorRT")
      << "backend_type '" << backend_type
      << "' selects Shadow's CPU context, which this GPU-only build does not provide";
  context_ = GetContext<DeviceType::kGPU>(arguments);
}

std::shared_ptr<Context>& Workspace::Ctx() { return context_; }

bool Workspace::HasBlob(const std::string& name) const { return blob_map_.count(name) > 0; }

DataType Workspace::GetBlobDataType(const std::string& name) const {
  CHECK(HasBlob(name)) << "Unknown blob: " + name;
  return blob_map_.at(name)->data_type();
}

std::vector<int> Workspace::GetBlobShape(const std::string& name) const {
  CHECK(HasBlob(name)) << "Unknown blob: " + name;
  return blob_map_.at(name)->shape();
}

std::shared_ptr<Blob> Workspace::GetBlob(const std::string& name) const {
  auto it = blob_map_.find(name);
  if (it == blob_map_.end()) {
    DLOG(WARNING) << "Blob " << name << " not in the workspace.";
    return nullptr;
  }
  return it->second;
}

std::shared_ptr<Blob> Workspace::CreateBlob(const std::string& name, DataType data_type,
                                            Allocator* allocator) {
  auto& slot = blob_map_[name];
  if (!slot) {
    slot = std::make_shared<Blob>(name, data_type,
                                  allocator != nullptr ? allocator : context_->allocator());
  }
  return slot;
}

std::shared_ptr<Blob> Workspace::CreateBlob(const std::string& name,
                                            const std::string& data_type_str,
                                            Allocator* allocator) {
  static const std::map<std::string, DataType> by_name = {
      {"int64", DataType::kI64},  {"int32", DataType::kI32},  {"int16", DataType::kI16},
      {"int8", DataType::kI8},    {"uint64", DataType::kU64}, {"uint32", DataType::kU32},
      {"uint16", DataType::kU16}, {"uint8", DataType::kU8},   {"float", DataType::kF32},
      {"bool", DataType::kBool}};
  auto it = by_name.find(data_type_str);
  if (it == by_name.end()) return nullptr;
  return CreateBlob(name, it->second, allocator);
}

std::shared_ptr<Blob> Workspace::CreateTempBlob(const std::vector<int>& shape,
                                                DataType data_type) {
  size_t count = 1;
  for (int d : shape) count *= static_cast<size_t>(d);
  CHECK_GT(count, 0);
  auto blob = std::make_shared<Blob>("temp", data_type, context_->allocator());
  blob->share_data(GetTempPtr(count * blob->elem_size()), shape);
  return blob;
}

void Workspace::GrowTempBuffer(size_t raw_size) {
  auto temp = CreateBlob(kTempBlobName, DataType::kI32);
  // Room for the alignment gaps of up to 8 temp blobs on top of the request.
  const size_t num_int = (raw_size + 8 * 256) / temp->elem_size() + 1;
  CHECK_LE(num_int, static_cast<size_t>(std::numeric_limits<int>::max()));
  temp->reshape({static_cast<int>(num_int)});
  temp_offset_ = 0;
}

size_t Workspace::GetWorkspaceSize() const {
  size_t total = 0;
  for (const auto& kv : blob_map_) total += kv.second->max_size();
  return total;
}

size_t Workspace::GetWorkspaceTempSize() const {
  const auto temp = GetBlob(kTempBlobName);
  return temp ? temp->max_size() : 0;
}

const void* Workspace::GetTempPtr(size_t raw_size) {
  const auto temp = GetBlob(kTempBlobName);
  CHECK_NOTNULL(temp);
  CHECK_LE(temp_offset_ + raw_size, temp->max_size());
  const auto* ptr = temp->data<unsigned char>() + temp_offset_;
  temp_offset_ = align_up(temp_offset_ + raw_size);
  return ptr;
}

}  // namespace Shadow
