// Workspace: the blob map, the device Context and a bump-allocated temp buffer,
// with the surface of shadow/core/workspace.hpp:13-51.  Not thread-safe: one
// network per thread, as in the reference.
#ifndef SHADOW_AMD_HOST_WORKSPACE_HPP_
#define SHADOW_AMD_HOST_WORKSPACE_HPP_

#include <map>
#include <memory>
#include <string>

#include "blob.hpp"

namespace Shadow {

class Workspace {
 public:
  // backend_type "Native" (or "TensorRT", which the reference also maps to the
  // GPU) selects the HIP context.  Anything else asked the reference for its CPU
  // context, which this build does not contain: that is an error here.
  explicit Workspace(const ArgumentHelper& arguments);
  Workspace(const Workspace&) = delete;
  Workspace& operator=(const Workspace&) = delete;

  std::shared_ptr<Context>& Ctx();

  bool HasBlob(const std::string& name) const;
  DataType GetBlobDataType(const std::string& name) const;
  std::vector<int> GetBlobShape(const std::string& name) const;
  std::shared_ptr<Blob> GetBlob(const std::string& name) const;  // nullptr if absent

  // Idempotent: an existing blob of that name is returned as it is.
  std::shared_ptr<Blob> CreateBlob(const std::string& name, DataType data_type,
                                   Allocator* allocator = nullptr);
  // "int64" .. "uint8", "float", "bool"; nullptr for an unknown type string.
  std::shared_ptr<Blob> CreateBlob(const std::string& name, const std::string& data_type_str,
                                   Allocator* allocator = nullptr);

  // A blob aliasing the next `count * elem_size` bytes of the temp buffer.  It
  // is valid until the next GrowTempBuffer, which rewinds the bump pointer.
  std::shared_ptr<Blob> CreateTempBlob(const std::vector<int>& shape, DataType data_type);
  void GrowTempBuffer(size_t raw_size);

  size_t GetWorkspaceSize() const;
  size_t GetWorkspaceTempSize() const;

 private:
  const void* GetTempPtr(size_t raw_size);

  std::shared_ptr<Context> context_;
  std::map<std::string, std::shared_ptr<Blob>> blob_map_;
  size_t temp_offset_ = 0;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_WORKSPACE_HPP_
