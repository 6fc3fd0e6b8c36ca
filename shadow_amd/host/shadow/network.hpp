// Network: the public entry of the reference (shadow/core/network.hpp:16-49,
// network_impl.hpp:8-68) over a Backend.  Forward() selects the device, runs the
// graph and synchronises the stream.
#ifndef SHADOW_AMD_HOST_NETWORK_HPP_
#define SHADOW_AMD_HOST_NETWORK_HPP_

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "backend.hpp"

namespace Shadow {

class Network {
 public:
  void LoadXModel(const shadow::NetParam& net_param, const ArgumentHelper& arguments);
  // Text form + packed weights (Native backend only).
  void LoadXModel(const std::string& proto_text, const void* weights_data,
                  const ArgumentHelper& arguments);

  void Forward(const std::map<std::string, void*>& data_map,
               const std::map<std::string, std::vector<int>>& shape_map = {});

  // locate "host": a host copy kept inside the blob; anything else: the device pointer.
  template <typename T>
  const T* GetBlobDataByName(const std::string& blob_name, const std::string& locate = "host") {
    auto blob = backend()->ws()->GetBlob(blob_name);
    CHECK_NOTNULL(blob) << "Unknown blob: " + blob_name;
    return locate == "host" ? blob->cpu_data<T>() : blob->data<T>();
  }
  std::vector<int> GetBlobShapeByName(const std::string& blob_name) const;

  const std::vector<std::string>& in_blob() const;
  const std::vector<std::string>& out_blob() const;

  bool has_argument(const std::string& name) const;
  template <typename T>
  T get_single_argument(const std::string& name, const T& default_value) const {
    return backend()->arg_helper().GetSingleArgument<T>(name, default_value);
  }
  template <typename T>
  std::vector<T> get_repeated_argument(const std::string& name,
                                       const std::vector<T>& default_value = {}) const {
    return backend()->arg_helper().GetRepeatedArgument<T>(name, default_value);
  }

  const std::shared_ptr<Backend>& backend() const;

 private:
  std::shared_ptr<Backend> backend_;
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_NETWORK_HPP_
