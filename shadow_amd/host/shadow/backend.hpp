// Backend: something that turns a NetParam into a runnable graph on a
// Workspace.  Surface of shadow/core/backend.hpp:13-49; creation by the
// "backend_type" argument as in shadow/core/backend.cpp:34-66, minus the
// dlopen of libbackend_<type>.so for types that are not linked in.
#ifndef SHADOW_AMD_HOST_BACKEND_HPP_
#define SHADOW_AMD_HOST_BACKEND_HPP_

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "params.hpp"
#include "registry.hpp"
#include "workspace.hpp"

namespace Shadow {

class Backend {
 public:
  virtual ~Backend() = default;

  virtual void LoadModel(const shadow::NetParam& net_param) = 0;
  // data_map: input blob name -> host pointer (device pointer when the backend
  // was created with device_input); shape_map optionally reshapes an input first.
  virtual void Run(const std::map<std::string, void*>& data_map,
                   const std::map<std::string, std::vector<int>>& shape_map) = 0;

  const ArgumentHelper& arg_helper() const { return arg_helper_; }
  const std::shared_ptr<Workspace>& ws() const { return ws_; }
  const std::vector<std::string>& in_blob() const { return in_blob_; }
  const std::vector<std::string>& out_blob() const { return out_blob_; }

 protected:
  ArgumentHelper arg_helper_;  // the loaded net's arguments
  std::shared_ptr<Workspace> ws_;
  std::vector<std::string> in_blob_, out_blob_;
};

// Throws when "backend_type" is missing or names a backend that is not registered.
std::shared_ptr<Backend> CreateBackend(const ArgumentHelper& arguments);

SHADOW_DECLARE_REGISTRY(BackendRegistry, Backend, const ArgumentHelper&);

#define REGISTER_BACKEND(name, ...) SHADOW_REGISTER_CLASS(BackendRegistry, name, __VA_ARGS__)

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_BACKEND_HPP_
