#include "shadow/network.hpp"

#include "shadow/native.hpp"

namespace Shadow {

const std::shared_ptr<Backend>& Network::backend() const {
  CHECK_NOTNULL(backend_) << "No model is loaded";
  return backend_;
}

void Network::LoadXModel(const shadow::NetParam& net_param, const ArgumentHelper& arguments) {
  backend_ = CreateBackend(arguments);
  backend_->LoadModel(net_param);
}

void Network::LoadXModel(const std::string& proto_text, const void* weights_data,
                         const ArgumentHelper& arguments) {
  auto created = CreateBackend(arguments);
  auto native = std::dynamic_pointer_cast<Native>(created);
  CHECK_NOTNULL(native) << "Text models are read by the Native backend only";
  native->LoadModel(proto_text, weights_data);
  backend_ = created;
}

void Network::Forward(const std::map<std::string, void*>& data_map,
                      const std::map<std::string, std::vector<int>>& shape_map) {
  backend()->ws()->Ctx()->switch_device();
  backend()->Run(data_map, shape_map);
  backend()->ws()->Ctx()->synchronize();
}

std::vector<int> Network::GetBlobShapeByName(const std::string& blob_name) const {
  return backend()->ws()->GetBlobShape(blob_name);
}

const std::vector<std::string>& Network::in_blob() const { return backend()->in_blob(); }
const std::vector<std::string>& Network::out_blob() const { return backend()->out_blob(); }

bool Network::has_argument(const std::string& name) const {
  return backend()->arg_helper().HasArgument(name);
}

}  // namespace Shadow
