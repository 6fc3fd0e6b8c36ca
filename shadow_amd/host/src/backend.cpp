#include "shadow/backend.hpp"

namespace Shadow {

std::shared_ptr<Backend> CreateBackend(const ArgumentHelper& arguments) {
  CHECK(arguments.HasArgument("backend_type"));
  const auto backend_type = arguments.GetSingleArgument<std::string>("backend_type", "");
  CHECK(!backend_type.empty());
  std::string known;
  for (const auto& key : BackendRegistry()->Keys()) known += (known.empty() ? "" : ", ") + key;
  CHECK(BackendRegistry()->Has(backend_type))
      << "Backend type: " << backend_type
      << " is not registered, currently registered backend types: [" << known << "]";
  return std::shared_ptr<Backend>(BackendRegistry()->Create(backend_type, arguments));
}

SHADOW_DEFINE_REGISTRY(BackendRegistry, Backend, const ArgumentHelper&);

}  // namespace Shadow
