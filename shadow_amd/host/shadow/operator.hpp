// Operator base class and registry: shadow/core/operator.hpp:19-80.
// The constructor creates every `top` blob in the workspace (type taken from the
// argument "<top>_type", default "float"); Run() is the only compute entry.
#ifndef SHADOW_AMD_HOST_OPERATOR_HPP_
#define SHADOW_AMD_HOST_OPERATOR_HPP_

#include <memory>
#include <string>
#include <vector>

#include "blas.hpp"
#include "blob.hpp"
#include "kernel.hpp"
#include "params.hpp"
#include "registry.hpp"
#include "workspace.hpp"

namespace Shadow {

class Operator {
 public:
  Operator(const shadow::OpParam& op_param, Workspace* ws);
  virtual ~Operator() = default;

  virtual void Run(const std::vector<std::shared_ptr<Blob>>& inputs,
                   std::vector<std::shared_ptr<Blob>>& outputs) = 0;

  bool has_argument(const std::string& name) const { return arg_helper_.HasArgument(name); }

  template <typename T>
  T get_single_argument(const std::string& name, const T& default_value) const {
    return arg_helper_.GetSingleArgument<T>(name, default_value);
  }
  template <typename T>
  std::vector<T> get_repeated_argument(const std::string& name,
                                       const std::vector<T>& default_value = {}) const {
    return arg_helper_.GetRepeatedArgument<T>(name, default_value);
  }
  // A repeated argument that may have been written as a single value.
  template <typename T>
  std::vector<T> get_repeated_argument(const std::string& name, const T& default_value) const {
    auto values = arg_helper_.GetRepeatedArgument<T>(name);
    if (values.empty()) values.push_back(arg_helper_.GetSingleArgument<T>(name, default_value));
    return values;
  }

  Workspace* ws() const { return ws_; }
  const shadow::OpParam& op_param() const { return op_param_; }
  const std::string& name() const { return op_param_.name(); }
  const std::string& type() const { return op_param_.type(); }

  // "name(Type): in(2,3) + in2(3) -> out(2,3) <- {arguments}" for the `debug` trace.
  std::string debug_log(const std::vector<std::shared_ptr<Blob>>& inputs,
                        const std::vector<std::shared_ptr<Blob>>& outputs) const;

 protected:
  Workspace* ws_ = nullptr;

 private:
  shadow::OpParam op_param_;
  ArgumentHelper arg_helper_;
};

// Throws when op_param.type() is not registered.
std::shared_ptr<Operator> CreateOperator(const shadow::OpParam& op_param, Workspace* ws);

SHADOW_DECLARE_REGISTRY(OperatorRegistry, Operator, const shadow::OpParam&, Workspace*);

#define REGISTER_OPERATOR(name, ...) SHADOW_REGISTER_CLASS(OperatorRegistry, name, __VA_ARGS__)

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_OPERATOR_HPP_
