// Kernel and operator registries, kernel selection, Operator base.
#include <sstream>

#include "shadow/kernel.hpp"
#include "shadow/operator.hpp"

namespace Shadow {

SHADOW_DEFINE_REGISTRY(KernelRegistry, Kernel);
SHADOW_DEFINE_REGISTRY(OperatorRegistry, Operator, const shadow::OpParam&, Workspace*);

namespace {

const char* device_tag(DeviceType d) {
  switch (d) {
    case DeviceType::kCPU: return "CPU";
    case DeviceType::kGPU: return "GPU";
    default: break;
  }
  LOG(FATAL) << "no kernel naming for this device type";
  return "";
}

// Preference order per device (shadow/core/kernel.cpp:8-10).
std::vector<std::string> flavours(DeviceType d) {
  if (d == DeviceType::kCPU) return {"DNNL", "NNPACK", "Default"};
  return {"CUDNN", "Default"};
}

VecString keys_containing(const std::string& hint) {
  VecString out;
  for (const auto& key : KernelRegistry()->Keys())
    if (key.find(hint) != std::string::npos) out.push_back(key);
  return out;
}

}  // namespace

VecString GetKernelKeys(DeviceType device_type) { return keys_containing(device_tag(device_type)); }

VecString GetKernelKeys(const std::string& op_type, DeviceType device_type) {
  return keys_containing(op_type + device_tag(device_type));
}

std::shared_ptr<Kernel> CreateKernel(const std::string& op_type, DeviceType device_type,
                                     const std::string& kernel_type) {
  std::string flavour = kernel_type;
  if (flavour.empty()) {
    flavour = "None";
    const auto candidates = GetKernelKeys(op_type, device_type);
    for (const auto& f : flavours(device_type)) {
      bool found = false;
      for (const auto& key : candidates) found = found || key.find(f) != std::string::npos;
      if (found) {
        flavour = f;
        break;
      }
    }
  }
  const std::string key = op_type + device_tag(device_type) + "(" + flavour + ")";
  std::shared_ptr<Kernel> kernel(KernelRegistry()->Create(key));
  LOG_IF(FATAL, kernel == nullptr) << "Kernel type: " << key << " is not registered";
  return kernel;
}

Operator::Operator(const shadow::OpParam& op_param, Workspace* ws)
    : ws_(ws), op_param_(op_param), arg_helper_(op_param) {
  for (const auto& top : op_param_.top()) {
    const auto type = get_single_argument<std::string>(top + "_type", "float");
    CHECK_NOTNULL(ws->CreateBlob(top, type))
        << name() << ": Failed to create output blob " << top << ", asked for type " << type;
  }
}

std::string Operator::debug_log(const std::vector<std::shared_ptr<Blob>>& inputs,
                                const std::vector<std::shared_ptr<Blob>>& outputs) const {
  auto describe = [](std::ostream& os, const std::vector<std::shared_ptr<Blob>>& blobs) {
    for (size_t b = 0; b < blobs.size(); ++b) {
      if (b) os << " + ";
      os << blobs[b]->name() << "(";
      for (int n = 0; n < blobs[b]->num_axes(); ++n) os << (n ? "," : "") << blobs[b]->shape(n);
      os << ")";
    }
  };
  std::ostringstream os;
  os << name() << "(" << type() << "): ";
  describe(os, inputs);
  os << " -> ";
  describe(os, outputs);
  os << " <- {";
  bool first = true;
  for (const auto& a : op_param_.arg()) {
    os << (first ? "" : ", ") << "\"" << a.name() << "\": ";
    first = false;
    if (a.has_s_i()) os << a.s_i();
    else if (a.has_s_f()) os << a.s_f();
    else if (a.has_s_s()) os << "\"" << a.s_s() << "\"";
    else {
      os << "[";
      bool f2 = true;
      for (int v : a.v_i()) os << (f2 ? "" : ",") << v, f2 = false;
      for (float v : a.v_f()) os << (f2 ? "" : ",") << v, f2 = false;
      for (const auto& v : a.v_s()) os << (f2 ? "" : ",") << "\"" << v << "\"", f2 = false;
      os << "]";
    }
  }
  os << "}";
  return os.str();
}

std::shared_ptr<Operator> CreateOperator(const shadow::OpParam& op_param, Workspace* ws) {
  std::shared_ptr<Operator> op(OperatorRegistry()->Create(op_param.type(), op_param, ws));
  CHECK_NOTNULL(op) << "Op type: " << op_param.type() << " is not registered";
  return op;
}

}  // namespace Shadow
