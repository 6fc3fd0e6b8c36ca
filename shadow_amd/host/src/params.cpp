#include "shadow/params.hpp"

namespace Shadow {

// Single-valued lookups.  A present argument of the wrong kind is an error
// (shadow/core/helper.cpp:36-37); bool rides on s_i like in the reference.
template <>
float ArgumentHelper::GetSingleArgument<float>(const std::string& name, const float& def) const {
  auto it = arguments_.find(name);
  if (it == arguments_.end()) return def;
  CHECK(it->second.has_s_f());
  return it->second.s_f();
}
template <>
int ArgumentHelper::GetSingleArgument<int>(const std::string& name, const int& def) const {
  auto it = arguments_.find(name);
  if (it == arguments_.end()) return def;
  CHECK(it->second.has_s_i());
  return it->second.s_i();
}
template <>
bool ArgumentHelper::GetSingleArgument<bool>(const std::string& name, const bool& def) const {
  auto it = arguments_.find(name);
  if (it == arguments_.end()) return def;
  CHECK(it->second.has_s_i());
  return it->second.s_i() != 0;
}
template <>
std::string ArgumentHelper::GetSingleArgument<std::string>(const std::string& name,
                                                           const std::string& def) const {
  auto it = arguments_.find(name);
  if (it == arguments_.end()) return def;
  CHECK(it->second.has_s_s());
  return it->second.s_s();
}

template <>
std::vector<float> ArgumentHelper::GetRepeatedArgument<float>(const std::string& name,
                                                              const std::vector<float>& def) const {
  auto it = arguments_.find(name);
  return it == arguments_.end() ? def : it->second.v_f();
}
template <>
std::vector<int> ArgumentHelper::GetRepeatedArgument<int>(const std::string& name,
                                                          const std::vector<int>& def) const {
  auto it = arguments_.find(name);
  return it == arguments_.end() ? def : it->second.v_i();
}
template <>
std::vector<bool> ArgumentHelper::GetRepeatedArgument<bool>(const std::string& name,
                                                            const std::vector<bool>& def) const {
  auto it = arguments_.find(name);
  if (it == arguments_.end()) return def;
  std::vector<bool> out;
  for (int v : it->second.v_i()) out.push_back(v != 0);
  return out;
}
template <>
std::vector<std::string> ArgumentHelper::GetRepeatedArgument<std::string>(
    const std::string& name, const std::vector<std::string>& def) const {
  auto it = arguments_.find(name);
  return it == arguments_.end() ? def : it->second.v_s();
}

template <>
void ArgumentHelper::AddSingleArgument<float>(const std::string& name, const float& v) {
  fresh(name)->set_s_f(v);
}
template <>
void ArgumentHelper::AddSingleArgument<int>(const std::string& name, const int& v) {
  fresh(name)->set_s_i(v);
}
template <>
void ArgumentHelper::AddSingleArgument<bool>(const std::string& name, const bool& v) {
  fresh(name)->set_s_i(v ? 1 : 0);
}
template <>
void ArgumentHelper::AddSingleArgument<std::string>(const std::string& name, const std::string& v) {
  fresh(name)->set_s_s(v);
}
template <>
void ArgumentHelper::AddRepeatedArgument<float>(const std::string& name, const std::vector<float>& v) {
  auto* a = fresh(name);
  for (float x : v) a->add_v_f(x);
}
template <>
void ArgumentHelper::AddRepeatedArgument<int>(const std::string& name, const std::vector<int>& v) {
  auto* a = fresh(name);
  for (int x : v) a->add_v_i(x);
}
template <>
void ArgumentHelper::AddRepeatedArgument<std::string>(const std::string& name,
                                                      const std::vector<std::string>& v) {
  auto* a = fresh(name);
  for (const auto& x : v) a->add_v_s(x);
}

namespace {
shadow::Argument* named(shadow::OpParam* param, const std::string& name) {
  auto* a = param->add_arg();
  a->set_name(name);
  return a;
}
}  // namespace

void add_s_f(shadow::OpParam* p, const std::string& n, float v) { named(p, n)->set_s_f(v); }
void add_s_i(shadow::OpParam* p, const std::string& n, int v) { named(p, n)->set_s_i(v); }
void add_s_s(shadow::OpParam* p, const std::string& n, const std::string& v) { named(p, n)->set_s_s(v); }
void add_v_f(shadow::OpParam* p, const std::string& n, const std::vector<float>& v) {
  auto* a = named(p, n);
  for (float x : v) a->add_v_f(x);
}
void add_v_i(shadow::OpParam* p, const std::string& n, const std::vector<int>& v) {
  auto* a = named(p, n);
  for (int x : v) a->add_v_i(x);
}
void add_v_s(shadow::OpParam* p, const std::string& n, const std::vector<std::string>& v) {
  auto* a = named(p, n);
  for (const auto& x : v) a->add_v_s(x);
}

}  // namespace Shadow
