// Model-description records and typed argument lookup.
//
// shadow::Argument / OpParam / NetParam carry the accessor names of Shadow's
// protobuf messages (shadow/proto/shadow.proto:14-47) and of its protobuf-free
// stand-ins (shadow/core/params.hpp:101-208), so operator code written against
// either compiles here unchanged.  ArgumentHelper mirrors
// shadow/core/helper.hpp:10-34 / helper.cpp:9-83.
#ifndef SHADOW_AMD_HOST_PARAMS_HPP_
#define SHADOW_AMD_HOST_PARAMS_HPP_

#include <map>
#include <string>
#include <vector>

#include "log.hpp"

namespace shadow {

class Argument {
 public:
  const std::string& name() const { return name_; }
  void set_name(const std::string& v) { name_ = v, has_name_ = true; }
  bool has_name() const { return has_name_; }

  bool has_s_f() const { return has_f_; }
  float s_f() const { return s_f_; }
  void set_s_f(float v) { s_f_ = v, has_f_ = true; }

  bool has_s_i() const { return has_i_; }
  int s_i() const { return s_i_; }
  void set_s_i(int v) { s_i_ = v, has_i_ = true; }

  bool has_s_s() const { return has_s_; }
  const std::string& s_s() const { return s_s_; }
  void set_s_s(const std::string& v) { s_s_ = v, has_s_ = true; }

  const std::vector<float>& v_f() const { return v_f_; }
  const std::vector<int>& v_i() const { return v_i_; }
  const std::vector<std::string>& v_s() const { return v_s_; }
  void add_v_f(float v) { v_f_.push_back(v); }
  void add_v_i(int v) { v_i_.push_back(v); }
  void add_v_s(const std::string& v) { v_s_.push_back(v); }
  int v_f_size() const { return static_cast<int>(v_f_.size()); }
  int v_i_size() const { return static_cast<int>(v_i_.size()); }
  int v_s_size() const { return static_cast<int>(v_s_.size()); }

 private:
  std::string name_;
  float s_f_ = 0.f;
  int s_i_ = 0;
  std::string s_s_;
  bool has_f_ = false, has_i_ = false, has_s_ = false, has_name_ = false;
  std::vector<float> v_f_;
  std::vector<int> v_i_;
  std::vector<std::string> v_s_;
};

class OpParam {
 public:
  const std::string& name() const { return name_; }
  void set_name(const std::string& v) { name_ = v, has_name_ = true; }
  bool has_name() const { return has_name_; }
  const std::string& type() const { return type_; }
  void set_type(const std::string& v) { type_ = v, op_has_type_ = true; }
  bool has_type() const { return op_has_type_; }

  const std::vector<std::string>& bottom() const { return bottom_; }
  const std::string& bottom(int i) const { return bottom_[i]; }
  void add_bottom(const std::string& v) { bottom_.push_back(v); }
  int bottom_size() const { return static_cast<int>(bottom_.size()); }

  const std::vector<std::string>& top() const { return top_; }
  const std::string& top(int i) const { return top_[i]; }
  void add_top(const std::string& v) { top_.push_back(v); }
  int top_size() const { return static_cast<int>(top_.size()); }

  const std::vector<Argument>& arg() const { return arg_; }
  Argument* add_arg() {
    arg_.emplace_back();
    return &arg_.back();
  }
  int arg_size() const { return static_cast<int>(arg_.size()); }

 private:
  std::string name_, type_;
  bool has_name_ = false, op_has_type_ = false;
  std::vector<std::string> bottom_, top_;
  std::vector<Argument> arg_;
};

// A blob declared by a model: name, element type ("float" when absent), shape
// and optionally its contents (shadow/core/params.hpp:54-98).
class Blob {
 public:
  const std::string& name() const { return name_; }
  void set_name(const std::string& v) { name_ = v, has_name_ = true; }
  bool has_name() const { return has_name_; }
  bool has_type() const { return has_type_; }
  const std::string& type() const { return type_; }
  void set_type(const std::string& v) { type_ = v, has_type_ = true; }

  const std::vector<int>& shape() const { return shape_; }
  void add_shape(int v) { shape_.push_back(v); }
  int shape_size() const { return static_cast<int>(shape_.size()); }

  const std::vector<float>& data_f() const { return data_f_; }
  void add_data_f(float v) { data_f_.push_back(v); }
  int data_f_size() const { return static_cast<int>(data_f_.size()); }
  const std::vector<int>& data_i() const { return data_i_; }
  void add_data_i(int v) { data_i_.push_back(v); }
  int data_i_size() const { return static_cast<int>(data_i_.size()); }
  const std::vector<std::vector<char>>& data_b() const { return data_b_; }
  const std::vector<char>& data_b(int i) const { return data_b_[i]; }
  void add_data_b(const std::vector<char>& v) { data_b_.push_back(v); }
  int data_b_size() const { return static_cast<int>(data_b_.size()); }

 private:
  std::string name_{"None"}, type_{"None"};
  bool has_type_ = false, has_name_ = false;
  std::vector<int> shape_;
  std::vector<float> data_f_;
  std::vector<int> data_i_;
  std::vector<std::vector<char>> data_b_;
};

class NetParam {
 public:
  const std::string& name() const { return name_; }
  void set_name(const std::string& v) { name_ = v, has_name_ = true; }
  bool has_name() const { return has_name_; }
  const std::vector<Blob>& blob() const { return blob_; }
  const Blob& blob(int i) const { return blob_[i]; }
  Blob* add_blob() {
    blob_.emplace_back();
    return &blob_.back();
  }
  int blob_size() const { return static_cast<int>(blob_.size()); }
  const std::vector<OpParam>& op() const { return op_; }
  const OpParam& op(int i) const { return op_[i]; }
  OpParam* add_op() {
    op_.emplace_back();
    return &op_.back();
  }
  int op_size() const { return static_cast<int>(op_.size()); }
  const std::vector<Argument>& arg() const { return arg_; }
  Argument* add_arg() {
    arg_.emplace_back();
    return &arg_.back();
  }

 private:
  std::string name_;
  bool has_name_ = false;
  std::vector<Blob> blob_;
  std::vector<OpParam> op_;
  std::vector<Argument> arg_;
};

// A model file: several networks under one name (shadow/proto/shadow.proto:42-47).
class MetaNetParam {
 public:
  const std::string& name() const { return name_; }
  void set_name(const std::string& v) { name_ = v, has_name_ = true; }
  bool has_name() const { return has_name_; }
  const std::vector<NetParam>& network() const { return network_; }
  const NetParam& network(int i) const { return network_[i]; }
  NetParam* add_network() {
    network_.emplace_back();
    return &network_.back();
  }
  int network_size() const { return static_cast<int>(network_.size()); }
  const std::vector<Argument>& arg() const { return arg_; }
  Argument* add_arg() {
    arg_.emplace_back();
    return &arg_.back();
  }

 private:
  std::string name_;
  bool has_name_ = false;
  std::vector<NetParam> network_;
  std::vector<Argument> arg_;
};

}  // namespace shadow

namespace Shadow {

class ArgumentHelper {
 public:
  ArgumentHelper() = default;

  // From anything with name() and arg(): OpParam, NetParam.
  template <typename Def>
  explicit ArgumentHelper(const Def& def) {
    for (const auto& a : def.arg()) {
      CHECK(!HasArgument(a.name()))
          << "Duplicated argument name: " << a.name() << " found in def: " << def.name();
      arguments_[a.name()] = a;
    }
  }

  bool HasArgument(const std::string& name) const { return arguments_.count(name) > 0; }

  template <typename T>
  T GetSingleArgument(const std::string& name, const T& default_value) const;
  template <typename T>
  std::vector<T> GetRepeatedArgument(const std::string& name,
                                     const std::vector<T>& default_value = std::vector<T>()) const;

  template <typename T>
  void AddSingleArgument(const std::string& name, const T& value);
  template <typename T>
  void AddRepeatedArgument(const std::string& name, const std::vector<T>& value);

 protected:
  shadow::Argument* fresh(const std::string& name) {
    CHECK(!HasArgument(name)) << "Duplicated argument name: " << name;
    auto& a = arguments_[name];
    a.set_name(name);
    return &a;
  }
  std::map<std::string, shadow::Argument> arguments_;
};

// shadow/core/helper.hpp:36-58: append a typed argument to an OpParam / NetParam.
void add_s_f(shadow::OpParam* param, const std::string& name, float value);
void add_s_i(shadow::OpParam* param, const std::string& name, int value);
void add_s_s(shadow::OpParam* param, const std::string& name, const std::string& value);
void add_v_f(shadow::OpParam* param, const std::string& name, const std::vector<float>& value);
void add_v_i(shadow::OpParam* param, const std::string& name, const std::vector<int>& value);
void add_v_s(shadow::OpParam* param, const std::string& name, const std::vector<std::string>& value);

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_PARAMS_HPP_
