#include "shadow/fusion.hpp"

#include <algorithm>
#include <set>

#include "shadow_hip.h"

namespace Shadow {

namespace {

constexpr int kActivateRelu = 1;  // shadow/operators/kernels/activate.hpp:12
constexpr int kEltwiseSum = 1;    // shadow/operators/kernels/eltwise.hpp:10
constexpr int kReduceAvg = 4;     // shadow/operators/kernels/reduce.hpp:18

using OpList = std::vector<std::shared_ptr<Operator>>;

// What the matcher sees of an operator: its parameters and arguments, nothing that
// needs a device.  The accessors carry Operator's names.
class Node {
 public:
  explicit Node(const shadow::OpParam& op_param) : op_param_(op_param), arg_helper_(op_param) {}
  const shadow::OpParam& op_param() const { return op_param_; }
  const std::string& name() const { return op_param_.name(); }
  const std::string& type() const { return op_param_.type(); }
  template <typename T>
  T get_single_argument(const std::string& name, const T& default_value) const {
    return arg_helper_.GetSingleArgument<T>(name, default_value);
  }
  template <typename T>
  std::vector<T> get_repeated_argument(const std::string& name) const {
    return arg_helper_.GetRepeatedArgument<T>(name);
  }

 private:
  shadow::OpParam op_param_;
  ArgumentHelper arg_helper_;
};
using NodeList = std::vector<Node>;

bool reads(const Node& op, const std::string& blob) {
  const auto& b = op.op_param().bottom();
  return std::find(b.begin(), b.end(), blob) != b.end();
}
bool writes(const Node& op, const std::string& blob) {
  const auto& t = op.op_param().top();
  return std::find(t.begin(), t.end(), blob) != t.end();
}

// What the reference's optimizer asks of a producer (exactly one successor,
// optimizer.py:87-94), on blob names that may be written again further down:
// between `producer` and the next operator that overwrites `blob`, `reader` is the
// only operator that reads it, and the network does not hand it out.
bool sole_reader(const NodeList& ops, const std::vector<std::string>& out_blob, const std::string& blob,
                 int producer, int reader) {
  if (std::find(out_blob.begin(), out_blob.end(), blob) != out_blob.end()) return false;
  bool seen = false;
  for (int j = producer + 1; j < static_cast<int>(ops.size()); ++j) {
    if (reads(ops[j], blob)) {
      if (j != reader) return false;
      seen = true;
    }
    if (writes(ops[j], blob)) break;
  }
  return seen;
}

// The first operator after `producer` that reads `blob` before it is overwritten.
int next_reader(const NodeList& ops, const std::string& blob, int producer) {
  for (int j = producer + 1; j < static_cast<int>(ops.size()); ++j) {
    if (reads(ops[j], blob)) return j;
    if (writes(ops[j], blob)) break;
  }
  return -1;
}

// The operator in front of `reader` that wrote `blob` last, or -1.
int last_writer(const NodeList& ops, const std::string& blob, int reader) {
  for (int j = reader - 1; j >= 0; --j)
    if (writes(ops[j], blob)) return j;
  return -1;
}

// The members run together where the last one stood.  That is the order of the
// file as long as no operator between them writes a blob the members read or
// write, or reads a blob they write.
bool movable(const NodeList& ops, const std::vector<int>& members) {
  std::set<std::string> in, out;
  for (int m : members) {
    in.insert(ops[m].op_param().bottom().begin(), ops[m].op_param().bottom().end());
    out.insert(ops[m].op_param().top().begin(), ops[m].op_param().top().end());
  }
  for (int j = members.front() + 1; j < members.back(); ++j) {
    if (std::find(members.begin(), members.end(), j) != members.end()) continue;
    for (const auto& t : ops[j].op_param().top())
      if (in.count(t) || out.count(t)) return false;
    for (const auto& b : ops[j].op_param().bottom())
      if (out.count(b)) return false;
  }
  return true;
}

bool is_relu(const Node& op) {
  return op.type() == "Activate" && op.get_single_argument<int>("type", 1) == kActivateRelu &&
         op.op_param().bottom_size() == 1 && op.op_param().top_size() == 1;
}

// Scale with its parameters as input blobs (not scale_value / bias_value, which
// are staged through the temp buffer on every run).
bool is_blob_scale(const Node& op) {
  if (op.type() != "Scale" || op.op_param().top_size() != 1) return false;
  const bool has_scale = op.get_single_argument<bool>("has_scale", false);
  const bool has_bias = op.get_single_argument<bool>("has_bias", false);
  return (has_scale || has_bias) && op.op_param().bottom_size() == (has_scale && has_bias ? 3 : 2);
}

bool is_residual_sum(const Node& op) {
  if (op.type() != "Eltwise" || op.op_param().bottom_size() != 2 || op.op_param().top_size() != 1) return false;
  if (op.get_single_argument<int>("operation", -1) != kEltwiseSum) return false;
  for (float c : op.get_repeated_argument<float>("coeff"))
    if (c != 1.f) return false;
  const auto& p = op.op_param();
  // an output that is one of the inputs is cleared before it is read
  // (shadow/operators/kernels/eltwise.hpp:37-44): nothing to gain from that form
  return p.bottom(0) != p.bottom(1) && p.top(0) != p.bottom(0) && p.top(0) != p.bottom(1);
}

bool is_mean(const Node& op) {
  return op.type() == "Reduce" && op.get_single_argument<int>("operation", 0) == kReduceAvg &&
         op.op_param().bottom_size() == 1 && op.op_param().top_size() == 1 &&
         op.op_param().top(0) != op.op_param().bottom(0);
}

std::shared_ptr<Blob> float_blob(Workspace* ws, const std::string& name) {
  auto blob = ws->GetBlob(name);
  return blob != nullptr && blob->data_type() == DataType::kF32 ? blob : nullptr;
}

// The Scale member's view of its input: the parameter blobs cover the axes from
// `axis` on, one parameter per run of `inner` elements
// (shadow/operators/kernels/scale.hpp:45-62).
struct ScaleView {
  std::shared_ptr<Blob> x, scale, bias;
  int num = 0, inner = 0;
};

// `input`: the blob the Scale member works on when that is not its own first
// input (a group whose earlier member stands in front of it).
bool view_scale(const Operator& op, Workspace* ws, ScaleView* v, const std::shared_ptr<Blob>& input = nullptr) {
  const auto& p = op.op_param();
  const bool has_scale = op.get_single_argument<bool>("has_scale", false);
  const bool has_bias = op.get_single_argument<bool>("has_bias", false);
  v->x = input != nullptr ? input : float_blob(ws, p.bottom(0));
  if (has_scale) v->scale = float_blob(ws, p.bottom(1));
  if (has_bias) v->bias = float_blob(ws, p.bottom(has_scale ? 2 : 1));
  if (v->x == nullptr || (has_scale && v->scale == nullptr) || (has_bias && v->bias == nullptr)) return false;
  if (has_scale && has_bias && v->scale->shape() != v->bias->shape()) return false;
  const auto& param = has_scale ? v->scale : v->bias;
  const int rank = v->x->num_axes();
  int axis = op.get_single_argument<int>("axis", 1);
  if (axis < 0) axis += rank;
  if (axis < 0 || axis + param->num_axes() > rank || v->x->count() == 0) return false;
  for (int k = 0; k < param->num_axes(); ++k)
    if (param->shape(k) != v->x->shape(axis + k)) return false;
  v->num = param->count();
  v->inner = v->x->count(axis + param->num_axes());
  return v->num > 0 && v->inner > 0;
}

// BatchNorm on stored statistics (shadow/operators/batch_norm_op.cpp:7-47): how a
// Caffe-style model holds a normalisation, the learned affine pair in the Scale
// behind it.
bool is_stats_batch_norm(const Node& op) {
  return op.type() == "BatchNorm" && op.op_param().top_size() == 1 &&
         (op.op_param().bottom_size() == 3 || op.op_param().bottom_size() == 4);
}

// The BatchNorm member's view of its input: one mean and one variance per channel
// (axis 1), the factor the optional fourth input carries, eps.
struct NormView {
  std::shared_ptr<Blob> x, mean, variance;
  int channel = 0;
  float scale_factor = 1, eps = 1e-5f;
};

bool view_batch_norm(const Operator& op, Workspace* ws, NormView* v) {
  const auto& p = op.op_param();
  v->x = float_blob(ws, p.bottom(0));
  v->mean = float_blob(ws, p.bottom(1));
  v->variance = float_blob(ws, p.bottom(2));
  if (v->x == nullptr || v->mean == nullptr || v->variance == nullptr) return false;
  if (v->x->num_axes() < 2 || v->x->count() == 0) return false;
  v->channel = v->x->shape(1);
  if (v->mean->count() != v->channel || v->variance->count() != v->channel) return false;
  if (p.bottom_size() == 4) {
    auto factor = float_blob(ws, p.bottom(3));
    if (factor == nullptr || factor->count() != 1) return false;
    float value = 1;
    factor->get_data<float>(&value, 1);  // synchronous device -> host read, as the operator does
    v->scale_factor = value == 0 ? 0 : 1 / value;
  }
  v->eps = op.get_single_argument<float>("eps", 1e-5);
  return true;
}

// The Scale behind a BatchNorm must work on the same channels: axis 1, one
// parameter per channel.
bool view_scale_per_channel(const Operator& scale, Workspace* ws, const NormView& n, ScaleView* v) {
  if (!view_scale(scale, ws, v, n.x)) return false;
  int axis = scale.get_single_argument<int>("axis", 1);
  if (axis < 0) axis += n.x->num_axes();
  return axis == 1 && v->num == n.channel && v->inner == n.x->count(2);
}

std::string label(const Node& op) { return op.name() + "(" + op.type() + ")"; }

// ---- Scale -> Activate(relu): shdw_hip_scale_bias with its relu epilogue ----
class ScaleRelu : public FusedGroup {
 public:
  ScaleRelu(const OpList& ops, int scale, int relu) : scale_(ops[scale]), relu_(ops[relu]) {
    members_ = {scale, relu};
  }

  bool Run(Workspace* ws) override {
    ScaleView v;
    if (!view_scale(*scale_, ws, &v)) return false;
    auto y = float_blob(ws, relu_->op_param().top(0));
    if (y == nullptr) return false;
    y->reshape(v.x->shape());
    SHADOW_HIP_CHECK(shdw_hip_scale_bias(v.x->count(), v.num, v.inner, v.x->data<float>(),
                                         v.scale ? v.scale->data<float>() : nullptr,
                                         v.bias ? v.bias->data<float>() : nullptr, 1,
                                         y->mutable_data<float>(), ws->Ctx()->stream()));
    return true;
  }


 private:
  std::shared_ptr<Operator> scale_, relu_;
};

// ---- [BatchNorm ->] Scale -> Eltwise(SUM) -> Activate(relu) [-> Reduce(AVG)]:
//      shdw_hip_scale_residual_relu, shdw_hip_batch_norm_scale_residual_relu ----
class ResidualTail : public FusedGroup {
 public:
  ResidualTail(const OpList& ops, int bn, int scale, int sum, int relu, int mean)
      : scale_(ops[scale]), sum_(ops[sum]), relu_(ops[relu]) {
    if (bn >= 0) {
      bn_ = ops[bn];
      members_.push_back(bn);
    }
    members_.insert(members_.end(), {scale, sum, relu});
    if (mean >= 0) {
      mean_ = ops[mean];
      members_.push_back(mean);
    }
    residual_first_ = sum_->op_param().bottom(1) == scale_->op_param().top(0);
  }

  bool Run(Workspace* ws) override {
    ScaleView v;
    NormView n;
    if (bn_ != nullptr) {
      if (!view_batch_norm(*bn_, ws, &n) || !view_scale_per_channel(*scale_, ws, n, &v)) return false;
    } else if (!view_scale(*scale_, ws, &v)) {
      return false;
    }
    auto r = float_blob(ws, sum_->op_param().bottom(residual_first_ ? 0 : 1));
    auto y = float_blob(ws, relu_->op_param().top(0));
    if (r == nullptr || y == nullptr || r->shape() != v.x->shape()) return false;
    if (y == v.scale || y == v.bias || y == n.mean || y == n.variance) return false;
    std::shared_ptr<Blob> mean;
    VecInt mean_shape, squeezed;
    if (mean_ != nullptr) {
      mean = float_blob(ws, mean_->op_param().top(0));
      if (mean == nullptr || mean == y || mean == v.x || mean == r) return false;
      if (mean == v.scale || mean == v.bias || mean == n.mean || mean == n.variance) return false;
      // the reduced axes must be exactly the run one parameter applies to
      const int rank = v.x->num_axes();
      VecInt axes = mean_->get_repeated_argument<int>("axes");
      if (axes.empty())
        for (int n = 0; n < rank; ++n) axes.push_back(n);
      std::vector<bool> listed(rank, false);
      for (int a : axes) {
        if (a < -rank || a >= rank) return false;
        listed[a < 0 ? a + rank : a] = true;
      }
      int first = rank;
      while (first > 0 && listed[first - 1]) --first;
      for (int n = 0; n < first; ++n)
        if (listed[n]) return false;
      if (first == rank || v.x->count(first) != v.inner) return false;
      mean_shape = v.x->shape();
      for (int n = first; n < rank; ++n) mean_shape[n] = 1;
      squeezed.assign(mean_shape.begin(), mean_shape.begin() + first);
    }
    y->reshape(v.x->shape());
    if (mean != nullptr) mean->reshape(mean_shape);
    const float* scale = v.scale ? v.scale->data<float>() : nullptr;
    const float* bias = v.bias ? v.bias->data<float>() : nullptr;
    float* mean_data = mean != nullptr ? mean->mutable_data<float>() : nullptr;
    if (bn_ != nullptr) {
      SHADOW_HIP_CHECK(shdw_hip_batch_norm_scale_residual_relu(
          v.x->count(), n.channel, v.inner, v.x->data<float>(), n.mean->data<float>(), n.variance->data<float>(),
          n.scale_factor, n.eps, scale, bias, r->data<float>(), residual_first_ ? 1 : 0, y->mutable_data<float>(),
          mean_data, ws->Ctx()->stream()));
    } else {
      SHADOW_HIP_CHECK(shdw_hip_scale_residual_relu(v.x->count(), v.num, v.inner, v.x->data<float>(), scale, bias,
                                                    r->data<float>(), residual_first_ ? 1 : 0,
                                                    y->mutable_data<float>(), mean_data, ws->Ctx()->stream()));
    }
    if (mean != nullptr && !mean_->get_single_argument<bool>("keep_dims", true)) mean->set_shape(squeezed);
    return true;
  }


 private:
  std::shared_ptr<Operator> bn_, scale_, sum_, relu_, mean_;
  bool residual_first_ = false;
};

// ---- BatchNorm -> Scale [-> Activate(relu)]: shdw_hip_batch_norm_scale ----
class BatchNormScale : public FusedGroup {
 public:
  BatchNormScale(const OpList& ops, int bn, int scale, int relu) : bn_(ops[bn]), scale_(ops[scale]) {
    members_ = {bn, scale};
    if (relu >= 0) {
      relu_ = ops[relu];
      members_.push_back(relu);
    }
  }

  bool Run(Workspace* ws) override {
    NormView n;
    ScaleView v;
    if (!view_batch_norm(*bn_, ws, &n) || !view_scale_per_channel(*scale_, ws, n, &v)) return false;
    const auto& last = relu_ != nullptr ? relu_ : scale_;
    auto y = float_blob(ws, last->op_param().top(0));
    if (y == nullptr || y == n.mean || y == n.variance || y == v.scale || y == v.bias) return false;
    y->reshape(n.x->shape());
    SHADOW_HIP_CHECK(shdw_hip_batch_norm_scale(
        n.x->count(), n.channel, v.inner, n.x->data<float>(), n.mean->data<float>(), n.variance->data<float>(),
        n.scale_factor, n.eps, v.scale ? v.scale->data<float>() : nullptr,
        v.bias ? v.bias->data<float>() : nullptr, relu_ != nullptr ? 1 : 0, y->mutable_data<float>(),
        ws->Ctx()->stream()));
    return true;
  }


 private:
  std::shared_ptr<Operator> bn_, scale_, relu_;
};

// ---- Eltwise -> Activate(relu): shdw_hip_eltwise_relu ----
// What closes a residual block once the converter has folded the normalisation into
// the convolution (optimizer.py:181-252): the add and the ReLU.
bool is_plain_eltwise(const Node& op) {
  if (op.type() != "Eltwise" || op.op_param().bottom_size() < 2 || op.op_param().top_size() != 1) return false;
  const int operation = op.get_single_argument<int>("operation", -1);
  if (operation < 0 || operation > 3) return false;
  const auto& p = op.op_param();
  for (const auto& b : p.bottom())
    if (b == p.top(0)) return false;  // an output among the inputs has its own pass-by-pass meaning
  return true;
}

class EltwiseRelu : public FusedGroup {
 public:
  EltwiseRelu(const OpList& ops, int eltwise, int relu) : eltwise_(ops[eltwise]), relu_(ops[relu]) {
    members_ = {eltwise, relu};
  }

  bool Run(Workspace* ws) override {
    const auto& p = eltwise_->op_param();
    const int operation = eltwise_->get_single_argument<int>("operation", -1);
    const VecFloat coeff_arg = eltwise_->get_repeated_argument<float>("coeff");
    if (!coeff_arg.empty() && (operation != kEltwiseSum || coeff_arg.size() != p.bottom().size())) return false;
    std::vector<const float*> ptrs;
    std::shared_ptr<Blob> first;
    for (const auto& name : p.bottom()) {
      auto blob = float_blob(ws, name);
      if (blob == nullptr || blob->count() == 0) return false;
      if (first == nullptr) first = blob;
      if (blob->shape() != first->shape()) return false;
      ptrs.push_back(blob->data<float>());
    }
    auto y = float_blob(ws, relu_->op_param().top(0));
    if (y == nullptr) return false;
    for (const auto& name : p.bottom())
      if (ws->GetBlob(name) == y) return false;
    VecFloat coeff(ptrs.size(), 1.f);
    std::copy(coeff_arg.begin(), coeff_arg.end(), coeff.begin());
    y->reshape(first->shape());
    SHADOW_HIP_CHECK(shdw_hip_eltwise_relu(operation, static_cast<int>(ptrs.size()), ptrs.data(),
                                           operation == kEltwiseSum ? coeff.data() : nullptr, first->count(),
                                           y->mutable_data<float>(), ws->Ctx()->stream()));
    return true;
  }


 private:
  std::shared_ptr<Operator> eltwise_, relu_;
};

}  // namespace

std::vector<int> FusedPlan::members() const {
  std::vector<int> all;
  for (int m : {bn, scale, eltwise, relu, mean})
    if (m >= 0) all.push_back(m);
  std::sort(all.begin(), all.end());
  return all;
}

std::vector<FusedPlan> PlanFusedGroups(const std::vector<shadow::OpParam>& op_params,
                                       const std::vector<std::string>& out_blob) {
  const NodeList ops(op_params.begin(), op_params.end());
  std::vector<FusedPlan> groups;
  std::vector<bool> taken(ops.size(), false);
  const int count = static_cast<int>(ops.size());
  // Residual tails first: a Scale whose output goes into a sum belongs there, with the BatchNorm
  // in front of it where there is one, and the tail can take the mean along.
  for (int i = 0; i < count; ++i) {
    if (taken[i] || !is_blob_scale(ops[i])) continue;
    const std::string& s = ops[i].op_param().top(0);
    const int next = next_reader(ops, s, i);
    if (next < 0 || taken[next]) continue;
    if (!is_residual_sum(ops[next]) || !sole_reader(ops, out_blob, s, i, next)) continue;
    const std::string& e = ops[next].op_param().top(0);
    const int relu = next_reader(ops, e, next);
    if (relu < 0 || taken[relu] || !is_relu(ops[relu])) continue;
    const std::string& y = ops[relu].op_param().top(0);
    // not in place: the sum itself is no longer written, so nobody else may want it;
    // in place: every reader further down sees the activated values either way
    if (y != e && !sole_reader(ops, out_blob, e, next, relu)) continue;
    if (y == e && next_reader(ops, e, next) != relu) continue;
    std::vector<int> members = {i, next, relu};
    if (!movable(ops, members)) continue;
    int mean = -1;
    for (int j = relu + 1; j < count; ++j) {
      if (!taken[j] && is_mean(ops[j]) && ops[j].op_param().bottom(0) == y) {
        std::vector<int> with_mean = {i, next, relu, j};
        if (movable(ops, with_mean)) mean = j;
        break;
      }
      if (writes(ops[j], y)) break;
    }
    // a BatchNorm whose output only this Scale reads comes along
    int bn = last_writer(ops, ops[i].op_param().bottom(0), i);
    if (bn >= 0) {
      const auto& sp = ops[i].op_param();
      const std::string& n = sp.bottom(0);
      bool ok = !taken[bn] && is_stats_batch_norm(ops[bn]) && sole_reader(ops, out_blob, n, bn, i);
      for (int k = 1; k < sp.bottom_size(); ++k) ok = ok && sp.bottom(k) != n;
      std::vector<int> with_bn = {bn, i, next, relu};
      if (mean >= 0) with_bn.push_back(mean);
      if (!ok || !movable(ops, with_bn)) bn = -1;
    }
    groups.push_back(FusedPlan{FusedPlan::kResidualTail, bn, i, next, relu, mean});
    taken[i] = taken[next] = taken[relu] = true;
    if (bn >= 0) taken[bn] = true;
    if (mean >= 0) taken[mean] = true;
  }
  // BatchNorm -> Scale [-> ReLU] next: it takes the Scale -> ReLU pair with it.
  for (int i = 0; i < count; ++i) {
    if (taken[i] || !is_stats_batch_norm(ops[i])) continue;
    const std::string& n = ops[i].op_param().top(0);
    const int scale = next_reader(ops, n, i);
    if (scale < 0 || taken[scale] || !is_blob_scale(ops[scale])) continue;
    const auto& sp = ops[scale].op_param();
    if (sp.bottom(0) != n) continue;
    bool as_parameter = false;  // the normalised blob must be the Scale's data, not one of its parameters
    for (int k = 1; k < sp.bottom_size(); ++k) as_parameter = as_parameter || sp.bottom(k) == n;
    if (as_parameter) continue;
    const std::string& s = sp.top(0);
    // in place the Scale output is the group's output; elsewhere the normalised blob is no longer written
    if (s != n && !sole_reader(ops, out_blob, n, i, scale)) continue;
    std::vector<int> members = {i, scale};
    if (!movable(ops, members)) continue;
    int relu = next_reader(ops, s, scale);
    if (relu >= 0 && (taken[relu] || !is_relu(ops[relu]))) relu = -1;
    if (relu >= 0 && ops[relu].op_param().top(0) != s && !sole_reader(ops, out_blob, s, scale, relu)) relu = -1;
    if (relu >= 0) {
      members.push_back(relu);
      if (!movable(ops, members)) relu = -1;
    }
    groups.push_back(FusedPlan{FusedPlan::kBatchNormScale, i, scale, -1, relu, -1});
    taken[i] = taken[scale] = true;
    if (relu >= 0) taken[relu] = true;
  }
  for (int i = 0; i < count; ++i) {
    if (taken[i] || !is_blob_scale(ops[i])) continue;
    const std::string& s = ops[i].op_param().top(0);
    const int next = next_reader(ops, s, i);
    if (next < 0 || taken[next] || !is_relu(ops[next])) continue;
    // in place the Scale output is the group's output and every later reader sees the
    // activated values either way; elsewhere it is no longer written
    if (ops[next].op_param().top(0) != s && !sole_reader(ops, out_blob, s, i, next)) continue;
    std::vector<int> members = {i, next};
    if (!movable(ops, members)) continue;
    groups.push_back(FusedPlan{FusedPlan::kScaleRelu, -1, i, -1, next, -1});
    taken[i] = taken[next] = true;
  }
  for (int i = 0; i < count; ++i) {
    if (taken[i] || !is_plain_eltwise(ops[i])) continue;
    const std::string& e = ops[i].op_param().top(0);
    const int relu = next_reader(ops, e, i);
    if (relu < 0 || taken[relu] || !is_relu(ops[relu])) continue;
    if (ops[relu].op_param().top(0) != e && !sole_reader(ops, out_blob, e, i, relu)) continue;
    std::vector<int> members = {i, relu};
    if (!movable(ops, members)) continue;
    groups.push_back(FusedPlan{FusedPlan::kEltwiseRelu, -1, -1, i, relu, -1});
    taken[i] = taken[relu] = true;
  }
  std::sort(groups.begin(), groups.end(), [](const FusedPlan& a, const FusedPlan& b) {
    return a.members().back() < b.members().back();
  });
  return groups;
}

std::string DescribeFusedPlan(const FusedPlan& plan, const std::vector<shadow::OpParam>& op_params) {
  const auto name = [&](int position) { return label(Node(op_params[position])); };
  const auto top = [&](int position) { return op_params[position].top(0); };
  switch (plan.kind) {
    case FusedPlan::kScaleRelu:
      return name(plan.scale) + " + " + name(plan.relu) + " -> " + top(plan.relu);
    case FusedPlan::kEltwiseRelu:
      return name(plan.eltwise) + " + " + name(plan.relu) + " -> " + top(plan.relu);
    case FusedPlan::kBatchNormScale: {
      std::string text = name(plan.bn) + " + " + name(plan.scale);
      if (plan.relu >= 0) text += " + " + name(plan.relu);
      return text + " -> " + top(plan.relu >= 0 ? plan.relu : plan.scale);
    }
    case FusedPlan::kResidualTail: {
      std::string text = name(plan.scale) + " + " + name(plan.eltwise) + " + " + name(plan.relu);
      if (plan.bn >= 0) text = name(plan.bn) + " + " + text;
      if (plan.mean >= 0) text += " + " + name(plan.mean);
      text += " -> " + top(plan.relu);
      if (plan.mean >= 0) text += ", " + top(plan.mean);
      return text;
    }
  }
  return "";
}

std::vector<std::unique_ptr<FusedGroup>> FindFusedGroups(const OpList& ops,
                                                         const std::vector<std::string>& out_blob) {
  std::vector<shadow::OpParam> op_params;
  for (const auto& op : ops) op_params.push_back(op->op_param());
  std::vector<std::unique_ptr<FusedGroup>> groups;
  for (const FusedPlan& plan : PlanFusedGroups(op_params, out_blob)) {
    std::unique_ptr<FusedGroup> group;
    switch (plan.kind) {
      case FusedPlan::kScaleRelu:
        group.reset(new ScaleRelu(ops, plan.scale, plan.relu));
        break;
      case FusedPlan::kEltwiseRelu:
        group.reset(new EltwiseRelu(ops, plan.eltwise, plan.relu));
        break;
      case FusedPlan::kBatchNormScale:
        group.reset(new BatchNormScale(ops, plan.bn, plan.scale, plan.relu));
        break;
      case FusedPlan::kResidualTail:
        group.reset(new ResidualTail(ops, plan.bn, plan.scale, plan.eltwise, plan.relu, plan.mean));
        break;
    }
    group->set_description(DescribeFusedPlan(plan, op_params));
    groups.push_back(std::move(group));
  }
  return groups;
}

}  // namespace Shadow
