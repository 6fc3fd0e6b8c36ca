// Fusion pass of the Native backend: runs of elementwise operators of a loaded
// network that one launch can stand for.  The reference fuses before the model is
// written (shadow/python/converter/shadow/optimizer.py:155-394, a producer with
// exactly one successor) and inside its convolution kernel
// (shadow/operators/kernels/conv.hpp:122-131, Bias then Activate); here the
// backend does it after Native::Initial has created the operators
// (shadow/backends/native/native.cpp:139-190), so a converted model runs as it is.
//
//   Scale(blob parameters) -> Activate(relu)                          one launch
//   [BatchNorm(global statistics) ->] Scale(blob parameters) -> Eltwise(SUM of 2, unit coefficients)
//                          -> Activate(relu) [-> Reduce(AVG over the trailing axes)]
//   BatchNorm(global statistics) -> Scale(blob parameters, one per channel) [-> Activate(relu)]
//   Eltwise(any operation, any number of inputs) -> Activate(relu)
//
// A blob that a group no longer writes (the Scale output, the Eltwise output when
// the Activate is not in place) must have the next member as its only reader and
// must not be an output of the network.  Results are those of the operators run
// one by one, bit for bit (the mean: the same fp64 sum rounded once).
#ifndef SHADOW_AMD_HOST_FUSION_HPP_
#define SHADOW_AMD_HOST_FUSION_HPP_

#include <memory>
#include <string>
#include <vector>

#include "operator.hpp"

namespace Shadow {

class FusedGroup {
 public:
  virtual ~FusedGroup() = default;

  // Positions of the members in the network's operator list, ascending.  The group
  // runs where its last member stood.
  const std::vector<int>& members() const { return members_; }

  // One launch for all members.  False when the blobs' present shapes or types do
  // not allow it (nothing has been written then): the caller runs the members one
  // by one, which also reports whatever is wrong with them.
  virtual bool Run(Workspace* ws) = 0;

  // "bn(Scale) + add(Eltwise) + relu(Activate) + gap(Reduce) -> e, pool"
  const std::string& describe() const { return description_; }
  void set_description(const std::string& text) { description_ = text; }

 protected:
  std::vector<int> members_;

 private:
  std::string description_;
};

// A group as the matcher finds it: positions in the operator list, -1 for a member
// the group does not have.  Found from the operators' parameters alone, so that the
// matching can be checked without a device.
struct FusedPlan {
  enum Kind { kScaleRelu, kResidualTail, kBatchNormScale, kEltwiseRelu };
  Kind kind;
  int bn, scale, eltwise, relu, mean;
  std::vector<int> members() const;  // ascending
};

// The groups of a network given as its operators' parameters, ordered by their last
// member; no operator is in two groups.
std::vector<FusedPlan> PlanFusedGroups(const std::vector<shadow::OpParam>& op_params,
                                       const std::vector<std::string>& out_blob);
std::string DescribeFusedPlan(const FusedPlan& plan, const std::vector<shadow::OpParam>& op_params);

// PlanFusedGroups over the parameters of `ops`, each plan as the group that runs it.
std::vector<std::unique_ptr<FusedGroup>> FindFusedGroups(
    const std::vector<std::shared_ptr<Operator>>& ops, const std::vector<std::string>& out_blob);

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_FUSION_HPP_
