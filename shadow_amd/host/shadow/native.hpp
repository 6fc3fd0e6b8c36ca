// The Native backend: blobs and operators of a NetParam on one Workspace, run
// in file order.  Behaviour of shadow/backends/native/native.{hpp,cpp}; model
// sources are a NetParam or the converter's text form plus a weight buffer
// (protobuf files are not read by this build).
#ifndef SHADOW_AMD_HOST_NATIVE_HPP_
#define SHADOW_AMD_HOST_NATIVE_HPP_

#include "backend.hpp"
#include "fusion.hpp"
#include "operator.hpp"

namespace Shadow {

class Native : public Backend {
 public:
  // Arguments: backend_type, device_id, default_cuda_stream (Workspace);
  // device_input (Run takes device pointers), debug (log every operator and every
  // fused group), fuse (default true: runs of elementwise operators that one launch
  // can stand for are run that way, see fusion.hpp; a blob inside such a run that
  // nothing else reads is then not written).
  explicit Native(const ArgumentHelper& arguments);

  void LoadModel(const shadow::NetParam& net_param) override;
  // proto_text: the text form.  Weights follow the order of the declared blobs:
  // one pointer per blob, or one packed buffer (each blob's raw_size() bytes).
  void LoadModel(const std::string& proto_text, const std::vector<const void*>& weights);
  void LoadModel(const std::string& proto_text, const void* weights_data);
  // A serialized NetParam in memory, or in the file `proto_bin`
  // (shadow/backends/native/native.cpp:11-21).
  void LoadModel(const void* proto_data, int proto_size);
  void LoadModel(const std::string& proto_bin);

  void Run(const std::map<std::string, void*>& data_map,
           const std::map<std::string, std::vector<int>>& shape_map) override;

  // One line per fused group (FusedGroup::describe), in running order.
  std::vector<std::string> fused() const;

 private:
  void RunOperator(Operator* op);
  void Initial(const shadow::NetParam& net_param);
  void SetInputData(const std::string& blob_name, const std::vector<int>& blob_shape,
                    const void* blob_data);
  // Returns the blob's size in bytes.  share_data aliases the caller's (device)
  // memory instead of copying.
  size_t SetWeightData(const std::string& blob_name, const std::vector<int>& blob_shape,
                       const void* blob_data, bool share_data);
  void CopyWeights(const shadow::NetParam& net_param, const std::vector<const void*>& weights);
  void CopyWeights(const shadow::NetParam& net_param, const void* weights_data);

  bool device_input_ = false, debug_ = false, fuse_ = true;
  std::vector<std::shared_ptr<Operator>> ops_;
  std::vector<std::unique_ptr<FusedGroup>> groups_;
  std::vector<int> group_of_;  // per operator: its group, or -1
};

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_NATIVE_HPP_
