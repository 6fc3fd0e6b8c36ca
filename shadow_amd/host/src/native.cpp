#include "shadow/native.hpp"

#include "shadow/io.hpp"
#include "shadow/parser.hpp"

namespace Shadow {

Native::Native(const ArgumentHelper& arguments) {
  device_input_ = arguments.GetSingleArgument<bool>("device_input", false);
  debug_ = arguments.GetSingleArgument<bool>("debug", false);
  fuse_ = arguments.GetSingleArgument<bool>("fuse", true);
  ws_ = std::make_shared<Workspace>(arguments);
}

void Native::LoadModel(const shadow::NetParam& net_param) { Initial(net_param); }

void Native::LoadModel(const std::string& proto_text, const std::vector<const void*>& weights) {
  shadow::NetParam net_param;
  CHECK(!proto_text.empty()) << "Error when loading proto: empty text";
  Parser::ParseNet(proto_text, &net_param);
  Initial(net_param);
  CopyWeights(net_param, weights);
}

void Native::LoadModel(const std::string& proto_text, const void* weights_data) {
  shadow::NetParam net_param;
  CHECK(!proto_text.empty()) << "Error when loading proto: empty text";
  Parser::ParseNet(proto_text, &net_param);
  Initial(net_param);
  CopyWeights(net_param, weights_data);
}

void Native::LoadModel(const void* proto_data, int proto_size) {
  shadow::NetParam net_param;
  CHECK(IO::ReadProtoFromArray(proto_data, proto_size, &net_param)) << "Error when loading proto array data";
  Initial(net_param);
}

void Native::LoadModel(const std::string& proto_bin) {
  shadow::NetParam net_param;
  CHECK(IO::ReadProtoFromBinaryFile(proto_bin, &net_param)) << "Error when loading proto binary file: " << proto_bin;
  Initial(net_param);
}

// Declared blobs first (with their contents when the NetParam carries them),
// then one operator per OpParam; the constructor of an operator creates its top
// blobs.  The single Input operator names the network inputs and gives their
// shapes as arguments called like the blobs (shadow/backends/native/native.cpp:139-190).
void Native::Initial(const shadow::NetParam& net_param) {
  for (const auto& blob : net_param.blob()) {
    const std::vector<int> blob_shape(blob.shape().begin(), blob.shape().end());
    const auto blob_type = blob.has_type() ? blob.type() : std::string("float");
    auto blob_ptr = ws_->CreateBlob(blob.name(), blob_type);
    CHECK_NOTNULL(blob_ptr) << "Failed to create blob " << blob.name() << ", asked for type "
                            << blob_type;
    blob_ptr->reshape(blob_shape);
    if (blob_ptr->data_type() == DataType::kF32) {
      if (blob.data_f_size() > 0) {
        CHECK_EQ(blob.data_f_size(), blob_ptr->count());
        SetWeightData(blob.name(), blob_shape, blob.data_f().data(), false);
      }
    } else if (blob.data_b_size() > 0 && !blob.data_b(0).empty()) {
      CHECK_EQ(blob.data_b(0).size(), blob_ptr->raw_size());
      SetWeightData(blob.name(), blob_shape, blob.data_b(0).data(), false);
    }
  }

  // The uploads above were enqueued on the context's stream from memory that
  // the caller's NetParam owns (the LoadModel overloads above destroy theirs on
  // return): wait for them here rather than rely on how the runtime treats
  // pageable sources.
  ws_->Ctx()->synchronize();

  ops_.clear(), in_blob_.clear();
  for (const auto& op_param : net_param.op()) {
    ops_.emplace_back(CreateOperator(op_param, ws_.get()));
    if (op_param.type() == "Input") {
      CHECK(in_blob_.empty());
      for (const auto& blob_name : op_param.top()) {
        ws_->GetBlob(blob_name)->reshape(ops_.back()->get_repeated_argument<int>(blob_name));
        in_blob_.push_back(blob_name);
      }
    }
  }

  arg_helper_ = ArgumentHelper(net_param);
  CHECK(arg_helper_.HasArgument("out_blob")) << "Network must have out_blob argument";
  out_blob_ = arg_helper_.GetRepeatedArgument<std::string>("out_blob");

  groups_.clear();
  group_of_.assign(ops_.size(), -1);
  if (fuse_) {
    groups_ = FindFusedGroups(ops_, out_blob_);
    for (size_t g = 0; g < groups_.size(); ++g) {
      for (int member : groups_[g]->members()) group_of_[member] = static_cast<int>(g);
      if (debug_) LOG(INFO) << "Fused: " << groups_[g]->describe();
    }
  }
  if (debug_) LOG(INFO) << "Initial Network!";
}

std::vector<std::string> Native::fused() const {
  std::vector<std::string> lines;
  for (const auto& group : groups_) lines.push_back(group->describe());
  return lines;
}

void Native::RunOperator(Operator* op) {
  std::vector<std::shared_ptr<Blob>> inputs, outputs;
  for (const auto& name : op->op_param().bottom()) {
    CHECK(ws_->HasBlob(name)) << op->name() << ": Can not find input blob " << name;
    inputs.push_back(ws_->GetBlob(name));
  }
  for (const auto& name : op->op_param().top()) {
    CHECK(ws_->HasBlob(name)) << op->name() << ":  Can not find output blob " << name;
    outputs.push_back(ws_->GetBlob(name));
  }
  op->Run(inputs, outputs);
  if (debug_) LOG(INFO) << op->debug_log(inputs, outputs);
}

void Native::Run(const std::map<std::string, void*>& data_map,
                 const std::map<std::string, std::vector<int>>& shape_map) {
  if (ops_.empty()) return;

  for (const auto& in_map : data_map) {
    const auto& blob_name = in_map.first;
    CHECK_NOTNULL(in_map.second) << blob_name << " has null data";
    const auto shape = shape_map.find(blob_name);
    SetInputData(blob_name, shape != shape_map.end() ? shape->second : std::vector<int>(),
                 in_map.second);
  }

  for (size_t i = 0; i < ops_.size(); ++i) {
    const int g = group_of_[i];
    if (g < 0) {
      RunOperator(ops_[i].get());
      continue;
    }
    // a group runs where its last member stands, as one launch; when the shapes of
    // this run do not fit it, as its members one by one
    auto& group = *groups_[g];
    if (static_cast<int>(i) != group.members().back()) continue;
    if (group.Run(ws_.get())) {
      if (debug_) LOG(INFO) << "Fused: " << group.describe();
    } else {
      for (int member : group.members()) RunOperator(ops_[member].get());
    }
  }
  if (debug_) LOG(INFO) << "Forward Network!";
}

void Native::SetInputData(const std::string& blob_name, const std::vector<int>& blob_shape,
                          const void* blob_data) {
  auto blob = ws_->GetBlob(blob_name);
  CHECK_NOTNULL(blob) << "Can not find blob " << blob_name;
  if (!blob_shape.empty()) blob->reshape(blob_shape);
  if (device_input_) {
    ws_->Ctx()->allocator()->copy(blob->raw_size(), blob_data, blob->mutable_data<void>());
  } else {
    blob->set_raw_data(blob_data);
  }
}

size_t Native::SetWeightData(const std::string& blob_name, const std::vector<int>& blob_shape,
                             const void* blob_data, bool share_data) {
  auto blob = ws_->GetBlob(blob_name);
  CHECK_NOTNULL(blob) << "Can not find blob " << blob_name;
  if (share_data) {
    blob->share_data(blob_data, blob_shape);
  } else {
    blob->reshape(blob_shape);
    blob->set_raw_data(blob_data);
  }
  return blob->raw_size();
}

void Native::CopyWeights(const shadow::NetParam& net_param,
                         const std::vector<const void*>& weights) {
  const bool share_weight = arg_helper_.GetSingleArgument<bool>("share_weight", false);
  CHECK_EQ(net_param.blob_size(), weights.size());
  for (int n = 0; n < net_param.blob_size(); ++n) {
    const auto& blob = net_param.blob(n);
    SetWeightData(blob.name(), std::vector<int>(blob.shape().begin(), blob.shape().end()),
                  weights[n], share_weight);
  }
}

void Native::CopyWeights(const shadow::NetParam& net_param, const void* weights_data) {
  const bool share_weight = arg_helper_.GetSingleArgument<bool>("share_weight", false);
  const auto* cursor = static_cast<const unsigned char*>(weights_data);
  for (const auto& blob : net_param.blob()) {
    cursor += SetWeightData(blob.name(), std::vector<int>(blob.shape().begin(), blob.shape().end()),
                            cursor, share_weight);
  }
}

REGISTER_BACKEND(Native, Native);

}  // namespace Shadow
