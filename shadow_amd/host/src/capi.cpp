// C facade over the C++ operator layer, for callers without a C++ toolchain
// (the Python tests, the smoke check).  It does what Native::Initial / Native::Run
// do around the operators (shadow/backends/native/native.cpp:171-172, 78-94):
// create operators from an OpParam, look their bottom/top blobs up by name, call
// Operator::Run.  Every function catches the std::runtime_error that a failed
// CHECK throws and reports it through shdw_host_last_error().
#include <cstring>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "shadow/fusion.hpp"
#include "shadow/io.hpp"
#include "shadow/kernel.hpp"
#include "shadow/native.hpp"
#include "shadow/network.hpp"
#include "shadow/operator.hpp"
#include "shadow/parser.hpp"
#include "shadow/workspace.hpp"

using namespace Shadow;

namespace {

thread_local std::string g_error;

template <typename F>
int guarded(F&& body) {
  try {
    body();
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return -1;
  }
}

Workspace* WS(void* p) { return static_cast<Workspace*>(p); }
shadow::OpParam* OP(void* p) { return static_cast<shadow::OpParam*>(p); }

struct OpHandle {
  std::shared_ptr<Operator> op;
};

int join(const std::vector<std::string>& keys, char* buf, size_t n) {
  std::string all;
  for (const auto& k : keys) all += (all.empty() ? "" : "\n") + k;
  if (buf != nullptr && n > 0) {
    std::strncpy(buf, all.c_str(), n - 1);
    buf[n - 1] = '\0';
  }
  return static_cast<int>(all.size());
}

}  // namespace

extern "C" {

const char* shdw_host_last_error(void) { return g_error.c_str(); }
// for the other translation units of the facade
int shdw_host_set_error(const char* text) {
  g_error = text ? text : "";
  return 0;
}

int shdw_host_kernel_keys(char* buf, size_t n) { return join(KernelRegistry()->Keys(), buf, n); }
int shdw_host_operator_keys(char* buf, size_t n) { return join(OperatorRegistry()->Keys(), buf, n); }

void* shdw_host_workspace_create(const char* backend_type, int device_id) {
  Workspace* ws = nullptr;
  guarded([&] {
    ArgumentHelper args;
    args.AddSingleArgument<std::string>("backend_type", backend_type ? backend_type : "");
    args.AddSingleArgument<int>("device_id", device_id);
    ws = new Workspace(args);
  });
  return ws;
}

void shdw_host_workspace_destroy(void* ws) { delete WS(ws); }

int shdw_host_sync(void* ws) {
  return guarded([&] { WS(ws)->Ctx()->synchronize(); });
}

int shdw_host_blob_create(void* ws, const char* name, const char* dtype) {
  return guarded([&] { CHECK_NOTNULL(WS(ws)->CreateBlob(name, std::string(dtype))); });
}

// reshape, then (data != NULL) copy count() elements in from the host
int shdw_host_blob_set(void* ws, const char* name, const int* shape, int rank, const void* data) {
  return guarded([&] {
    auto blob = WS(ws)->GetBlob(name);
    CHECK_NOTNULL(blob) << "Unknown blob: " << name;
    blob->reshape(VecInt(shape, shape + rank));
    if (data != nullptr) {
      if (blob->data_type() == DataType::kF32) blob->set_data<float>(data, blob->count());
      else if (blob->data_type() == DataType::kI32) blob->set_data<std::int32_t>(data, blob->count());
      else LOG(FATAL) << "shdw_host_blob_set: float and int32 blobs only";
      WS(ws)->Ctx()->synchronize();  // the host buffer may go away after return
    }
  });
}

// Writes up to max_rank dims; returns the rank, or -1 on error.
int shdw_host_blob_shape(void* ws, const char* name, int* shape, int max_rank) {
  int rank = -1;
  guarded([&] {
    auto blob = WS(ws)->GetBlob(name);
    CHECK_NOTNULL(blob) << "Unknown blob: " << name;
    rank = blob->num_axes();
    for (int n = 0; n < rank && n < max_rank; ++n) shape[n] = blob->shape(n);
  });
  return rank;
}

int shdw_host_blob_get(void* ws, const char* name, void* out, int count) {
  return guarded([&] {
    auto blob = WS(ws)->GetBlob(name);
    CHECK_NOTNULL(blob) << "Unknown blob: " << name;
    if (blob->data_type() == DataType::kF32) blob->get_data<float>(out, count);
    else if (blob->data_type() == DataType::kI32) blob->get_data<std::int32_t>(out, count);
    else LOG(FATAL) << "shdw_host_blob_get: float and int32 blobs only";
    WS(ws)->Ctx()->synchronize();
  });
}

void* shdw_host_opparam_create(const char* type, const char* name) {
  auto* p = new shadow::OpParam();
  p->set_type(type);
  p->set_name(name);
  return p;
}
void shdw_host_opparam_destroy(void* p) { delete OP(p); }
void shdw_host_opparam_add_bottom(void* p, const char* name) { OP(p)->add_bottom(name); }
void shdw_host_opparam_add_top(void* p, const char* name) { OP(p)->add_top(name); }
void shdw_host_opparam_arg_i(void* p, const char* name, int v) { add_s_i(OP(p), name, v); }
void shdw_host_opparam_arg_f(void* p, const char* name, float v) { add_s_f(OP(p), name, v); }
void shdw_host_opparam_arg_s(void* p, const char* name, const char* v) { add_s_s(OP(p), name, v); }
void shdw_host_opparam_arg_vi(void* p, const char* name, const int* v, int n) {
  add_v_i(OP(p), name, std::vector<int>(v, v + n));
}
void shdw_host_opparam_arg_vf(void* p, const char* name, const float* v, int n) {
  add_v_f(OP(p), name, std::vector<float>(v, v + n));
}

// Runs the operator's constructor (argument checks, output blob creation,
// kernel lookup).  NULL on error.
void* shdw_host_op_create(void* ws, void* opparam) {
  OpHandle* h = nullptr;
  guarded([&] {
    auto op = CreateOperator(*OP(opparam), WS(ws));
    h = new OpHandle{op};
  });
  return h;
}
void shdw_host_op_destroy(void* op) { delete static_cast<OpHandle*>(op); }

// One iteration of the backend's op loop for this operator; asynchronous.
int shdw_host_op_run(void* ws, void* op) {
  return guarded([&] {
    auto& oper = static_cast<OpHandle*>(op)->op;
    std::vector<std::shared_ptr<Blob>> inputs, outputs;
    for (const auto& name : oper->op_param().bottom()) {
      auto blob = WS(ws)->GetBlob(name);
      CHECK_NOTNULL(blob) << oper->name() << ": Failed to find input blob " << name;
      inputs.push_back(blob);
    }
    for (const auto& name : oper->op_param().top()) {
      auto blob = WS(ws)->GetBlob(name);
      CHECK_NOTNULL(blob) << oper->name() << ": Failed to find output blob " << name;
      outputs.push_back(blob);
    }
    oper->Run(inputs, outputs);
  });
}

int shdw_host_op_debug_log(void* ws, void* op, char* buf, size_t n) {
  int len = -1;
  guarded([&] {
    auto& oper = static_cast<OpHandle*>(op)->op;
    std::vector<std::shared_ptr<Blob>> inputs, outputs;
    for (const auto& name : oper->op_param().bottom()) inputs.push_back(WS(ws)->GetBlob(name));
    for (const auto& name : oper->op_param().top()) outputs.push_back(WS(ws)->GetBlob(name));
    len = join({oper->debug_log(inputs, outputs)}, buf, n);
  });
  return len;
}

// ---- models: the text form, and a Network over the Native backend ----

// Host-only.  Parses the text and writes its canonical spelling; returns the
// length, or -1 when the text is malformed.
int shdw_host_parse_net(const char* proto_text, char* buf, size_t n) {
  int len = -1;
  guarded([&] {
    shadow::NetParam net;
    Parser::ParseNet(proto_text, &net);
    len = join({Parser::DumpNet(net)}, buf, n);
  });
  return len;
}

// Host-only.  The groups the Native backend's fusion pass would form for this text
// model, one description per line in the order they would run; returns the length,
// or -1 when the text is malformed or names no out_blob.
int shdw_host_plan_fusion(const char* proto_text, char* buf, size_t n) {
  int len = -1;
  guarded([&] {
    shadow::NetParam net;
    Parser::ParseNet(proto_text, &net);
    const ArgumentHelper arguments(net);
    CHECK(arguments.HasArgument("out_blob")) << "Network must have out_blob argument";
    const std::vector<shadow::OpParam> ops(net.op().begin(), net.op().end());
    std::vector<std::string> lines;
    for (const FusedPlan& plan : PlanFusedGroups(ops, arguments.GetRepeatedArgument<std::string>("out_blob")))
      lines.push_back(DescribeFusedPlan(plan, ops));
    len = join(lines, buf, n);
  });
  return len;
}

namespace {

// network_index < 0: `data` is a serialized NetParam; otherwise a MetaNetParam
// whose network(network_index) is taken.
void read_binary_net(const void* data, int size, int network_index, shadow::NetParam* net) {
  if (network_index < 0) {
    CHECK(IO::ReadProtoFromArray(data, size, net)) << "Error when loading proto array data";
  } else {
    shadow::MetaNetParam meta;
    CHECK(IO::ReadProtoFromArray(data, size, &meta)) << "Error when loading proto array data";
    CHECK_LT(network_index, meta.network_size());
    *net = meta.network(network_index);
  }
}

int copy_out(const std::string& bytes, void* buf, size_t n) {
  if (buf != nullptr && n >= bytes.size()) std::memcpy(buf, bytes.data(), bytes.size());
  return static_cast<int>(bytes.size());
}

}  // namespace

// Host-only.  Decodes a binary model and writes the canonical text form of the
// chosen network (the text form carries no blob contents); returns the length,
// or -1 when the bytes are malformed.
int shdw_host_parse_net_binary(const void* data, int size, int network_index, char* buf, size_t n) {
  int len = -1;
  guarded([&] {
    shadow::NetParam net;
    read_binary_net(data, size, network_index, &net);
    len = join({Parser::DumpNet(net)}, buf, n);
  });
  return len;
}

// Host-only.  Decodes and re-encodes a binary NetParam (is_meta == 0) or
// MetaNetParam; returns the encoded length (the bytes are copied when they fit
// `n`), or -1 when the input is malformed.
int shdw_host_proto_reencode(const void* data, int size, int is_meta, void* buf, size_t n) {
  int len = -1;
  guarded([&] {
    std::string bytes;
    if (is_meta) {
      shadow::MetaNetParam meta;
      CHECK(IO::ReadProtoFromArray(data, size, &meta)) << "Error when loading proto array data";
      IO::WriteProtoToString(meta, &bytes);
    } else {
      shadow::NetParam net;
      CHECK(IO::ReadProtoFromArray(data, size, &net)) << "Error when loading proto array data";
      IO::WriteProtoToString(net, &bytes);
    }
    len = copy_out(bytes, buf, n);
  });
  return len;
}

// Host-only.  The same through files: reads `path_in`, writes `path_out`.
// 0 on success, -1 when the file is missing or malformed.
int shdw_host_proto_file_reencode(const char* path_in, const char* path_out, int is_meta) {
  return guarded([&] {
    if (is_meta) {
      shadow::MetaNetParam meta;
      CHECK(IO::ReadProtoFromBinaryFile(path_in, &meta)) << "Error when loading proto binary file: " << path_in;
      CHECK(IO::WriteProtoToBinaryFile(meta, path_out));
    } else {
      shadow::NetParam net;
      CHECK(IO::ReadProtoFromBinaryFile(path_in, &net)) << "Error when loading proto binary file: " << path_in;
      CHECK(IO::WriteProtoToBinaryFile(net, path_out));
    }
  });
}

// Host-only.  The text form encoded as a binary NetParam.
int shdw_host_serialize_net(const char* proto_text, void* buf, size_t n) {
  int len = -1;
  guarded([&] {
    shadow::NetParam net;
    Parser::ParseNet(proto_text, &net);
    std::string bytes;
    IO::WriteProtoToString(net, &bytes);
    len = copy_out(bytes, buf, n);
  });
  return len;
}

int shdw_host_backend_keys(char* buf, size_t n) { return join(BackendRegistry()->Keys(), buf, n); }

// weights: one packed host buffer in declared-blob order, or NULL when the
// model declares no blobs.  device_input: Forward takes device pointers and
// copies device to device.  NULL on error.
void* shdw_host_network_create(const char* backend_type, int device_id, int debug,
                               int device_input, int fuse, const char* proto_text, const void* weights) {
  Network* net = nullptr;
  guarded([&] {
    ArgumentHelper args;
    args.AddSingleArgument<std::string>("backend_type", backend_type ? backend_type : "");
    args.AddSingleArgument<int>("device_id", device_id);
    args.AddSingleArgument<bool>("debug", debug != 0);
    args.AddSingleArgument<bool>("device_input", device_input != 0);
    args.AddSingleArgument<bool>("fuse", fuse != 0);
    std::unique_ptr<Network> made(new Network());
    made->LoadXModel(std::string(proto_text ? proto_text : ""), weights, args);
    made->backend()->ws()->Ctx()->synchronize();  // the weight buffer may go away after return
    net = made.release();
  });
  return net;
}

// The same from a binary model whose blobs carry their contents
// (network_index as in shdw_host_parse_net_binary).
void* shdw_host_network_create_from_binary(const char* backend_type, int device_id, int debug,
                                           int device_input, int fuse, const void* data, int size,
                                           int network_index) {
  Network* net = nullptr;
  guarded([&] {
    ArgumentHelper args;
    args.AddSingleArgument<std::string>("backend_type", backend_type ? backend_type : "");
    args.AddSingleArgument<int>("device_id", device_id);
    args.AddSingleArgument<bool>("debug", debug != 0);
    args.AddSingleArgument<bool>("device_input", device_input != 0);
    args.AddSingleArgument<bool>("fuse", fuse != 0);
    shadow::NetParam net_param;
    read_binary_net(data, size, network_index, &net_param);
    std::unique_ptr<Network> made(new Network());
    made->LoadXModel(net_param, args);
    made->backend()->ws()->Ctx()->synchronize();
    net = made.release();
  });
  return net;
}

void shdw_host_network_destroy(void* net) { delete static_cast<Network*>(net); }

// which: 0 = input blob names, 1 = output blob names, 2 = the fused groups of the
// Native backend, one description each (newline separated)
int shdw_host_network_io(void* net, int which, char* buf, size_t n) {
  int len = -1;
  guarded([&] {
    auto* nw = static_cast<Network*>(net);
    if (which == 2) {
      auto native = std::dynamic_pointer_cast<Native>(nw->backend());
      len = join(native != nullptr ? native->fused() : std::vector<std::string>(), buf, n);
    } else {
      len = join(which == 0 ? nw->in_blob() : nw->out_blob(), buf, n);
    }
  });
  return len;
}

// count inputs: names[i] -> data[i] (host pointers, or device pointers for a
// network created with device_input); ranks[i] > 0 reshapes that input
// first with the next ranks[i] entries of `shapes`.
int shdw_host_network_forward(void* net, int count, const char* const* names, void* const* data,
                              const int* ranks, const int* shapes) {
  return guarded([&] {
    std::map<std::string, void*> data_map;
    std::map<std::string, std::vector<int>> shape_map;
    const int* cursor = shapes;
    for (int i = 0; i < count; ++i) {
      data_map[names[i]] = data[i];
      const int rank = ranks != nullptr ? ranks[i] : 0;
      if (rank > 0) {
        shape_map[names[i]] = std::vector<int>(cursor, cursor + rank);
        cursor += rank;
      }
    }
    static_cast<Network*>(net)->Forward(data_map, shape_map);
  });
}

// The operators of the network once more on whatever its input blobs hold, enqueued
// on the context's stream and not waited for (Backend::Run without Network::Forward's
// synchronize): for a caller that times or overlaps several runs.
int shdw_host_network_run(void* net) {
  return guarded([&] {
    auto* nw = static_cast<Network*>(net);
    nw->backend()->ws()->Ctx()->switch_device();
    nw->backend()->Run({}, {});
  });
}

// The context's stream (a hipStream_t), NULL on error.
void* shdw_host_network_stream(void* net) {
  void* stream = nullptr;
  guarded([&] { stream = static_cast<Network*>(net)->backend()->ws()->Ctx()->stream(); });
  return stream;
}

int shdw_host_network_blob_shape(void* net, const char* name, int* shape, int max_rank) {
  int rank = -1;
  guarded([&] {
    auto* nw = static_cast<Network*>(net);
    CHECK(nw->backend()->ws()->HasBlob(name)) << "Unknown blob: " << name;
    const auto dims = nw->GetBlobShapeByName(name);
    rank = static_cast<int>(dims.size());
    for (int n = 0; n < rank && n < max_rank; ++n) shape[n] = dims[n];
  });
  return rank;
}

// float blobs only
int shdw_host_network_blob_get(void* net, const char* name, float* out, int count) {
  return guarded([&] {
    auto* nw = static_cast<Network*>(net);
    auto blob = nw->backend()->ws()->GetBlob(name);
    CHECK_NOTNULL(blob) << "Unknown blob: " << name;
    CHECK_LE(count, blob->count());
    const float* host = nw->GetBlobDataByName<float>(name, "host");
    nw->backend()->ws()->Ctx()->synchronize();
    std::memcpy(out, host, sizeof(float) * static_cast<size_t>(count));
  });
}

// Host-only probes of ArgumentHelper / CreateKernel / CreateOperator error paths
// (no device needed): each returns 0 when the call succeeded, -1 when it threw.
int shdw_host_probe_create_kernel(const char* op_type, int gpu) {
  return guarded([&] { CreateKernel(op_type, gpu ? DeviceType::kGPU : DeviceType::kCPU); });
}
int shdw_host_probe_argument(const char* kind, const char* ask_as) {
  return guarded([&] {
    ArgumentHelper args;
    if (std::string(kind) == "int") args.AddSingleArgument<int>("x", 3);
    if (std::string(kind) == "float") args.AddSingleArgument<float>("x", 3.f);
    if (std::string(kind) == "string") args.AddSingleArgument<std::string>("x", "3");
    if (std::string(ask_as) == "int") args.GetSingleArgument<int>("x", 0);
    if (std::string(ask_as) == "float") args.GetSingleArgument<float>("x", 0.f);
    if (std::string(ask_as) == "string") args.GetSingleArgument<std::string>("x", "");
    if (std::string(ask_as) == "dup") args.AddSingleArgument<int>("x", 4);
  });
}

}  // extern "C"
