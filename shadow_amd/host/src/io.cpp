#include "shadow/io.hpp"

#include <cstdint>
#include <cstring>
#include <fstream>
#include <iterator>
#include <limits>

namespace Shadow {

namespace IO {

namespace {

enum WireType { kVarint = 0, kFixed64 = 1, kBytes = 2, kFixed32 = 5 };

// A bounded view of the bytes of one message.
class Reader {
 public:
  Reader(const uint8_t* begin, const uint8_t* end) : cur_(begin), end_(end) {}

  bool done() const { return cur_ == end_; }
  bool ok() const { return ok_; }
  void fail() { ok_ = false, cur_ = end_; }

  uint64_t varint() {
    uint64_t value = 0;
    for (int shift = 0; shift < 70; shift += 7) {
      if (cur_ == end_) break;
      const uint8_t byte = *cur_++;
      if (shift < 64) value |= static_cast<uint64_t>(byte & 0x7f) << shift;
      if (!(byte & 0x80)) return value;
    }
    fail();  // ran out of bytes, or more than ten of them
    return 0;
  }
  uint32_t fixed32() {
    if (end_ - cur_ < 4) {
      fail();
      return 0;
    }
    uint32_t v;
    std::memcpy(&v, cur_, 4);  // little endian on the wire and on the host
    cur_ += 4;
    return v;
  }
  float float32() {
    const uint32_t bits = fixed32();
    float v;
    std::memcpy(&v, &bits, 4);
    return v;
  }
  // int32 fields travel as sign-extended 64-bit varints
  int int32() { return static_cast<int>(static_cast<uint32_t>(varint())); }

  Reader sub() {
    const uint64_t len = varint();
    if (!ok_ || len > static_cast<uint64_t>(end_ - cur_)) {
      fail();
      return Reader(end_, end_);
    }
    Reader r(cur_, cur_ + len);
    cur_ += len;
    return r;
  }
  std::string str() {
    Reader r = sub();
    return std::string(reinterpret_cast<const char*>(r.cur_), r.end_ - r.cur_);
  }
  std::vector<char> bytes() {
    Reader r = sub();
    return std::vector<char>(reinterpret_cast<const char*>(r.cur_), reinterpret_cast<const char*>(r.end_));
  }
  void skip(uint32_t wire_type) {
    switch (wire_type) {
      case kVarint: varint(); break;
      case kFixed64:
        if (end_ - cur_ < 8) fail(); else cur_ += 8;
        break;
      case kBytes: sub(); break;
      case kFixed32: fixed32(); break;
      default: fail();  // groups and reserved types do not occur in these messages
    }
  }
  // Next field; false at the end of the message or after an error.
  bool next(uint32_t* field, uint32_t* wire_type) {
    if (!ok_ || done()) return false;
    const uint64_t tag = varint();
    *field = static_cast<uint32_t>(tag >> 3), *wire_type = static_cast<uint32_t>(tag & 7);
    if (*field == 0) fail();
    return ok_;
  }

 private:
  const uint8_t *cur_, *end_;
  bool ok_ = true;
};

// A repeated scalar: one element per tag, or one length-delimited run of them.
template <typename Add>
void repeated_float(Reader& r, uint32_t wire_type, Add add) {
  if (wire_type == kBytes) {
    Reader run = r.sub();
    while (run.ok() && !run.done()) add(run.float32());
    if (!run.ok()) r.fail();
  } else if (wire_type == kFixed32) {
    add(r.float32());
  } else {
    r.fail();
  }
}
template <typename Add>
void repeated_int32(Reader& r, uint32_t wire_type, Add add) {
  if (wire_type == kBytes) {
    Reader run = r.sub();
    while (run.ok() && !run.done()) add(run.int32());
    if (!run.ok()) r.fail();
  } else if (wire_type == kVarint) {
    add(r.int32());
  } else {
    r.fail();
  }
}
bool expect(Reader& r, uint32_t wire_type, uint32_t wanted) {
  if (wire_type != wanted) r.fail();
  return r.ok();
}

void read(Reader r, shadow::Blob* blob, bool* ok) {
  uint32_t field, wt;
  while (r.next(&field, &wt)) {
    switch (field) {
      case 1: if (expect(r, wt, kBytes)) blob->set_name(r.str()); break;
      case 2: if (expect(r, wt, kBytes)) blob->set_type(r.str()); break;
      case 3: repeated_int32(r, wt, [&](int v) { blob->add_shape(v); }); break;
      case 4: repeated_float(r, wt, [&](float v) { blob->add_data_f(v); }); break;
      case 5: repeated_int32(r, wt, [&](int v) { blob->add_data_i(v); }); break;
      case 6: if (expect(r, wt, kBytes)) blob->add_data_b(r.bytes()); break;
      default: r.skip(wt);
    }
  }
  *ok = *ok && r.ok();
}

void read(Reader r, shadow::Argument* arg, bool* ok) {
  uint32_t field, wt;
  while (r.next(&field, &wt)) {
    switch (field) {
      case 1: if (expect(r, wt, kBytes)) arg->set_name(r.str()); break;
      case 2: if (expect(r, wt, kFixed32)) arg->set_s_f(r.float32()); break;
      case 3: if (expect(r, wt, kVarint)) arg->set_s_i(r.int32()); break;
      case 4: if (expect(r, wt, kBytes)) arg->set_s_s(r.str()); break;
      case 5: repeated_float(r, wt, [&](float v) { arg->add_v_f(v); }); break;
      case 6: repeated_int32(r, wt, [&](int v) { arg->add_v_i(v); }); break;
      case 7: if (expect(r, wt, kBytes)) arg->add_v_s(r.str()); break;
      default: r.skip(wt);
    }
  }
  *ok = *ok && r.ok();
}

void read(Reader r, shadow::OpParam* op, bool* ok) {
  uint32_t field, wt;
  while (r.next(&field, &wt)) {
    switch (field) {
      case 1: if (expect(r, wt, kBytes)) op->set_name(r.str()); break;
      case 2: if (expect(r, wt, kBytes)) op->set_type(r.str()); break;
      case 3: if (expect(r, wt, kBytes)) op->add_bottom(r.str()); break;
      case 4: if (expect(r, wt, kBytes)) op->add_top(r.str()); break;
      case 11: if (expect(r, wt, kBytes)) read(r.sub(), op->add_arg(), ok); break;
      default: r.skip(wt);
    }
  }
  *ok = *ok && r.ok();
}

void read(Reader r, shadow::NetParam* net, bool* ok) {
  uint32_t field, wt;
  while (r.next(&field, &wt)) {
    switch (field) {
      case 1: if (expect(r, wt, kBytes)) net->set_name(r.str()); break;
      case 5: if (expect(r, wt, kBytes)) read(r.sub(), net->add_blob(), ok); break;
      case 11: if (expect(r, wt, kBytes)) read(r.sub(), net->add_op(), ok); break;
      case 12: if (expect(r, wt, kBytes)) read(r.sub(), net->add_arg(), ok); break;
      default: r.skip(wt);
    }
  }
  *ok = *ok && r.ok();
}

void read(Reader r, shadow::MetaNetParam* meta, bool* ok) {
  uint32_t field, wt;
  while (r.next(&field, &wt)) {
    switch (field) {
      case 1: if (expect(r, wt, kBytes)) meta->set_name(r.str()); break;
      case 11: if (expect(r, wt, kBytes)) read(r.sub(), meta->add_network(), ok); break;
      case 12: if (expect(r, wt, kBytes)) read(r.sub(), meta->add_arg(), ok); break;
      default: r.skip(wt);
    }
  }
  *ok = *ok && r.ok();
}

template <typename Proto>
bool read_array(const void* data, int size, Proto* proto) {
  if (size < 0 || (size > 0 && data == nullptr)) return false;
  const auto* begin = static_cast<const uint8_t*>(data);
  bool ok = true;
  read(Reader(begin, begin + size), proto, &ok);
  return ok;
}

template <typename Proto>
bool read_file(const std::string& proto_file, Proto* proto) {
  std::ifstream ifs(proto_file, std::ios::binary);
  CHECK(ifs.is_open()) << "File not found: " << proto_file;
  const std::string bytes((std::istreambuf_iterator<char>(ifs)), std::istreambuf_iterator<char>());
  CHECK_LE(bytes.size(), static_cast<size_t>(std::numeric_limits<int>::max()));
  return read_array(bytes.data(), static_cast<int>(bytes.size()), proto);
}

// ------------------------------------------------------------------ writer ---
void put_varint(std::string* out, uint64_t v) {
  while (v >= 0x80) {
    out->push_back(static_cast<char>((v & 0x7f) | 0x80));
    v >>= 7;
  }
  out->push_back(static_cast<char>(v));
}
void put_tag(std::string* out, uint32_t field, uint32_t wire_type) { put_varint(out, (field << 3) | wire_type); }
void put_fixed32(std::string* out, float v) {
  char raw[4];
  std::memcpy(raw, &v, 4);
  out->append(raw, 4);
}
void put_int32(std::string* out, int v) { put_varint(out, static_cast<uint64_t>(static_cast<int64_t>(v))); }
void put_bytes(std::string* out, uint32_t field, const char* data, size_t size) {
  put_tag(out, field, kBytes);
  put_varint(out, size);
  out->append(data, size);
}
void put_string(std::string* out, uint32_t field, const std::string& v) { put_bytes(out, field, v.data(), v.size()); }

// proto2 writes an optional field only when it was set (an empty string that was
// set is written); the records keep a presence bit per optional field.
void write(const shadow::Argument& arg, std::string* out) {
  if (arg.has_name()) put_string(out, 1, arg.name());
  if (arg.has_s_f()) put_tag(out, 2, kFixed32), put_fixed32(out, arg.s_f());
  if (arg.has_s_i()) put_tag(out, 3, kVarint), put_int32(out, arg.s_i());
  if (arg.has_s_s()) put_string(out, 4, arg.s_s());
  for (float v : arg.v_f()) put_tag(out, 5, kFixed32), put_fixed32(out, v);
  for (int v : arg.v_i()) put_tag(out, 6, kVarint), put_int32(out, v);
  for (const auto& v : arg.v_s()) put_string(out, 7, v);
}

void write(const shadow::Blob& blob, std::string* out) {
  if (blob.has_name()) put_string(out, 1, blob.name());
  if (blob.has_type()) put_string(out, 2, blob.type());
  for (int v : blob.shape()) put_tag(out, 3, kVarint), put_int32(out, v);
  if (blob.data_f_size() > 0) {
    put_bytes(out, 4, reinterpret_cast<const char*>(blob.data_f().data()), blob.data_f().size() * sizeof(float));
  }
  if (blob.data_i_size() > 0) {
    std::string run;
    for (int v : blob.data_i()) put_int32(&run, v);
    put_bytes(out, 5, run.data(), run.size());
  }
  for (const auto& v : blob.data_b()) put_bytes(out, 6, v.data(), v.size());
}

void write(const shadow::OpParam& op, std::string* out);
void write(const shadow::NetParam& net, std::string* out);

template <typename Sub>
void put_message(std::string* out, uint32_t field, const Sub& sub) {
  std::string body;
  write(sub, &body);
  put_bytes(out, field, body.data(), body.size());
}

void write(const shadow::OpParam& op, std::string* out) {
  if (op.has_name()) put_string(out, 1, op.name());
  if (op.has_type()) put_string(out, 2, op.type());
  for (const auto& v : op.bottom()) put_string(out, 3, v);
  for (const auto& v : op.top()) put_string(out, 4, v);
  for (const auto& a : op.arg()) put_message(out, 11, a);
}

void write(const shadow::NetParam& net, std::string* out) {
  if (net.has_name()) put_string(out, 1, net.name());
  for (const auto& b : net.blob()) put_message(out, 5, b);
  for (const auto& o : net.op()) put_message(out, 11, o);
  for (const auto& a : net.arg()) put_message(out, 12, a);
}

void write(const shadow::MetaNetParam& meta, std::string* out) {
  if (meta.has_name()) put_string(out, 1, meta.name());
  for (const auto& n : meta.network()) put_message(out, 11, n);
  for (const auto& a : meta.arg()) put_message(out, 12, a);
}

template <typename Proto>
bool write_file(const Proto& proto, const std::string& proto_file) {
  std::string bytes;
  write(proto, &bytes);
  std::ofstream ofs(proto_file, std::ios::binary);
  CHECK(ofs.is_open()) << "File open failed: " << proto_file;
  ofs.write(bytes.data(), static_cast<std::streamsize>(bytes.size()));
  return ofs.good();
}

}  // namespace

bool ReadProtoFromArray(const void* proto_data, int proto_size, shadow::NetParam* proto) {
  return read_array(proto_data, proto_size, proto);
}
bool ReadProtoFromArray(const void* proto_data, int proto_size, shadow::MetaNetParam* proto) {
  return read_array(proto_data, proto_size, proto);
}
bool ReadProtoFromBinaryFile(const std::string& proto_file, shadow::NetParam* proto) {
  return read_file(proto_file, proto);
}
bool ReadProtoFromBinaryFile(const std::string& proto_file, shadow::MetaNetParam* proto) {
  return read_file(proto_file, proto);
}
void WriteProtoToString(const shadow::NetParam& proto, std::string* out) { write(proto, out); }
void WriteProtoToString(const shadow::MetaNetParam& proto, std::string* out) { write(proto, out); }
bool WriteProtoToBinaryFile(const shadow::NetParam& proto, const std::string& proto_file) {
  return write_file(proto, proto_file);
}
bool WriteProtoToBinaryFile(const shadow::MetaNetParam& proto, const std::string& proto_file) {
  return write_file(proto, proto_file);
}

}  // namespace IO

}  // namespace Shadow
