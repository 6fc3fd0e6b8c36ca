// Binary model files without the protobuf library.
//
// A converted model is a serialized shadow.MetaNetParam (or a bare NetParam):
// shadow/proto/shadow.proto:5-47, read in the reference through libprotobuf by
// IO::ReadProtoFromBinaryFile / ReadProtoFromArray (shadow/util/io.cpp:42-59).
// The five messages use only varint, 32-bit and length-delimited fields, so the
// wire format is decoded here directly: unknown fields are skipped by wire
// type, repeated scalars are accepted packed or unpacked, and a message that
// ends inside a field is an error.  The writers emit what libprotobuf would
// (fields in number order, data_f / data_i packed) so a file written here loads
// in the reference.
#ifndef SHADOW_AMD_HOST_IO_HPP_
#define SHADOW_AMD_HOST_IO_HPP_

#include <string>

#include "params.hpp"

namespace Shadow {

namespace IO {

// false on malformed input (the destination is then partly filled).
bool ReadProtoFromArray(const void* proto_data, int proto_size, shadow::NetParam* proto);
bool ReadProtoFromArray(const void* proto_data, int proto_size, shadow::MetaNetParam* proto);

// CHECK-fails when the file cannot be opened, like the reference.
bool ReadProtoFromBinaryFile(const std::string& proto_file, shadow::NetParam* proto);
bool ReadProtoFromBinaryFile(const std::string& proto_file, shadow::MetaNetParam* proto);

void WriteProtoToString(const shadow::NetParam& proto, std::string* out);
void WriteProtoToString(const shadow::MetaNetParam& proto, std::string* out);
bool WriteProtoToBinaryFile(const shadow::NetParam& proto, const std::string& proto_file);
bool WriteProtoToBinaryFile(const shadow::MetaNetParam& proto, const std::string& proto_file);

}  // namespace IO

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_IO_HPP_
