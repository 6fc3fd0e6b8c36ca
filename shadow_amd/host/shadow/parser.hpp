// Reader for the line-oriented model text the converter writes for builds
// without protobuf (shadow/python/converter/shadow/transformer.py:30-65):
//
//   [net name]
//   [{arg, s_i, [1]}; {arg, v_s, [a # b]}; ...]                     net arguments
//   [{blob, float, [64 # 3 # 7 # 7]}; ...]                           declared blobs
//   [Type] | [name] | [nb nt na] | [b0; b1] | [t0] | [{arg, ...}]    one line per op
//
// The reference reads this with one hand-written function per operator type
// that copies the arguments it knows and fills in defaults
// (shadow/core/parser.cpp:1045-1913).  Operators here look arguments up with
// their own defaults, so one generic reader carries every argument over.
#ifndef SHADOW_AMD_HOST_PARSER_HPP_
#define SHADOW_AMD_HOST_PARSER_HPP_

#include <string>

#include "params.hpp"

namespace Shadow {

namespace Parser {

// Throws (CHECK) on malformed text.
void ParseNet(const std::string& proto_text, shadow::NetParam* net);

// The same text form, one canonical spelling (single spaces, "%.9g" floats,
// which round-trip every fp32 value).  ParseNet(DumpNet(n)) == n.
std::string DumpNet(const shadow::NetParam& net);

}  // namespace Parser

}  // namespace Shadow

#endif  // SHADOW_AMD_HOST_PARSER_HPP_
