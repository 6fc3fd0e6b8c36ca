#include "shadow/parser.hpp"

#include <cstdio>
#include <cstdlib>

namespace Shadow {

namespace Parser {

namespace {

std::string trim(const std::string& s) {
  const char* blank = " \t\r\n";
  const auto b = s.find_first_not_of(blank);
  if (b == std::string::npos) return "";
  return s.substr(b, s.find_last_not_of(blank) - b + 1);
}

// Pieces between separators; empty pieces are dropped, as the reference's
// tokenizer does (shadow/util/util.hpp tokenize).
std::vector<std::string> split(const std::string& s, const std::string& separators) {
  std::vector<std::string> out;
  size_t pos = 0;
  while (pos <= s.size()) {
    const size_t end = s.find_first_of(separators, pos);
    const std::string piece = s.substr(pos, end == std::string::npos ? std::string::npos : end - pos);
    if (!piece.empty()) out.push_back(piece);
    if (end == std::string::npos) break;
    pos = end + 1;
  }
  return out;
}

// "[...]" / "{...}" -> "..."
std::string unwrap(const std::string& s, char open, char close) {
  const std::string t = trim(s);
  CHECK(t.size() >= 2 && t.front() == open && t.back() == close)
      << "Expected " << open << "..." << close << " but found: " << t;
  return t.substr(1, t.size() - 2);
}

int to_int(const std::string& s) {
  char* end = nullptr;
  const std::string t = trim(s);
  const long v = std::strtol(t.c_str(), &end, 10);
  CHECK(!t.empty() && *end == '\0') << "Not an integer: " << s;
  return static_cast<int>(v);
}

float to_float(const std::string& s) {
  char* end = nullptr;
  const std::string t = trim(s);
  const float v = std::strtof(t.c_str(), &end);
  CHECK(!t.empty() && *end == '\0') << "Not a number: " << s;
  return v;
}

// "{name, type, [value]}; {name, type, [v # v]}; ..."
template <typename Def>
void parse_arguments(const std::string& text, Def* def) {
  for (const auto& item : split(text, ";")) {
    if (trim(item).empty()) continue;
    const auto part = split(unwrap(item, '{', '}'), ",");
    CHECK_EQ(part.size(), 3) << "Argument needs {name, type, [value]}: " << item;
    const std::string name = trim(part[0]), type = trim(part[1]);
    const std::string value = unwrap(part[2], '[', ']');
    auto* arg = def->add_arg();
    arg->set_name(name);
    if (type == "s_f") {
      arg->set_s_f(to_float(value));
    } else if (type == "s_i") {
      arg->set_s_i(to_int(value));
    } else if (type == "s_s") {
      arg->set_s_s(value);
    } else if (type == "v_f") {
      for (const auto& v : split(value, "#")) arg->add_v_f(to_float(v));
    } else if (type == "v_i") {
      for (const auto& v : split(value, "#")) arg->add_v_i(to_int(v));
    } else if (type == "v_s") {
      for (const auto& v : split(value, "#")) arg->add_v_s(trim(v));
    } else {
      LOG(FATAL) << "Unsupported argument type " << type;
    }
  }
}

}  // namespace

void ParseNet(const std::string& proto_text, shadow::NetParam* net) {
  const auto lines = split(proto_text, "\n");
  CHECK_GE(lines.size(), 3) << "A model needs a name line, an argument line and a blob line";

  net->set_name(unwrap(lines[0], '[', ']'));
  parse_arguments(unwrap(lines[1], '[', ']'), net);

  for (const auto& item : split(unwrap(lines[2], '[', ']'), ";")) {
    if (trim(item).empty()) continue;
    const auto part = split(unwrap(item, '{', '}'), ",");
    CHECK_EQ(part.size(), 3) << "Blob needs {name, type, [shape]}: " << item;
    auto* blob = net->add_blob();
    blob->set_name(trim(part[0]));
    blob->set_type(trim(part[1]));
    for (const auto& dim : split(unwrap(part[2], '[', ']'), "#")) blob->add_shape(to_int(dim));
  }

  for (size_t n = 3; n < lines.size(); ++n) {
    if (trim(lines[n]).empty()) continue;
    const auto field = split(lines[n], "|");
    CHECK_EQ(field.size(), 6) << "Operator line needs six |-separated fields: " << lines[n];
    auto* op = net->add_op();
    op->set_type(unwrap(field[0], '[', ']'));
    op->set_name(unwrap(field[1], '[', ']'));
    const auto counts = split(unwrap(field[2], '[', ']'), " ");
    CHECK_EQ(counts.size(), 3);
    if (to_int(counts[0]) > 0)
      for (const auto& b : split(unwrap(field[3], '[', ']'), ";")) op->add_bottom(trim(b));
    if (to_int(counts[1]) > 0)
      for (const auto& t : split(unwrap(field[4], '[', ']'), ";")) op->add_top(trim(t));
    if (to_int(counts[2]) > 0) parse_arguments(unwrap(field[5], '[', ']'), op);
    CHECK_EQ(op->bottom_size(), to_int(counts[0])) << op->name() << ": bottom count";
    CHECK_EQ(op->top_size(), to_int(counts[1])) << op->name() << ": top count";
    CHECK_EQ(op->arg_size(), to_int(counts[2])) << op->name() << ": argument count";
  }
}

namespace {

std::string join(const std::vector<std::string>& items, const std::string& sep) {
  std::string out;
  for (const auto& it : items) out += (out.empty() ? "" : sep) + it;
  return out;
}

std::string number(float v) {
  char buf[32];
  std::snprintf(buf, sizeof(buf), "%.9g", v);
  return buf;
}

std::string dump_argument(const shadow::Argument& arg) {
  std::string type, value;
  std::vector<std::string> items;
  if (arg.has_s_i()) {
    type = "s_i", value = std::to_string(arg.s_i());
  } else if (arg.has_s_f()) {
    type = "s_f", value = number(arg.s_f());
  } else if (arg.has_s_s()) {
    type = "s_s", value = arg.s_s();
  } else if (arg.v_i_size() > 0) {
    type = "v_i";
    for (int v : arg.v_i()) items.push_back(std::to_string(v));
  } else if (arg.v_f_size() > 0) {
    type = "v_f";
    for (float v : arg.v_f()) items.push_back(number(v));
  } else {
    type = "v_s";
    items = arg.v_s();
  }
  if (!items.empty()) value = join(items, " # ");
  return "{" + arg.name() + ", " + type + ", [" + value + "]}";
}

template <typename Def>
std::string dump_arguments(const Def& def) {
  std::vector<std::string> items;
  for (const auto& arg : def.arg()) items.push_back(dump_argument(arg));
  return "[" + join(items, "; ") + "]";
}

}  // namespace

std::string DumpNet(const shadow::NetParam& net) {
  std::string out = "[" + net.name() + "]\n" + dump_arguments(net) + "\n";
  std::vector<std::string> blobs;
  for (const auto& blob : net.blob()) {
    std::vector<std::string> dims;
    for (int d : blob.shape()) dims.push_back(std::to_string(d));
    blobs.push_back("{" + blob.name() + ", " + (blob.has_type() ? blob.type() : "float") + ", [" +
                    join(dims, " # ") + "]}");
  }
  out += "[" + join(blobs, "; ") + "]\n";
  for (const auto& op : net.op()) {
    out += "[" + op.type() + "] | [" + op.name() + "] | [" + std::to_string(op.bottom_size()) + " " +
           std::to_string(op.top_size()) + " " + std::to_string(op.arg_size()) + "] | [" +
           join(op.bottom(), "; ") + "] | [" + join(op.top(), "; ") + "] | " + dump_arguments(op) +
           "\n";
  }
  return out;
}

}  // namespace Parser

}  // namespace Shadow
