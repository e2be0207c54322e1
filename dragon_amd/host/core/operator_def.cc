#include "core/operator_def.h"

#include <cctype>
#include <cstdlib>

namespace dragon {

const Argument* OperatorDef::FindArg(const string& name) const {
  for (const auto& a : arg) {
    if (a.name == name) return &a;
  }
  return nullptr;
}

Argument* OperatorDef::AddArg(const string& name) {
  arg.emplace_back();
  arg.back().name = name;
  return &arg.back();
}

namespace {

class Lexer {
 public:
  explicit Lexer(const string& text) : text_(text), pos_(0) {}

  // Token kinds: identifier, number, quoted string, one of ":{}", end.
  bool Next(string* token, char* kind) {
    while (pos_ < text_.size() && std::isspace(static_cast<unsigned char>(text_[pos_]))) ++pos_;
    if (pos_ >= text_.size()) {
      *kind = 0;
      return false;
    }
    const char c = text_[pos_];
    if (c == ':' || c == '{' || c == '}') {
      *token = string(1, c);
      *kind = c;
      ++pos_;
      return true;
    }
    if (c == '"' || c == '\'') {
      const char quote = c;
      string out;
      ++pos_;
      while (pos_ < text_.size() && text_[pos_] != quote) {
        if (text_[pos_] == '\\' && pos_ + 1 < text_.size()) ++pos_;
        out.push_back(text_[pos_++]);
      }
      CHECK(pos_ < text_.size()) << "\nUnterminated string in operator definition.";
      ++pos_;
      *token = out;
      *kind = 's';
      return true;
    }
    size_t begin = pos_;
    while (pos_ < text_.size() && !std::isspace(static_cast<unsigned char>(text_[pos_])) &&
           text_[pos_] != ':' && text_[pos_] != '{' && text_[pos_] != '}') {
      ++pos_;
    }
    *token = text_.substr(begin, pos_ - begin);
    *kind = (std::isdigit(static_cast<unsigned char>((*token)[0])) || (*token)[0] == '-' ||
             (*token)[0] == '+' || (*token)[0] == '.')
        ? 'n'
        : 'i';
    return true;
  }

 private:
  const string& text_;
  size_t pos_;
};

struct Parser {
  Lexer lex;
  explicit Parser(const string& text) : lex(text) {}

  string Value(char* kind) {
    string tok;
    char k;
    CHECK(lex.Next(&tok, &k) && k == ':') << "\nExpected ':' in operator definition.";
    CHECK(lex.Next(&tok, kind) && (*kind == 's' || *kind == 'n' || *kind == 'i'))
        << "\nExpected a value in operator definition.";
    return tok;
  }

  void OpenBlock() {
    string tok;
    char k;
    CHECK(lex.Next(&tok, &k)) << "\nExpected '{'.";
    if (k == ':') CHECK(lex.Next(&tok, &k)) << "\nExpected '{'.";
    CHECK(k == '{') << "\nExpected '{' in operator definition.";
  }

  void ParseArgument(Argument* a) {
    OpenBlock();
    string tok;
    char k, vk;
    while (lex.Next(&tok, &k) && k != '}') {
      CHECK(k == 'i') << "\nExpected a field name, got: " << tok;
      if (tok == "name") {
        a->name = Value(&vk);
      } else if (tok == "f") {
        a->f = std::strtof(Value(&vk).c_str(), nullptr), a->has_f = true;
      } else if (tok == "i") {
        a->i = std::strtoll(Value(&vk).c_str(), nullptr, 10), a->has_i = true;
      } else if (tok == "s") {
        a->s = Value(&vk), a->has_s = true;
      } else if (tok == "floats") {
        a->floats.push_back(std::strtof(Value(&vk).c_str(), nullptr));
      } else if (tok == "ints") {
        a->ints.push_back(std::strtoll(Value(&vk).c_str(), nullptr, 10));
      } else if (tok == "strings") {
        a->strings.push_back(Value(&vk));
      } else {
        LOG(FATAL) << "Unknown Argument field: " << tok;
      }
    }
  }

  void ParseDeviceOption(DeviceOption* d) {
    OpenBlock();
    string tok;
    char k, vk;
    while (lex.Next(&tok, &k) && k != '}') {
      if (tok == "device_type") {
        const string v = Value(&vk);
        if (vk == 'n') {
          d->device_type = std::atoi(v.c_str());
        } else if (v == "PROTO_CPU") {
          d->device_type = PROTO_CPU;
        } else if (v == "PROTO_CUDA") {
          d->device_type = PROTO_CUDA;
        } else if (v == "PROTO_MPS") {
          d->device_type = PROTO_MPS;
        } else if (v == "PROTO_MLU") {
          d->device_type = PROTO_MLU;
        } else if (v == "PROTO_HIP") {
          d->device_type = PROTO_HIP;
        } else {
          LOG(FATAL) << "Unknown device type: " << v;
        }
      } else if (tok == "device_id") {
        d->device_id = std::atoi(Value(&vk).c_str());
      } else if (tok == "random_seed") {
        d->random_seed = static_cast<uint32_t>(std::strtoul(Value(&vk).c_str(), nullptr, 10));
      } else {
        LOG(FATAL) << "Unknown DeviceOption field: " << tok;
      }
    }
  }

  OperatorDef Parse() {
    OperatorDef def;
    string tok;
    char k, vk;
    while (lex.Next(&tok, &k)) {
      CHECK(k == 'i') << "\nExpected a field name, got: " << tok;
      if (tok == "name") {
        def.name = Value(&vk);
      } else if (tok == "type") {
        def.type = Value(&vk);
      } else if (tok == "input") {
        def.input.push_back(Value(&vk));
      } else if (tok == "output") {
        def.output.push_back(Value(&vk));
      } else if (tok == "arg") {
        def.arg.emplace_back();
        ParseArgument(&def.arg.back());
      } else if (tok == "device_option") {
        ParseDeviceOption(&def.device_option);
        def.has_device_option = true;
      } else {
        LOG(FATAL) << "Unknown OperatorDef field: " << tok;
      }
    }
    return def;
  }
};

string Quote(const string& s) {
  string out = "\"";
  for (char c : s) {
    if (c == '"' || c == '\\') out.push_back('\\');
    out.push_back(c);
  }
  return out + "\"";
}

} // namespace

OperatorDef ParseOperatorDef(const string& text) { return Parser(text).Parse(); }

string PrintOperatorDef(const OperatorDef& def) {
  std::stringstream ss;
  ss.precision(9);
  if (!def.name.empty()) ss << "name: " << Quote(def.name) << " ";
  ss << "type: " << Quote(def.type) << " ";
  for (const auto& s : def.input) ss << "input: " << Quote(s) << " ";
  for (const auto& s : def.output) ss << "output: " << Quote(s) << " ";
  for (const auto& a : def.arg) {
    ss << "arg { name: " << Quote(a.name) << " ";
    if (a.has_f) ss << "f: " << a.f << " ";
    if (a.has_i) ss << "i: " << a.i << " ";
    if (a.has_s) ss << "s: " << Quote(a.s) << " ";
    for (float v : a.floats) ss << "floats: " << v << " ";
    for (int64_t v : a.ints) ss << "ints: " << v << " ";
    for (const auto& v : a.strings) ss << "strings: " << Quote(v) << " ";
    ss << "} ";
  }
  if (def.has_device_option) {
    ss << "device_option { device_type: " << def.device_option.device_type
       << " device_id: " << def.device_option.device_id << " } ";
  }
  return ss.str();
}

} // namespace dragon
