// Protobuf-free OperatorDef / Argument / DeviceOption with the field names of
// dragon/proto/dragon.proto:56-116, plus a reader and writer for the protobuf
// text format restricted to those messages, so that a definition can cross a C
// boundary as a string.
#pragma once

#include "core/common.h"

namespace dragon {

// dragon/proto/dragon.proto:56-65 closes the enum at MLU = 3; the HIP device
// is the next value.
enum DeviceTypeProto { PROTO_CPU = 0, PROTO_CUDA = 1, PROTO_MPS = 2, PROTO_MLU = 3, PROTO_HIP = 4 };

struct DeviceOption {
  int device_type = PROTO_CPU;
  int device_id = 0;
  uint32_t random_seed = 3;
};

// dragon/proto/dragon.proto:79-96
struct Argument {
  string name;
  bool has_f = false, has_i = false, has_s = false;
  float f = 0.f;
  int64_t i = 0;
  string s;
  vector<float> floats;
  vector<int64_t> ints;
  vector<string> strings;
};

// dragon/proto/dragon.proto:99-116
struct OperatorDef {
  string name;
  string type;
  vector<string> input;
  vector<string> output;
  vector<Argument> arg;
  DeviceOption device_option;
  bool has_device_option = false;

  const Argument* FindArg(const string& name) const;
  Argument* AddArg(const string& name);
};

// Parses `name: "x" type: "LayerNorm" input: "a" arg { name: "axis" i: -1 }
// device_option { device_type: 4 device_id: 0 }` (whitespace and newlines are
// free). LOG(FATAL)s on malformed text.
OperatorDef ParseOperatorDef(const string& text);
string PrintOperatorDef(const OperatorDef& def);

} // namespace dragon
