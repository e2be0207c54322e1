#include "core/operator.h"

namespace dragon {

DEFINE_REGISTRY(HIPOperatorRegistry, OperatorBase, const OperatorDef&, Workspace*);

OperatorBase::OperatorBase(const OperatorDef& def, Workspace* ws)
    : ws_(ws), def_(def), phase_("TRAIN"), data_format_("NCHW") {
  // Arguments every operator understands (dragon/core/operator.cc:6-33).
  handle_ = def.name;
  for (const auto& a : def.arg) {
    if (a.name == "name" && a.has_s) handle_ = a.s;
    if (a.name == "handle" && a.has_s) handle_ = a.s;
    if (a.name == "phase" && a.has_s) phase_ = a.s;
    if (a.name == "dtype" && a.has_s) dtype_ = a.s;
    if (a.name == "data_format" && a.has_s) data_format_ = a.s;
  }
  for (const auto& name : def.input) inputs_.push_back(ws->GetTensor(name));
  for (const auto& name : def.output) outputs_.push_back(ws->CreateTensor(name));
}

OperatorBase* OperatorBase::New(const OperatorDef& def, Workspace* ws) {
  const OpSchema* schema = OpSchemaRegistry::Schema(def.type);
  if (schema != nullptr) schema->Verify(def);
  switch (def.device_option.device_type) {
    case PROTO_HIP:
      CHECK(HIPOperatorRegistry()->Has(def.type))
          << "\nOperator(" << def.type << ") is not registered for the HIP device.";
      return HIPOperatorRegistry()->Create(def.type, def, ws);
    case PROTO_CPU:
      LOG(FATAL) << "Operator(" << def.type << "): the CPU operators are not part of this build; "
                 << "set device_option.device_type to PROTO_HIP.";
      break;
    default:
      LOG(FATAL) << "Unknown device: " << def.device_option.device_type;
  }
  return nullptr;
}

OperatorBase* OperatorBase::DeriveFrom(const OperatorDef& def) {
  CHECK_EQ(def.type, def_.type) << "\nA cached operator can only be rebound to its own type.";
  inputs_.clear();
  outputs_.clear();
  for (const auto& name : def.input) inputs_.push_back(ws_->GetTensor(name));
  for (const auto& name : def.output) outputs_.push_back(ws_->CreateTensor(name));
  def_.input = def.input;
  def_.output = def.output;
  def_.name = def.name;
  handle_ = def.name;
  for (const auto& a : def.arg) {
    if ((a.name == "name" || a.name == "handle") && a.has_s) handle_ = a.s;
  }
  return this;
}

Tensor& OperatorBase::Input(int i) {
  const int n = InputSize();
  CHECK(i >= -n && i < n) << "\nOperator(" << type() << ") has " << n << " inputs, requested " << i;
  return *inputs_[i < 0 ? i + n : i];
}

Tensor* OperatorBase::Output(int i) {
  const int n = OutputSize();
  CHECK(i >= -n && i < n) << "\nOperator(" << type() << ") has " << n << " outputs, requested " << i;
  return outputs_[i < 0 ? i + n : i];
}

Tensor* OperatorBase::Output(int i, const vector<int>& inputs) {
  Tensor* y = Output(i);
  const OpSchema* schema = OpSchemaRegistry::Schema(def_.type);
  for (int j : inputs) {
    Tensor& x = Input(j);
    if (&x == y) return y;  // the definition itself names the same tensor
    if (schema != nullptr && schema->CheckInplace(j, i) && x.name() == y->name()) return y->MapFrom(&x);
  }
  return y;
}

Tensor& OperatorBase::Input(const string& name) { return *ws_->GetTensor(handle_ + "/" + name); }

Tensor* OperatorBase::Output(const string& name) { return ws_->CreateTensor(handle_ + "/" + name); }

string OperatorBase::MessageForUnsupported(const string& value, const vector<string>& support) const {
  std::stringstream ss;
  ss << "Unsupported type of Operator(" << type() << "): " << value << "\n<" << type()
     << "Op> supports the following type(s): {";
  for (size_t i = 0; i < support.size(); ++i) ss << (i ? ", " : " ") << support[i];
  ss << " }";
  return ss.str();
}

template <>
float OperatorBase::GetArgument<float>(const string& name, const float& default_value) {
  const Argument* a = def_.FindArg(name);
  if (a == nullptr) return default_value;
  CHECK(a->has_f) << "\nArgument(" << name << ") does not hold a float.";
  return a->f;
}
template <>
double OperatorBase::GetArgument<double>(const string& name, const double& default_value) {
  const Argument* a = def_.FindArg(name);
  if (a == nullptr) return default_value;
  CHECK(a->has_f) << "\nArgument(" << name << ") does not hold a float.";
  return static_cast<double>(a->f);
}
template <>
int64_t OperatorBase::GetArgument<int64_t>(const string& name, const int64_t& default_value) {
  const Argument* a = def_.FindArg(name);
  if (a == nullptr) return default_value;
  CHECK(a->has_i) << "\nArgument(" << name << ") does not hold an integer.";
  return a->i;
}
template <>
string OperatorBase::GetArgument<string>(const string& name, const string& default_value) {
  const Argument* a = def_.FindArg(name);
  if (a == nullptr) return default_value;
  CHECK(a->has_s) << "\nArgument(" << name << ") does not hold a string.";
  return a->s;
}
template <>
vector<int64_t> OperatorBase::GetRepeatedArgument<int64_t>(const string& name) {
  const Argument* a = def_.FindArg(name);
  return a == nullptr ? vector<int64_t>() : a->ints;
}
template <>
vector<float> OperatorBase::GetRepeatedArgument<float>(const string& name) {
  const Argument* a = def_.FindArg(name);
  return a == nullptr ? vector<float>() : a->floats;
}
template <>
vector<string> OperatorBase::GetRepeatedArgument<string>(const string& name) {
  const Argument* a = def_.FindArg(name);
  return a == nullptr ? vector<string>() : a->strings;
}

// ---------------------------------------------------------------- schema

bool OpSchema::Verify(const OperatorDef& def) const {
  const int in = static_cast<int>(def.input.size()), out = static_cast<int>(def.output.size());
  const string where = "\n[" + file_ + ":" + std::to_string(line_) + "] Operator(" + def.type + ") ";
  CHECK(in >= min_input_ && in <= max_input_)
      << where << "takes between " << min_input_ << " and " << max_input_ << " inputs, got " << in << ".";
  CHECK(out >= min_output_ && out <= max_output_)
      << where << "makes between " << min_output_ << " and " << max_output_ << " outputs, got " << out << ".";
  for (int i = 0; i < in; ++i) {
    if (def.input[i] == "NULL") continue;
    for (int j = 0; j < out; ++j) {
      if (def.output[j] == "NULL") continue;
      if (def.input[i] == def.output[j]) {
        CHECK(CheckInplace(i, j)) << where << "Input(" << i << ") and Output(" << j
                                  << ") can not be set to inplace.";
      }
    }
  }
  return true;
}

bool OpSchema::CheckInplace(int input, int output) const {
  for (const auto& p : inplace_) {
    if (p.first == input && p.second == output) return true;
  }
  return false;
}

std::map<string, OpSchema>& OpSchemaRegistry::schema_map() {
  static std::map<string, OpSchema> m;
  return m;
}

OpSchema& OpSchemaRegistry::NewSchema(const string& type, const string& file, int line) {
  auto& m = schema_map();
  CHECK(m.count(type) == 0) << "\nOpSchema(" << type << ") has been registered.";
  m.emplace(type, OpSchema(type, file, line));
  return m[type];
}

const OpSchema* OpSchemaRegistry::Schema(const string& type) {
  auto& m = schema_map();
  auto it = m.find(type);
  return it == m.end() ? nullptr : &it->second;
}

} // namespace dragon
