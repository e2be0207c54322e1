// Operator base classes, schema, registration macros and dtype dispatch:
// what dragon/core/operator.h:30-471, dragon/core/operator.cc:6-212 and
// dragon/core/operator_schema.{h,cc} provide, restricted to what the
// normalisation and softmax operators use.
#pragma once

#include "core/common.h"
#include "core/context.h"
#include "core/operator_def.h"
#include "core/registry.h"
#include "core/tensor.h"
#include "core/workspace.h"

namespace dragon {

class OperatorBase {
 public:
  OperatorBase(const OperatorDef& def, Workspace* ws);
  virtual ~OperatorBase() {}

  // Picks the registry for def.device_option().device_type() and constructs
  // the operator (dragon/core/operator.cc:69-98).
  static OperatorBase* New(const OperatorDef& def, Workspace* ws);

  // Rebinds inputs and outputs of a cached operator to another definition of
  // the same type (dragon/core/operator.cc:100-117).
  OperatorBase* DeriveFrom(const OperatorDef& def);

  virtual void Run(int stream = 0, bool sync = true) = 0;
  virtual void Setup() {}

  Tensor& Input(int i);
  Tensor* Output(int i);
  // Output i, sharing the memory of the first listed input that may be
  // overwritten in place when the definition names the same tensor.
  Tensor* Output(int i, const vector<int>& inputs);
  // Side tensors "<handle>/<name>" in the workspace: written by the forward
  // operator, read by its gradient (dragon/core/operator.cc:42-44,65-67).
  Tensor& Input(const string& name);
  Tensor* Output(const string& name);

  int InputSize() const { return static_cast<int>(inputs_.size()); }
  int OutputSize() const { return static_cast<int>(outputs_.size()); }

  template <typename T>
  T GetArgument(const string& name, const T& default_value);
  template <typename T>
  vector<T> GetRepeatedArgument(const string& name);

  const string& name() const { return def_.name; }
  const string& type() const { return def_.type; }
  const string& phase() const { return phase_; }
  const string& handle() const { return handle_; }
  const string& data_format() const { return data_format_; }
  const string& dtype() const { return dtype_; }
  const OperatorDef& def() const { return def_; }
  Workspace* workspace() const { return ws_; }
  void SwitchToPhase(const string& phase) { phase_ = phase; }

  string MessageForUnsupported(const string& value, const vector<string>& support) const;

 protected:
  Workspace* ws_;
  OperatorDef def_;
  string phase_, handle_, dtype_, data_format_;
  vector<Tensor*> inputs_, outputs_;
};

template <class Context>
class Operator : public OperatorBase {
 public:
  Operator(const OperatorDef& def, Workspace* ws) : OperatorBase(def, ws), ctx_(def.device_option) {}

  // dragon/core/operator.h:214-219
  void Run(int stream = 0, bool sync = true) final {
    Setup();
    ctx()->SwitchToDevice(stream);
    RunOnDevice();
    if (sync) ctx()->FinishDeviceComputation();
  }

  virtual void RunOnDevice() = 0;
  Context* ctx() { return &ctx_; }

 protected:
  Context ctx_;
};

#define USE_OPERATOR_FUNCTIONS                   \
  using OperatorBase::Input;                     \
  using OperatorBase::Output;                    \
  using OperatorBase::InputSize;                 \
  using OperatorBase::OutputSize;                \
  using OperatorBase::phase;                     \
  using OperatorBase::handle;                    \
  using OperatorBase::data_format;               \
  using OperatorBase::GetArgument;               \
  using Operator<Context>::ctx

#define OP_SINGLE_ARG(type, name, default) OperatorBase::GetArgument<type>(name, (default))
#define OP_REPEATED_ARG(type, name) OperatorBase::GetRepeatedArgument<type>(name)

// Canonical axis from the "axis" argument with bounds check
// (dragon/core/operator.h:376-384).
#define GET_OP_AXIS_ARG(name, num_axes, default)                                        \
  auto name = OP_SINGLE_ARG(int64_t, #name, default);                                   \
  name = name < 0 ? name + (num_axes) : name;                                           \
  CHECK(name >= 0 && name < (num_axes))                                                 \
      << "\nExcepted the <" << #name << "> in [-" << (num_axes) << ", " << (num_axes)   \
      << "), got " << OP_SINGLE_ARG(int64_t, #name, default) << ".";

// Shape and dtype check of a parameter tensor (dragon/core/operator.h:300-314).
#define INITIALIZE_TENSOR_VIA_SPEC(tensor, shape, type)                                  \
  do {                                                                                   \
    CHECK((tensor).template IsType<type>())                                              \
        << "\nExcepted the type of Tensor(" << (tensor).name() << ") is "                \
        << NameOf(TypeOf<type>::value) << ", got " << NameOf((tensor).meta()) << ".";    \
    const vec64_t expected_shape = (shape);                                              \
    CHECK((tensor).dims() == expected_shape)                                             \
        << "\nExcepted Tensor(" << (tensor).name() << ")'s dimensions are "             \
        << DimsToString(expected_shape) << ", got " << DimsToString((tensor).dims()) << "."; \
  } while (0)

// Calls op->DoRunWithType<T>() for the floating type of `tensor`
// (DispatchHelper<dtypes::Floating>, dragon/core/operator.h:256-296).
struct FloatingDispatch {
  template <class Op>
  static void Call(Op* op, const Tensor& tensor) {
    switch (tensor.meta()) {
      case DType::kFloat16: op->template DoRunWithType<float16>(); break;
      case DType::kBFloat16: op->template DoRunWithType<bfloat16>(); break;
      case DType::kFloat32: op->template DoRunWithType<float>(); break;
      case DType::kFloat64: op->template DoRunWithType<double>(); break;
      default:
        LOG(FATAL) << op->MessageForUnsupported(NameOf(tensor.meta()),
                                                {"float16", "bfloat16", "float32", "float64"});
    }
  }
};

// DispatchHelper<dtypes::Loss> (dragon/core/types.h:90): float and double.
struct LossDispatch {
  template <class Op>
  static void Call(Op* op, const Tensor& tensor) {
    switch (tensor.meta()) {
      case DType::kFloat32: op->template DoRunWithType<float>(); break;
      case DType::kFloat64: op->template DoRunWithType<double>(); break;
      default:
        LOG(FATAL) << op->MessageForUnsupported(NameOf(tensor.meta()), {"float32", "float64"});
    }
  }
};

// Input/output arity and in-place permissions of an operator type
// (dragon/core/operator_schema.h, operator_schema.cc:5-28).
class OpSchema {
 public:
  OpSchema() {}
  OpSchema(const string& type, const string& file, int line) : type_(type), file_(file), line_(line) {}

  OpSchema& NumInputs(int n) { return NumInputs(n, n); }
  OpSchema& NumInputs(int lo, int hi) {
    min_input_ = lo, max_input_ = hi;
    return *this;
  }
  OpSchema& NumOutputs(int n) { return NumOutputs(n, n); }
  OpSchema& NumOutputs(int lo, int hi) {
    min_output_ = lo, max_output_ = hi;
    return *this;
  }
  OpSchema& AllowInplace(const vector<std::pair<int, int>>& pairs) {
    inplace_ = pairs;
    return *this;
  }
  bool Verify(const OperatorDef& def) const;  // LOG(FATAL)s on violation
  bool CheckInplace(int input, int output) const;

 private:
  string type_, file_;
  int line_ = 0;
  int min_input_ = 0, max_input_ = 1 << 30, min_output_ = 0, max_output_ = 1 << 30;
  vector<std::pair<int, int>> inplace_;
};

class OpSchemaRegistry {
 public:
  static OpSchema& NewSchema(const string& type, const string& file, int line);
  static const OpSchema* Schema(const string& type);

 private:
  static std::map<string, OpSchema>& schema_map();
};

#define OPERATOR_SCHEMA(name) \
  static ::dragon::OpSchema* g_schema_##name = &::dragon::OpSchemaRegistry::NewSchema(#name, __FILE__, __LINE__)

// Per-device operator registries. Only the HIP one is populated here; the
// switch in OperatorBase::New reports every other device type as unavailable.
DECLARE_REGISTRY(HIPOperatorRegistry, OperatorBase, const OperatorDef&, Workspace*);

#define REGISTER_HIP_OPERATOR(name, ...) REGISTER_CLASS(HIPOperatorRegistry, name, __VA_ARGS__)
#define DEPLOY_HIP_OPERATOR(name)                      \
  REGISTER_HIP_OPERATOR(name, name##Op<HIPContext>);   \
  template class name##Op<HIPContext>;

} // namespace dragon
