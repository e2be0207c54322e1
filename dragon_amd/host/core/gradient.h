// Gradient definitions of the operators on this path: which operator computes
// the gradient, from which tensors, into which. Follows the GradientMaker
// classes registered next to each operator in the reference
// (dragon/core/gradient.h:43-181; layer_norm_op.cc:60-74, group_norm_op.cc:112-126,
// batch_norm_op.cc:254-268, softmax_op.cc:62, log_softmax_op.cc:62, lp_norm_op.cc:88).
#pragma once

#include "core/common.h"
#include "core/operator_def.h"
#include "core/registry.h"

namespace dragon {

class GradientMakerBase {
 public:
  GradientMakerBase(const OperatorDef& def, const vector<string>& g_outputs)
      : def_(def), g_outputs_(g_outputs), g_inputs_(def.input.size()) {}
  virtual ~GradientMakerBase() {}

  // Builds the gradient definitions: arguments and device option are copied
  // from the forward definition and a "name" argument carries the forward
  // operator's name, so that the gradient operator finds the forward
  // operator's side tensors (dragon/core/gradient.h:43-71).
  void Make();
  virtual void CreateGradientDefs() = 0;

  const vector<OperatorDef>& grad_defs() const { return grad_defs_; }
  const vector<string>& grad_inputs() const { return g_inputs_; }

 protected:
  const OperatorDef& def() const { return def_; }
  string I(int i) const { return def_.input.at(i); }
  string O(int i) const { return def_.output.at(i); }
  string GO(int i) const { return g_outputs_.at(i); }
  string GI(int i) {
    g_inputs_.at(i) = def_.input.at(i) + "_grad";
    return g_inputs_[i];
  }
  void AddGradientDef(const string& type, const vector<string>& inputs, const vector<string>& outputs);

 private:
  const OperatorDef& def_;
  vector<string> g_outputs_, g_inputs_;
  vector<OperatorDef> grad_defs_;
};

DECLARE_REGISTRY(GradientRegistry, GradientMakerBase, const OperatorDef&, const vector<string>&);
#define REGISTER_GRADIENT(name, ...) REGISTER_CLASS(GradientRegistry, name, __VA_ARGS__)

// Y = f(X) whose gradient needs only (Y, dY) and may overwrite dY
// (dragon/core/gradient.h:171-181).
class InplaceGradientMaker final : public GradientMakerBase {
 public:
  using GradientMakerBase::GradientMakerBase;
  void CreateGradientDefs() override {
    AddGradientDef(def().type + "Gradient", {O(0), GO(0)}, {GI(0)});
  }
};

// Y1..Ym = f(X1..Xn) whose gradient operator takes (X1..Xn, dY1..dYm) and
// produces (dX1..dXn) (dragon/core/gradient.h:132-150).
class GenericGradientMaker final : public GradientMakerBase {
 public:
  using GradientMakerBase::GradientMakerBase;
  void CreateGradientDefs() override {
    vector<string> inputs(def().input.begin(), def().input.end());
    vector<string> outputs;
    for (size_t i = 0; i < def().output.size(); ++i) inputs.push_back(GO(static_cast<int>(i)));
    for (size_t i = 0; i < def().input.size(); ++i) outputs.push_back(GI(static_cast<int>(i)));
    AddGradientDef(def().type + "Gradient", inputs, outputs);
  }
};

// Gradient definitions of `def` given the names of the output gradients.
// `grad_inputs` receives the name of each input's gradient ("" if none).
vector<OperatorDef> MakeGradientDefs(const OperatorDef& def, const vector<string>& g_outputs,
                                     vector<string>* grad_inputs);

} // namespace dragon
