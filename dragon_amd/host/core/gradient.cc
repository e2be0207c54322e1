#include "core/gradient.h"

namespace dragon {

DEFINE_REGISTRY(GradientRegistry, GradientMakerBase, const OperatorDef&, const vector<string>&);

void GradientMakerBase::AddGradientDef(const string& type, const vector<string>& inputs,
                                       const vector<string>& outputs) {
  OperatorDef g;
  g.type = type;
  g.input = inputs;
  g.output = outputs;
  grad_defs_.push_back(g);
}

void GradientMakerBase::Make() {
  CreateGradientDefs();
  string cache_key;
  for (auto& g : grad_defs_) {
    g.name = def_.name.empty() ? "" : def_.name + "_grad";
    g.device_option = def_.device_option;
    g.has_device_option = def_.has_device_option;
    bool has_name_arg = false;
    for (const auto& a : def_.arg) {
      if (a.name == "cache_key") {
        cache_key = a.s;
        continue;
      }
      if (a.name == "name") has_name_arg = true;
      g.arg.push_back(a);
    }
    if (!has_name_arg) {
      Argument* a = g.AddArg("name");
      a->s = def_.name, a->has_s = true;
    }
    if (!cache_key.empty()) {
      Argument* a = g.AddArg("cache_key");
      a->s = cache_key + "/grad", a->has_s = true;
    }
  }
}

vector<OperatorDef> MakeGradientDefs(const OperatorDef& def, const vector<string>& g_outputs,
                                     vector<string>* grad_inputs) {
  CHECK(GradientRegistry()->Has(def.type)) << "\nOperator(" << def.type << ") has no gradient.";
  std::unique_ptr<GradientMakerBase> maker(GradientRegistry()->Create(def.type, def, g_outputs));
  maker->Make();
  if (grad_inputs != nullptr) *grad_inputs = maker->grad_inputs();
  return maker->grad_defs();
}

} // namespace dragon
