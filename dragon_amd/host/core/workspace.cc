#include "core/workspace.h"

#include "core/operator.h"

namespace dragon {

Workspace::Workspace(const string& name) : name_(name) {}

Workspace::~Workspace() {}

Tensor* Workspace::CreateTensor(const string& name) {
  auto it = tensors_.find(name);
  if (it != tensors_.end()) return it->second.get();
  auto* tensor = new Tensor(name);
  tensors_[name].reset(tensor);
  return tensor;
}

Tensor* Workspace::TryGetTensor(const string& name) const {
  auto it = tensors_.find(name);
  return it == tensors_.end() ? nullptr : it->second.get();
}

Tensor* Workspace::GetTensor(const string& name) const {
  Tensor* tensor = TryGetTensor(name);
  CHECK(tensor != nullptr) << "\nTensor(" << name << ") is not in workspace " << name_ << ".";
  return tensor;
}

void Workspace::ResetTensor(const string& name) { tensors_.erase(name); }

vector<string> Workspace::tensors() const {
  vector<string> names;
  for (const auto& kv : tensors_) names.push_back(kv.first);
  return names;
}

void Workspace::RunOperator(const OperatorDef& def, int stream, bool sync) {
  // Operators are cached under the "cache_key" argument, the convention of the
  // reference's eager executor (dragon/python/core/autograph/op_lib.py:56-92,
  // dragon/core/workspace.cc:73-94); without one the operator lives for this call.
  const Argument* key = def.FindArg("cache_key");
  if (key != nullptr && key->has_s) {
    auto it = operators_.find(key->s);
    if (it == operators_.end()) {
      it = operators_.emplace(key->s, std::unique_ptr<OperatorBase>(OperatorBase::New(def, this))).first;
    }
    it->second->DeriveFrom(def)->Run(stream, sync);
  } else {
    std::unique_ptr<OperatorBase> op(OperatorBase::New(def, this));
    op->Run(stream, sync);
  }
}

} // namespace dragon
