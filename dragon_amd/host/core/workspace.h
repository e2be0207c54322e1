// Workspace: owns named tensors, caches operators by their cache key and runs
// operator definitions, the roles of dragon/core/workspace.h and
// dragon/core/workspace.cc:73-94 this path needs. It also hands out scratch:
// data<T, Context>(n, name) returns the named buffer tensor ("BufferShared" by
// default) grown to at least n elements and never shrunk
// (dragon/core/workspace.h:81-92).
#pragma once

#include "core/common.h"
#include "core/operator_def.h"
#include "core/tensor.h"

namespace dragon {

class OperatorBase;

class Workspace {
 public:
  explicit Workspace(const string& name);
  ~Workspace();

  const string& name() const { return name_; }

  bool HasTensor(const string& name) const { return tensors_.count(name) > 0; }
  Tensor* CreateTensor(const string& name);
  Tensor* GetTensor(const string& name) const;  // LOG(FATAL) when missing
  Tensor* TryGetTensor(const string& name) const;
  void ResetTensor(const string& name);
  vector<string> tensors() const;

  // Creates (or fetches from the cache) the operator of `def` and runs it on
  // `stream`; `sync` waits for the stream afterwards.
  void RunOperator(const OperatorDef& def, int stream = 0, bool sync = true);
  size_t num_cached_operators() const { return operators_.size(); }

  template <typename T, class Context>
  T* data(size_t n, const string& name = "BufferShared", Context* ctx = nullptr) {
    Tensor* buffer = CreateTensor(name);
    const size_t have = buffer->has_memory() ? buffer->nbytes() : 0;
    const size_t need = n * sizeof(T);
    if (have < need || !buffer->IsType<T>()) {
      const size_t bytes = need > have ? need : have;
      buffer->Reshape({static_cast<int64_t>((bytes + sizeof(T) - 1) / sizeof(T))});
    }
    return buffer->template mutable_data<T, Context>(ctx);
  }

 private:
  string name_;
  std::map<string, std::unique_ptr<Tensor>> tensors_;
  std::map<string, std::unique_ptr<OperatorBase>> operators_;
};

} // namespace dragon
