// Tensor: name, shape, element type and a (possibly shared) UnifiedMemory.
// The subset of dragon/core/tensor.h the normalisation and softmax operators
// use: Reshape / ReshapeLike, count / dim / ndim, typed data access through a
// context, name and type queries.
#pragma once

#include "core/common.h"
#include "core/context.h"
#include "core/memory.h"

namespace dragon {

class Tensor {
 public:
  Tensor() {}
  explicit Tensor(const string& name) : name_(name) {}

  Tensor* Reshape(const vec64_t& dims) {
    dims_ = dims;
    size_ = 1;
    for (auto d : dims) {
      CHECK_GE(d, 0) << "\nNegative dimension in shape " << DimsToString(dims);
      size_ *= static_cast<size_t>(d);
    }
    return this;
  }
  Tensor* ReshapeLike(const Tensor& other) { return Reshape(other.dims_); }

  // Shares the memory of `other` (the in-place output convention).
  Tensor* MapFrom(Tensor* other) {
    if (other != this) {
      memory_ = other->memory_;
      meta_ = other->meta_;
      capacity_ = other->capacity_;
    }
    return this;
  }

  const string& name() const { return name_; }
  bool has_name() const { return !name_.empty() && name_ != "NULL"; }
  const vec64_t& dims() const { return dims_; }
  int ndim() const { return static_cast<int>(dims_.size()); }
  int64_t dim(int i) const {
    const int n = ndim();
    CHECK(i >= -n && i < n) << "\nTensor(" << name_ << ") has no axis " << i;
    return dims_[i < 0 ? i + n : i];
  }
  int64_t count() const { return static_cast<int64_t>(size_); }
  int64_t count(int start, int end) const {
    int64_t n = 1;
    for (int i = start; i < end; ++i) n *= dim(i);
    return n;
  }
  int64_t count(int start) const { return count(start, ndim()); }
  size_t size() const { return size_; }
  size_t nbytes() const { return size_ * SizeOf(meta_); }
  size_t capacity() const { return capacity_; }
  DType meta() const { return meta_; }
  void set_meta(DType meta) { meta_ = meta; }
  bool has_memory() const { return memory_ != nullptr; }
  UnifiedMemory* memory() const { return memory_.get(); }

  template <typename T>
  bool IsType() const {
    return meta_ == TypeOf<T>::value;
  }

  // Typed access. mutable_data (re)allocates when the type changes or the
  // tensor outgrew its capacity; capacity is rounded up to 512 bytes
  // (dragon/core/tensor.h:331).
  template <typename T, class Context>
  T* mutable_data(Context* ctx = nullptr) {
    const DType want = TypeOf<T>::value;
    const size_t bytes = size_ * sizeof(T);
    if (!memory_ || meta_ != want || capacity_ < bytes) {
      meta_ = want;
      capacity_ = (bytes + 511) / 512 * 512;
      memory_.reset(new UnifiedMemory(capacity_ ? capacity_ : 512));
    }
    return static_cast<T*>(raw_mutable_data<Context>(ctx));
  }

  template <typename T, class Context>
  const T* data(Context* ctx = nullptr) {
    CHECK(memory_ != nullptr) << "\nTensor(" << name_ << ") has no memory: it was never written.";
    CHECK(meta_ == TypeOf<T>::value)
        << "\nTensor(" << name_ << ") holds " << NameOf(meta_) << ", requested "
        << NameOf(TypeOf<T>::value) << ".";
    return static_cast<const T*>(raw_data<Context>(ctx));
  }

  template <class Context>
  const void* raw_data(Context* ctx = nullptr);
  template <class Context>
  void* raw_mutable_data(Context* ctx = nullptr);

 private:
  string name_;
  vec64_t dims_;
  size_t size_ = 0, capacity_ = 0;
  DType meta_ = DType::kUndefined;
  std::shared_ptr<UnifiedMemory> memory_;
};

template <>
inline const void* Tensor::raw_data<CPUContext>(CPUContext*) {
  return memory_->cpu_data();
}
template <>
inline void* Tensor::raw_mutable_data<CPUContext>(CPUContext*) {
  return memory_->mutable_cpu_data();
}
template <>
inline const void* Tensor::raw_data<HIPContext>(HIPContext* ctx) {
  return memory_->hip_data(ctx ? ctx->device() : HIPContext::current_device());
}
template <>
inline void* Tensor::raw_mutable_data<HIPContext>(HIPContext* ctx) {
  return memory_->mutable_hip_data(ctx ? ctx->device() : HIPContext::current_device());
}

} // namespace dragon
