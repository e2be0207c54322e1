// Device contexts. CPUContext is the host side (what tensors fed from and
// fetched to the host live in); HIPContext is the MI355X device context that
// sits next to it: stream, per-stream scratch workspace, memory management,
// with the member set every Dragon device context offers
// (dragon/core/context.h:61-169 for the CPU one, dragon/core/context_cuda.h:156-332
// and dragon/core/context_mlu.h:124-284 for device ones). HIPContext reaches the
// device only through the C ABI of include/dragon_hip.h.
#pragma once

#include "core/common.h"
#include "core/operator_def.h"

namespace dragon {

class Workspace;

class CPUContext {
 public:
  CPUContext() {}
  explicit CPUContext(const DeviceOption& option) : random_seed_(option.random_seed) {}

  static void* New(size_t size);
  static void Memset(size_t n, void* ptr, int value = 0) { std::memset(ptr, value, n); }
  template <class DestContext, class SrcContext>
  static void Memcpy(size_t n, void* dest, const void* src) { std::memcpy(dest, src, n); }
  static void Delete(void* ptr);

  void SwitchToDevice() {}
  void SwitchToDevice(int) {}
  void FinishDeviceComputation() {}
  int device() const { return 0; }
  int stream() const { return 0; }
  uint32_t random_seed() const { return random_seed_; }
  static std::mutex& mutex();

 private:
  uint32_t random_seed_ = 3;
};

// Thread-local device state: lazily created streams indexed by
// (device, stream id) and one scratch workspace per (device, stream), as
// CUDAObjects does (dragon/core/context_cuda.h:38-152, context_cuda.cc:35-46,120-129).
class HIPObjects {
 public:
  HIPObjects();
  ~HIPObjects();

  // Stream 0 is the legacy default stream (a null handle); others are created
  // non-blocking at the default priority on first use.
  void* stream(int device_id, int stream_id);
  Workspace* workspace(int device_id, int stream_id);
  // How many stream ids of the device have been handed out (id 0 included).
  int num_streams(int device_id) const;
  // The seed operators created for the device start from (CUDAObjects::SetRandomSeed's role).
  void SetRandomSeed(int device_id, int seed);
  int GetRandomSeed(int device_id) const;
  void SetDevice(int device_id);

  static constexpr int kMaxDevices = 16;

 private:
  vector<void*> streams_[kMaxDevices];
  vector<std::unique_ptr<Workspace>> workspaces_[kMaxDevices];
  int seeds_[kMaxDevices];
};

class HIPContext {
 public:
  HIPContext() : device_id_(0), random_seed_(3) {}
  explicit HIPContext(int device) : device_id_(device), random_seed_(3) {}
  explicit HIPContext(const DeviceOption& option);

  // Context::New / Memset / Memcpy / Delete on the current device.
  static void* New(size_t size);
  static void Memset(size_t n, void* ptr, int value = 0);
  template <class DestContext, class SrcContext>
  static void Memcpy(size_t n, void* dest, const void* src);
  static void Memcpy(size_t n, void* dest, const void* src, int kind);
  static void Delete(void* ptr);
  static void SynchronizeStream(void* stream);

  void MemsetAsync(size_t n, void* ptr, int value = 0);
  template <class DestContext, class SrcContext>
  void MemcpyAsync(size_t n, void* dest, const void* src);
  void MemcpyAsync(size_t n, void* dest, const void* src, int kind);

  // Operator::Run calls these around RunOnDevice (dragon/core/operator.h:214-219).
  void SwitchToDevice() { SwitchToDevice(0); }
  void SwitchToDevice(int stream);
  void FinishDeviceComputation();

  // The scratch workspace of the current (device, stream).
  Workspace* workspace();
  void* hip_stream();
  void* hip_stream(int device, int stream);

  int device() const { return device_id_; }
  int stream() const { return stream_id_; }
  void set_stream(int stream) { stream_id_ = stream; }
  uint32_t random_seed() const { return random_seed_; }

  static int device_count();
  static int current_device();
  static std::mutex& mutex();
  static HIPObjects& objects();

 private:
  int device_id_, stream_id_ = 0;
  uint32_t random_seed_;
};

// A stream of the calling thread's device objects behind a handle that a front
// end can hold (CUDAStream's role, dragon/core/context_cuda.h:339-395): the next
// unused stream id of the device, created non-blocking at the default priority.
class HIPStream {
 public:
  explicit HIPStream(int device_id);
  bool Query();
  void Synchronize();
  void* impl() const { return impl_; }
  int device_id() const { return device_id_; }
  int stream_id() const { return stream_id_; }

 private:
  int device_id_, stream_id_;
  void* impl_;
};

// Switches the current device for a scope (CUDADeviceGuard's role).
class HIPDeviceGuard {
 public:
  explicit HIPDeviceGuard(int new_id);
  ~HIPDeviceGuard();

 private:
  int prev_id_;
};

// Aborts through LOG(FATAL) with the library's message when a C-ABI call
// returns a non-zero status.
void HipCheck(int status, const char* what);
#define HIP_CHECK(expr) ::dragon::HipCheck((expr), #expr)

} // namespace dragon
