#include "core/context.h"

#include <cstdlib>

#include "core/workspace.h"
#include "dragon_hip.h"

namespace dragon {

// ---------------------------------------------------------------- CPUContext

void* CPUContext::New(size_t size) {
  void* data = nullptr;
  const size_t aligned = (size + 63) / 64 * 64;
  CHECK(posix_memalign(&data, 64, aligned ? aligned : 64) == 0) << "\nFailed to allocate " << size << " bytes.";
  return data;
}

void CPUContext::Delete(void* ptr) { std::free(ptr); }

std::mutex& CPUContext::mutex() {
  static std::mutex m;
  return m;
}

// ---------------------------------------------------------------- helpers

void HipCheck(int status, const char* what) {
  if (status != 0) {
    LOG(FATAL) << "HIP error in " << what << ": " << dragon_hip_status_string(status) << " (status "
               << status << ")";
  }
}

// ---------------------------------------------------------------- HIPObjects

HIPObjects::HIPObjects() {
  for (int& seed : seeds_) seed = 3;  // DEFAULT_RNG_SEED of the reference's device objects
}

int HIPObjects::num_streams(int device_id) const {
  CHECK(device_id >= 0 && device_id < kMaxDevices) << "\nBad device id: " << device_id;
  const size_t n = streams_[device_id].size();
  return n == 0 ? 1 : static_cast<int>(n);  // id 0, the default stream, always exists
}

void HIPObjects::SetRandomSeed(int device_id, int seed) {
  CHECK(device_id >= 0 && device_id < kMaxDevices) << "\nBad device id: " << device_id;
  seeds_[device_id] = seed;
}

int HIPObjects::GetRandomSeed(int device_id) const {
  CHECK(device_id >= 0 && device_id < kMaxDevices) << "\nBad device id: " << device_id;
  return seeds_[device_id];
}

void HIPObjects::SetDevice(int device_id) { HIP_CHECK(dragon_hip_set_device(device_id)); }

HIPObjects::~HIPObjects() {
  for (int d = 0; d < kMaxDevices; ++d) {
    for (size_t i = 1; i < streams_[d].size(); ++i) {
      if (streams_[d][i] != nullptr) dragon_hip_stream_destroy(streams_[d][i]);
    }
  }
}

void* HIPObjects::stream(int device_id, int stream_id) {
  CHECK(device_id >= 0 && device_id < kMaxDevices) << "\nBad device id: " << device_id;
  auto& streams = streams_[device_id];
  if (streams.size() <= static_cast<size_t>(stream_id)) streams.resize(stream_id + 1, nullptr);
  if (stream_id > 0 && streams[stream_id] == nullptr) {
    HIPDeviceGuard guard(device_id);
    HIP_CHECK(dragon_hip_stream_create(&streams[stream_id]));
  }
  return streams[stream_id];
}

Workspace* HIPObjects::workspace(int device_id, int stream_id) {
  CHECK(device_id >= 0 && device_id < kMaxDevices) << "\nBad device id: " << device_id;
  auto& workspaces = workspaces_[device_id];
  if (workspaces.size() <= static_cast<size_t>(stream_id)) workspaces.resize(stream_id + 1);
  if (!workspaces[stream_id]) {
    workspaces[stream_id].reset(new Workspace(
        "HIPScratch:" + std::to_string(device_id) + ":" + std::to_string(stream_id)));
  }
  return workspaces[stream_id].get();
}

// ---------------------------------------------------------------- HIPContext

HIPContext::HIPContext(const DeviceOption& option)
    : device_id_(option.device_id), random_seed_(option.random_seed) {
  CHECK_EQ(option.device_type, static_cast<int>(PROTO_HIP)) << "\nExcepted a HIP device option.";
}

void* HIPContext::New(size_t size) {
  void* data = nullptr;
  HIP_CHECK(dragon_hip_malloc(&data, size));
  return data;
}

void HIPContext::Memset(size_t n, void* ptr, int value) {
  HIP_CHECK(dragon_hip_memset_async(ptr, value, n, nullptr));
  SynchronizeStream(nullptr);
}

void HIPContext::Memcpy(size_t n, void* dest, const void* src, int kind) {
  HIP_CHECK(dragon_hip_memcpy_async(dest, src, n, kind, nullptr));
  SynchronizeStream(nullptr);
}

template <>
void HIPContext::Memcpy<HIPContext, CPUContext>(size_t n, void* dest, const void* src) {
  Memcpy(n, dest, src, 1);
}
template <>
void HIPContext::Memcpy<CPUContext, HIPContext>(size_t n, void* dest, const void* src) {
  Memcpy(n, dest, src, 2);
}
template <>
void HIPContext::Memcpy<HIPContext, HIPContext>(size_t n, void* dest, const void* src) {
  Memcpy(n, dest, src, 3);
}

void HIPContext::Delete(void* ptr) { HIP_CHECK(dragon_hip_free(ptr)); }

void HIPContext::SynchronizeStream(void* stream) { HIP_CHECK(dragon_hip_stream_sync(stream)); }

void HIPContext::MemsetAsync(size_t n, void* ptr, int value) {
  HIP_CHECK(dragon_hip_memset_async(ptr, value, n, hip_stream()));
}

void HIPContext::MemcpyAsync(size_t n, void* dest, const void* src, int kind) {
  HIP_CHECK(dragon_hip_memcpy_async(dest, src, n, kind, hip_stream()));
}

template <>
void HIPContext::MemcpyAsync<HIPContext, CPUContext>(size_t n, void* dest, const void* src) {
  MemcpyAsync(n, dest, src, 1);
}
template <>
void HIPContext::MemcpyAsync<CPUContext, HIPContext>(size_t n, void* dest, const void* src) {
  MemcpyAsync(n, dest, src, 2);
}
template <>
void HIPContext::MemcpyAsync<HIPContext, HIPContext>(size_t n, void* dest, const void* src) {
  MemcpyAsync(n, dest, src, 3);
}

void HIPContext::SwitchToDevice(int stream) {
  HIP_CHECK(dragon_hip_set_device(device_id_));
  stream_id_ = stream;
}

void HIPContext::FinishDeviceComputation() { SynchronizeStream(hip_stream()); }

Workspace* HIPContext::workspace() { return objects().workspace(device_id_, stream_id_); }

void* HIPContext::hip_stream() { return hip_stream(device_id_, stream_id_); }

void* HIPContext::hip_stream(int device, int stream) { return objects().stream(device, stream); }

int HIPContext::device_count() {
  int count = 0;
  dragon_hip_device_count(&count);
  return count;
}

int HIPContext::current_device() {
  int device = 0;
  HIP_CHECK(dragon_hip_get_device(&device));
  return device;
}

std::mutex& HIPContext::mutex() {
  static std::mutex m;
  return m;
}

HIPObjects& HIPContext::objects() {
  static thread_local HIPObjects objects;
  return objects;
}

HIPStream::HIPStream(int device_id) : device_id_(device_id) {
  HIPObjects& objects = HIPContext::objects();
  stream_id_ = objects.num_streams(device_id);
  impl_ = objects.stream(device_id, stream_id_);
}

bool HIPStream::Query() {
  int done = 0;
  HIP_CHECK(dragon_hip_stream_query(impl_, &done));
  return done != 0;
}

void HIPStream::Synchronize() { HIPContext::SynchronizeStream(impl_); }

HIPDeviceGuard::HIPDeviceGuard(int new_id) : prev_id_(HIPContext::current_device()) {
  if (prev_id_ != new_id) HIP_CHECK(dragon_hip_set_device(new_id));
}

HIPDeviceGuard::~HIPDeviceGuard() {
  int now = 0;
  if (dragon_hip_get_device(&now) == 0 && now != prev_id_) dragon_hip_set_device(prev_id_);
}

} // namespace dragon
