#include "core/memory.h"

#include "core/context.h"

namespace dragon {

UnifiedMemory::~UnifiedMemory() {
  if (cpu_ptr_) CPUContext::Delete(cpu_ptr_);
  if (hip_ptr_) {
    HIPDeviceGuard guard(device_id_);
    HIPContext::Delete(hip_ptr_);
  }
}

void UnifiedMemory::ToCPU() {
  switch (state_) {
    case UNINITIALIZED:
      // Fresh memory is zero-filled, as the reference does (memory.cc:12-13).
      cpu_ptr_ = CPUContext::New(size_);
      CPUContext::Memset(size_, cpu_ptr_);
      state_ = STATE_AT_CPU;
      break;
    case STATE_AT_HIP: {
      if (cpu_ptr_ == nullptr) cpu_ptr_ = CPUContext::New(size_);
      HIPDeviceGuard guard(device_id_);
      HIPContext::Memcpy<CPUContext, HIPContext>(size_, cpu_ptr_, hip_ptr_);
      state_ = SYNCED;
      break;
    }
    case STATE_AT_CPU:
    case SYNCED:
      break;
  }
}

void UnifiedMemory::ToHIP(int device) {
  switch (state_) {
    case UNINITIALIZED: {
      HIPDeviceGuard guard(device);
      hip_ptr_ = HIPContext::New(size_);
      HIPContext::Memset(size_, hip_ptr_);
      device_id_ = device;
      state_ = STATE_AT_HIP;
      break;
    }
    case STATE_AT_CPU: {
      HIPDeviceGuard guard(device);
      if (hip_ptr_ == nullptr) {
        hip_ptr_ = HIPContext::New(size_);
        device_id_ = device;
      }
      CHECK_EQ(device_id_, device) << "\nMemory lives on another device.";
      HIPContext::Memcpy<HIPContext, CPUContext>(size_, hip_ptr_, cpu_ptr_);
      state_ = SYNCED;
      break;
    }
    case STATE_AT_HIP:
    case SYNCED:
      CHECK_EQ(device_id_, device) << "\nMemory lives on another device.";
      break;
  }
}

const void* UnifiedMemory::cpu_data() {
  ToCPU();
  return cpu_ptr_;
}

const void* UnifiedMemory::hip_data(int device) {
  ToHIP(device);
  return hip_ptr_;
}

void* UnifiedMemory::mutable_cpu_data() {
  ToCPU();
  state_ = STATE_AT_CPU;
  return cpu_ptr_;
}

void* UnifiedMemory::mutable_hip_data(int device) {
  ToHIP(device);
  state_ = STATE_AT_HIP;
  return hip_ptr_;
}

} // namespace dragon
