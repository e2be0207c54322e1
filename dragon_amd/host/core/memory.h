// UnifiedMemory: one logical buffer with a host copy and a device copy that
// are allocated lazily and synchronised on access, following
// dragon/core/memory.h:28-41 and dragon/core/memory.cc:9-83,142-202 with a
// STATE_AT_HIP state next to STATE_AT_CPU.
#pragma once

#include "core/common.h"

namespace dragon {

class UnifiedMemory {
 public:
  enum State { UNINITIALIZED = 0, STATE_AT_CPU = 1, STATE_AT_HIP = 2, SYNCED = 3 };

  UnifiedMemory() {}
  explicit UnifiedMemory(size_t size) : size_(size) {}
  ~UnifiedMemory();
  UnifiedMemory(const UnifiedMemory&) = delete;
  UnifiedMemory& operator=(const UnifiedMemory&) = delete;

  // Read access: brings the requested side up to date.
  const void* cpu_data();
  const void* hip_data(int device);
  // Write access: brings the side up to date and marks it the owner.
  void* mutable_cpu_data();
  void* mutable_hip_data(int device);

  size_t size() const { return size_; }
  // Bytes held on the given device ("cpu" or "hip"), 0 when nothing is allocated there.
  size_t size(const string& device_type, int device_id) const {
    if (device_type == "cpu") return cpu_ptr_ ? size_ : 0;
    if (device_type == "hip") return hip_ptr_ && device_id_ == device_id ? size_ : 0;
    return 0;
  }
  // Where the up-to-date copy lives (UnifiedMemory::info's "device_type" / "device_id").
  string device_type() const { return state_ == STATE_AT_HIP ? "hip" : "cpu"; }
  State state() const { return state_; }
  int device() const { return device_id_; }

 private:
  void ToCPU();
  void ToHIP(int device);

  State state_ = UNINITIALIZED;
  size_t size_ = 0;
  void* cpu_ptr_ = nullptr;
  void* hip_ptr_ = nullptr;
  int device_id_ = 0;
};

} // namespace dragon
