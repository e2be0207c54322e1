// Device-context plumbing of the C ABI: thin wrappers over the HIP runtime so
// that a host-side HIPContext needs no HIP header. Mirrors what Dragon's device
// contexts provide (dragon/core/context_cuda.h:156-332).
#include "common.h"
#include "dragon_hip_testing.h"

namespace {
inline int st(hipError_t e) { return e == hipSuccess ? DRAGON_HIP_OK : static_cast<int>(e); }

// Items of the single-read kernels (slices.h) whose wait ran out, counted on
// the device that ran them. Every device holds its own copy of the word.
__device__ uint32_t g_exchange_gave_up;
std::atomic<uint32_t> g_exchange_patience{0};
} // namespace

namespace dragon_hip {

uint32_t exchange_patience() { return g_exchange_patience.load(std::memory_order_relaxed); }

uint32_t* exchange_gave_up_counter() {
  static std::atomic<uint32_t*> resolved[kMaxDevices];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  uint32_t* p = resolved[device].load(std::memory_order_acquire);
  if (p) return p;
  void* addr = nullptr;
  if (hipGetSymbolAddress(&addr, HIP_SYMBOL(g_exchange_gave_up)) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  p = static_cast<uint32_t*>(addr);
  resolved[device].store(p, std::memory_order_release);
  return p;
}

} // namespace dragon_hip

extern "C" {

const char* dragon_hip_status_string(int status) {
  switch (status) {
    case DRAGON_HIP_OK: return "ok";
    case DRAGON_HIP_EINVAL: return "invalid argument (size, layout, null pointer or alignment)";
    case DRAGON_HIP_EDTYPE: return "unsupported dtype";
    case DRAGON_HIP_ESCRATCH: return "scratch buffer missing or too small";
    case DRAGON_HIP_ENODEVICE: return "no HIP device";
    case DRAGON_HIP_ETIMEOUT: return "timed out (not returned by any entry point)";
    case DRAGON_HIP_ELIMIT:
      return "shape needs more scratch than the static buffer of the no-allocation entry point";
    default: break;
  }
  if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
  return "unknown status";
}

int dragon_hip_device_count(int* count) {
  if (!count) return DRAGON_HIP_EINVAL;
  const hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) {
    *count = 0;
    (void)hipGetLastError();
  }
  return DRAGON_HIP_OK;
}
int dragon_hip_set_device(int device) { return st(hipSetDevice(device)); }
int dragon_hip_get_device(int* device) { return device ? st(hipGetDevice(device)) : DRAGON_HIP_EINVAL; }
int dragon_hip_device_name(int device, char* buf, size_t buf_bytes) {
  if (!buf || buf_bytes == 0) return DRAGON_HIP_EINVAL;
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return st(e);
  snprintf(buf, buf_bytes, "%s (%s)", prop.name, prop.gcnArchName);
  return DRAGON_HIP_OK;
}
int dragon_hip_device_capability(int device, int* major, int* minor) {
  if (!major || !minor) return DRAGON_HIP_EINVAL;
  hipDeviceProp_t prop;
  const hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return st(e);
  *major = prop.major, *minor = prop.minor;
  return DRAGON_HIP_OK;
}
int dragon_hip_device_sync(void) { return st(hipDeviceSynchronize()); }
int dragon_hip_mem_info(size_t* free_bytes, size_t* total_bytes) {
  if (!free_bytes || !total_bytes) return DRAGON_HIP_EINVAL;
  return st(hipMemGetInfo(free_bytes, total_bytes));
}
int dragon_hip_stream_create(void** stream) {
  if (!stream) return DRAGON_HIP_EINVAL;
  hipStream_t s;
  const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
  *stream = e == hipSuccess ? s : nullptr;
  return st(e);
}
int dragon_hip_stream_destroy(void* stream) { return st(hipStreamDestroy(static_cast<hipStream_t>(stream))); }
int dragon_hip_stream_query(void* stream, int* done) {
  if (!done) return DRAGON_HIP_EINVAL;
  const hipError_t e = hipStreamQuery(static_cast<hipStream_t>(stream));
  if (e == hipErrorNotReady) {
    *done = 0;
    return DRAGON_HIP_OK;
  }
  *done = e == hipSuccess ? 1 : 0;
  return st(e);
}
int dragon_hip_stream_sync(void* stream) { return st(hipStreamSynchronize(static_cast<hipStream_t>(stream))); }
int dragon_hip_malloc(void** ptr, size_t bytes) {
  if (!ptr) return DRAGON_HIP_EINVAL;
  return st(hipMalloc(ptr, bytes));
}
int dragon_hip_free(void* ptr) { return st(hipFree(ptr)); }
int dragon_hip_host_malloc(void** ptr, size_t bytes) {
  if (!ptr) return DRAGON_HIP_EINVAL;
  return st(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
}
int dragon_hip_host_free(void* ptr) { return st(hipHostFree(ptr)); }
int dragon_hip_memset_async(void* ptr, int value, size_t bytes, void* stream) {
  return st(hipMemsetAsync(ptr, value, bytes, static_cast<hipStream_t>(stream)));
}
int dragon_hip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
  static const hipMemcpyKind kinds[] = {hipMemcpyHostToHost, hipMemcpyHostToDevice,
                                        hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice};
  if (kind < 0 || kind > 3) return DRAGON_HIP_EINVAL;
  return st(hipMemcpyAsync(dst, src, bytes, kinds[kind], static_cast<hipStream_t>(stream)));
}
int dragon_hip_event_create(void** event) {
  if (!event) return DRAGON_HIP_EINVAL;
  hipEvent_t e;
  const hipError_t r = hipEventCreate(&e);
  *event = r == hipSuccess ? e : nullptr;
  return st(r);
}
int dragon_hip_event_destroy(void* event) { return st(hipEventDestroy(static_cast<hipEvent_t>(event))); }
int dragon_hip_event_record(void* event, void* stream) {
  return st(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}
int dragon_hip_event_sync(void* event) { return st(hipEventSynchronize(static_cast<hipEvent_t>(event))); }
int dragon_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!ms) return DRAGON_HIP_EINVAL;
  return st(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}


int dragon_hip_exchange_timed_out(void) {
  uint32_t* word = dragon_hip::exchange_gave_up_counter();
  uint32_t n = 0;
  if (!word || hipMemcpy(&n, word, sizeof(n), hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n > 0x7fffffffu ? 0x7fffffff : static_cast<int>(n);
}

void dragon_hip_exchange_reset(unsigned patience) {
  g_exchange_patience.store(patience, std::memory_order_relaxed);
  uint32_t* word = dragon_hip::exchange_gave_up_counter();
  if (word && hipMemset(word, 0, sizeof(uint32_t)) != hipSuccess) (void)hipGetLastError();
}

} // extern "C"
