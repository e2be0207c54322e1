// Streaming probes: plain read, copy and fill kernels over a buffer, 16 bytes
// per lane per access with a grid-stride loop. They have no counterpart in the
// reference; the benchmark uses them to measure what fraction of the nominal
// HBM bandwidth a pure streaming kernel reaches on the device at hand, the
// practical ceiling every norm / softmax kernel is compared with, and the
// profiler uses the copy as the known-size kernel that calibrates its byte
// counters.
#include "common.h"

namespace dragon_hip {
namespace {

__global__ __launch_bounds__(256) void probe_read(const u32x4* __restrict__ src, size_t n,
                                                  uint32_t* __restrict__ sink) {
  uint32_t acc = 0;
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * 256) {
    const u32x4 v = src[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  // Never true for the probe's zero-filled input; keeps the loads alive.
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

__global__ __launch_bounds__(256) void probe_copy(const u32x4* __restrict__ src,
                                                  u32x4* __restrict__ dst, size_t n) {
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * 256) {
    __builtin_nontemporal_store(src[i], dst + i);
  }
}

__global__ __launch_bounds__(256) void probe_fill(u32x4* __restrict__ dst, size_t n) {
  const u32x4 v = {1u, 2u, 3u, 4u};
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * 256) {
    __builtin_nontemporal_store(v, dst + i);
  }
}

} // namespace
} // namespace dragon_hip

extern "C" int dragon_hip_stream_probe(int mode, const void* src, void* dst, size_t bytes,
                                       void* stream) {
  using namespace dragon_hip;
  if (bytes == 0) return DRAGON_HIP_OK;
  if (bytes % 16 != 0 || !dst || (mode != 2 && !src)) return DRAGON_HIP_EINVAL;
  if (!aligned16(src) || !aligned16(dst)) return DRAGON_HIP_EINVAL;
  const size_t n = bytes / 16;
  const size_t want = (n + 255) / 256;
  const unsigned grid = static_cast<unsigned>(want < static_cast<size_t>(num_cus()) * 64
                                                  ? want : static_cast<size_t>(num_cus()) * 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == 0) {
    hipLaunchKernelGGL(probe_read, dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(src), n,
                       static_cast<uint32_t*>(dst));
  } else if (mode == 1) {
    hipLaunchKernelGGL(probe_copy, dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(src),
                       static_cast<u32x4*>(dst), n);
  } else if (mode == 2) {
    hipLaunchKernelGGL(probe_fill, dim3(grid), dim3(256), 0, s, static_cast<u32x4*>(dst), n);
  } else {
    return DRAGON_HIP_EINVAL;
  }
  return status_of_launch();
}
