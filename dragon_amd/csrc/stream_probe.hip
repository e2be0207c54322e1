// Streaming probes: plain read, copy, fill and two-reads-one-write kernels over
// large buffers. They have no counterpart in the reference; the benchmark uses
// them to measure what a pure streaming kernel reaches on the device at hand
// at the read : write mixes of the norm / softmax kernels (1 : 0, 1 : 1, 0 : 1,
// 2 : 1), the practical ceiling beside the nominal HBM peak, and the profiler
// uses the copy as the known-size kernel that calibrates its byte counters.
//
// Every thread keeps kInFlight independent 16-byte loads outstanding: a
// workgroup takes a chunk of kInFlight x 256 packets, and within a chunk load k
// of thread t is packet k * 256 + t, so each wavefront access is one contiguous
// KiB. Measured on MI355X over 1 GiB buffers (fractions of the nominal 8 TB/s):
// one load in flight per thread and a grid-stride loop read 10-30% low, which
// made kernels appear to beat the probe; four loads in flight, non-temporal
// loads (each byte is used once) and one chunk per workgroup give 7.1 TB/s
// read-only (0.89), 6.2 TB/s copy (0.78), 6.0 TB/s fill (0.75), 6.25 TB/s for
// two reads and one write (0.78); eight or sixteen loads in flight, plain loads
// or a persistent grid are each 3-10% slower.
#include "common.h"

namespace dragon_hip {
namespace {

// The default shape of the probe, and the ones a caller may ask for instead
// (dragon_hip_stream_probe_shape): which shape streams fastest depends on the
// size of the tensors, so a benchmark that wants a ceiling takes the best of them.
constexpr int kDefaultThreads = 256;
constexpr int kDefaultInFlight = 4;

__device__ __forceinline__ u32x4 load16(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store16(u32x4* p, const u32x4 v) { __builtin_nontemporal_store(v, p); }

// kReads source tensors of n packets each (laid out back to back from src),
// kWrites destination tensors. The chunked body covers whole chunks; the
// packets past the last whole chunk are walked one by one.
template <int kReads, int kWrites, int kProbeThreads, int kInFlight>
__global__ __launch_bounds__(kProbeThreads) void probe_stream(const u32x4* __restrict__ src,
                                                              u32x4* __restrict__ dst, size_t n,
                                                              uint32_t* __restrict__ sink) {
  constexpr size_t kChunk = static_cast<size_t>(kProbeThreads) * kInFlight;  // packets
  const size_t chunks = n / kChunk;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (size_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const size_t base = c * kChunk + threadIdx.x;
    u32x4 v[kInFlight];
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      if constexpr (kReads == 0) {
        v[k] = u32x4{1u, 2u, 3u, static_cast<uint32_t>(k)};
      } else {
        v[k] = load16(src + base + k * kProbeThreads);
      }
    }
    if constexpr (kReads == 2) {
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) v[k] ^= load16(src + n + base + k * kProbeThreads);
    }
#pragma unroll
    for (int k = 0; k < kInFlight; ++k) {
      if constexpr (kWrites == 1) {
        store16(dst + base + k * kProbeThreads, v[k]);
      } else {
        acc ^= v[k];
      }
    }
  }
  for (size_t i = chunks * kChunk + static_cast<size_t>(blockIdx.x) * kProbeThreads + threadIdx.x;
       i < n; i += static_cast<size_t>(gridDim.x) * kProbeThreads) {
    u32x4 v = {1u, 2u, 3u, 4u};
    if constexpr (kReads >= 1) v = load16(src + i);
    if constexpr (kReads == 2) v ^= load16(src + n + i);
    if constexpr (kWrites == 1) {
      store16(dst + i, v);
    } else {
      acc ^= v;
    }
  }
  if constexpr (kWrites == 0) {
    // Keeps the loads alive; one word at most is written, and only for data that
    // folds to this constant.
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc.x;
  }
}

// Two reads and one write as a persistent kernel streams them: chunk c of workgroup b is
// b + c * grid, kDepth chunks are requested ahead into a ring of register tiles over which
// the loop is unrolled (a tile never moves between registers), and kBarrier puts a workgroup
// barrier between a chunk's loads and its stores. Measured on MI355X over three 64 MB tensors
// (cold), per call: one chunk per workgroup 32.0 us; persistent 1024-thread workgroups, one
// chunk ahead, 34.8 us; two chunks ahead 1-3 us more. A wavefront's loads and stores complete in issue order, so in a loop the wait for a
// chunk's loads also waits for the stores issued before them.
template <int kThreads, int kInFlight, int kDepth, bool kBarrier>
__global__ __launch_bounds__(kThreads) void probe_persistent(const u32x4* __restrict__ a,
                                                             const u32x4* __restrict__ b,
                                                             u32x4* __restrict__ c, const size_t chunks) {
  constexpr int kRing = kDepth + 1;
  constexpr size_t kChunk = static_cast<size_t>(kThreads) * kInFlight;
  u32x4 ra[kRing][kInFlight], rb[kRing][kInFlight];
  size_t chunk = blockIdx.x;
  auto request = [&](const int k, const size_t at) {
    const size_t from = at < chunks ? at : 0;
#pragma unroll
    for (int i = 0; i < kInFlight; ++i) {
      ra[k][i] = load16(a + from * kChunk + i * kThreads + threadIdx.x);
      rb[k][i] = load16(b + from * kChunk + i * kThreads + threadIdx.x);
    }
  };
#pragma unroll
  for (int k = 0; k < kDepth; ++k) request(k, chunk + static_cast<size_t>(k) * gridDim.x);
  while (chunk < chunks) {
#pragma unroll
    for (int k = 0; k < kRing; ++k) {
      if (chunk < chunks) {
        request((k + kDepth) % kRing, chunk + static_cast<size_t>(kDepth) * gridDim.x);
        u32x4 o[kInFlight];
#pragma unroll
        for (int i = 0; i < kInFlight; ++i) o[i] = ra[k][i] ^ rb[k][i];
        if (kBarrier) __syncthreads();
#pragma unroll
        for (int i = 0; i < kInFlight; ++i) store16(c + chunk * kChunk + i * kThreads + threadIdx.x, o[i]);
        chunk += gridDim.x;
      }
    }
  }
}

// The same with the roles split: the first half of the workgroup loads and leaves its result
// in LDS, the second half writes the previous chunk's result out. A wavefront that only
// stores never waits for loads and one that only loads never waits for store
// acknowledgements (34.8 -> 32.5 us per call for the 1024-thread shape above).
template <int kThreads, int kInFlight, int kDepth>
__global__ __launch_bounds__(kThreads) void probe_persistent_split(const u32x4* __restrict__ a,
                                                                   const u32x4* __restrict__ b,
                                                                   u32x4* __restrict__ c,
                                                                   const size_t chunks) {
  constexpr int kHalf = kThreads / 2;
  constexpr size_t kChunk = static_cast<size_t>(kHalf) * kInFlight;
  constexpr int kRing = kDepth + 1;
  __shared__ u32x4 buf[2][kInFlight][kHalf];
  const bool loader = threadIdx.x < kHalf;
  const int t = threadIdx.x % kHalf;
  u32x4 ra[kRing][kInFlight], rb[kRing][kInFlight];
  size_t chunk = blockIdx.x;
  auto request = [&](const int k, const size_t at) {
    const size_t from = at < chunks ? at : 0;
#pragma unroll
    for (int i = 0; i < kInFlight; ++i) {
      ra[k][i] = load16(a + from * kChunk + i * kHalf + t);
      rb[k][i] = load16(b + from * kChunk + i * kHalf + t);
    }
  };
  if (loader) {
#pragma unroll
    for (int k = 0; k < kDepth; ++k) request(k, chunk + static_cast<size_t>(k) * gridDim.x);
  }
  int parity = 0;
  size_t prev = 0;
  bool have_prev = false;
  // One trip more than there are chunks: the last trip only writes the last chunk out.
  while (chunk < chunks || have_prev) {
#pragma unroll
    for (int k = 0; k < kRing; ++k) {
      if (chunk < chunks || have_prev) {
        const bool cur = chunk < chunks;
        if (loader) {
          if (cur) {
            request((k + kDepth) % kRing, chunk + static_cast<size_t>(kDepth) * gridDim.x);
#pragma unroll
            for (int i = 0; i < kInFlight; ++i) buf[parity][i][t] = ra[k][i] ^ rb[k][i];
          }
        } else if (have_prev) {
#pragma unroll
          for (int i = 0; i < kInFlight; ++i) store16(c + prev * kChunk + i * kHalf + t, buf[parity ^ 1][i][t]);
        }
        __syncthreads();
        have_prev = cur;
        prev = chunk;
        parity ^= 1;
        chunk += gridDim.x;
      }
    }
  }
}

template <int kThreads, int kInFlight>
int launch_probe(int mode, const void* src, void* dst, size_t bytes, hipStream_t s) {
  const size_t n = bytes / 16;
  constexpr size_t kChunk = static_cast<size_t>(kThreads) * kInFlight;
  const size_t chunks = n / kChunk;
  const size_t want = chunks > 0 ? chunks : (n + kThreads - 1) / kThreads;
  const size_t cap = 0x7fffffffu;  // one chunk per workgroup up to the launch limit
  const unsigned grid = static_cast<unsigned>(want < cap ? want : cap);
  const u32x4* sp = static_cast<const u32x4*>(src);
  u32x4* dp = static_cast<u32x4*>(dst);
  uint32_t* sink = static_cast<uint32_t*>(dst);
  switch (mode) {
    case 0:
      hipLaunchKernelGGL((probe_stream<1, 0, kThreads, kInFlight>), dim3(grid), dim3(kThreads), 0, s, sp, dp, n, sink);
      break;
    case 1:
      hipLaunchKernelGGL((probe_stream<1, 1, kThreads, kInFlight>), dim3(grid), dim3(kThreads), 0, s, sp, dp, n, sink);
      break;
    case 2:
      hipLaunchKernelGGL((probe_stream<0, 1, kThreads, kInFlight>), dim3(grid), dim3(kThreads), 0, s, sp, dp, n, sink);
      break;
    case 3:
      hipLaunchKernelGGL((probe_stream<2, 1, kThreads, kInFlight>), dim3(grid), dim3(kThreads), 0, s, sp, dp, n, sink);
      break;
    default: return DRAGON_HIP_EINVAL;
  }
  return status_of_launch();
}

} // namespace
} // namespace dragon_hip

extern "C" int dragon_hip_stream_probe_shape(int mode, int threads, int in_flight, const void* src,
                                             void* dst, size_t bytes, void* stream) {
  using namespace dragon_hip;
  if (bytes == 0) return DRAGON_HIP_OK;
  if (bytes % 16 != 0 || !dst || (mode != 2 && !src)) return DRAGON_HIP_EINVAL;
  if (!aligned16(src) || !aligned16(dst)) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SHAPE(T, F) \
  if (threads == T && in_flight == F) return launch_probe<T, F>(mode, src, dst, bytes, s);
  SHAPE(64, 1) SHAPE(64, 2) SHAPE(64, 4) SHAPE(256, 1) SHAPE(256, 2) SHAPE(256, 4) SHAPE(256, 8)
  SHAPE(512, 2) SHAPE(1024, 2)
#undef SHAPE
  return DRAGON_HIP_EINVAL;
}

extern "C" int dragon_hip_stream_probe_persistent(int threads, int in_flight, int per_cu, int depth,
                                                  int barrier, int store_waves, const void* src,
                                                  void* dst, size_t bytes, void* stream) {
  using namespace dragon_hip;
  if (bytes == 0) return DRAGON_HIP_OK;
  if (bytes % 16 != 0 || !src || !dst || !aligned16(src) || !aligned16(dst)) return DRAGON_HIP_EINVAL;
  if (per_cu < 1 || per_cu * threads > 2048 || depth < 0 || depth > 3) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t n = bytes / 16;
  const u32x4* a = static_cast<const u32x4*>(src);
  const u32x4* b = a + n;
  u32x4* c = static_cast<u32x4*>(dst);
  const unsigned grid = static_cast<unsigned>(per_cu) * num_cus();
#define SHAPE(T, F, D)                                                                            \
  if (threads == T && in_flight == F && depth == D) {                                             \
    if (store_waves) {                                                                            \
      const size_t chunks = n / (static_cast<size_t>(T / 2) * F);                                 \
      if (chunks * (T / 2) * F != n) return DRAGON_HIP_EINVAL;                                    \
      hipLaunchKernelGGL((probe_persistent_split<T, F, D>), dim3(grid), dim3(T), 0, s, a, b, c, chunks); \
    } else {                                                                                      \
      const size_t chunks = n / (static_cast<size_t>(T) * F);                                     \
      if (chunks * T * F != n) return DRAGON_HIP_EINVAL;                                          \
      if (barrier) {                                                                              \
        hipLaunchKernelGGL((probe_persistent<T, F, D, true>), dim3(grid), dim3(T), 0, s, a, b, c, chunks); \
      } else {                                                                                    \
        hipLaunchKernelGGL((probe_persistent<T, F, D, false>), dim3(grid), dim3(T), 0, s, a, b, c, chunks); \
      }                                                                                           \
    }                                                                                             \
    return status_of_launch();                                                                    \
  }
#define DEPTHS(T, F) SHAPE(T, F, 0) SHAPE(T, F, 1) SHAPE(T, F, 2) SHAPE(T, F, 3)
  DEPTHS(256, 1) DEPTHS(256, 2) DEPTHS(512, 1) DEPTHS(512, 2) DEPTHS(1024, 1) DEPTHS(1024, 2)
#undef DEPTHS
#undef SHAPE
  return DRAGON_HIP_EINVAL;
}

extern "C" int dragon_hip_stream_probe(int mode, const void* src, void* dst, size_t bytes,
                                       void* stream) {
  return dragon_hip_stream_probe_shape(mode, dragon_hip::kDefaultThreads, dragon_hip::kDefaultInFlight,
                                       src, dst, bytes, stream);
}
