// Shared device-side building blocks for the gfx950 norm / softmax kernels:
// 16-byte packet I/O with conversion to the accumulator type, wave64 and
// workgroup reductions, and the launch helpers every entry point uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <atomic>

#include "dragon_hip.h"

namespace dragon_hip {

constexpr int kWaveSize = 64;  // CDNA wavefront width
constexpr int kMaxDevices = 64;  // per-device state is kept in arrays of this size

// Compute units of the current device (256 on MI355X: 8 XCDs x 32), asked of the
// runtime once per device. Where no device answers (size queries on a host
// without one) the MI355X figure is assumed.
inline int num_cus() {
  constexpr int kAssumed = 256;
  static std::atomic<int> cached[kMaxDevices];
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    (void)hipGetLastError();
    return kAssumed;
  }
  int n = cached[device].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
      n <= 0) {
    (void)hipGetLastError();
    n = kAssumed;
  }
  cached[device].store(n, std::memory_order_relaxed);
  return n;
}

// ---------------------------------------------------------------------------
// Launch trace. Every kernel launch of the library goes through the macro below,
// which notes the kernel's spelling and workgroup size in a per-thread trace when
// one is being recorded and, in plan-only mode, launches nothing. The plan query
// of the C ABI (dragon_hip_plan_name) runs an entry point that way with made-up
// addresses: it reports which kernel flavours a call would take without touching
// a device, so that a test can pin the routing of the shapes that matter.
// ---------------------------------------------------------------------------
struct LaunchTrace {
  bool recording = false;
  bool plan_only = false;  // record only: no kernel is launched
  char text[1024];
  size_t used = 0;
};
inline LaunchTrace& launch_trace() {
  static thread_local LaunchTrace trace;
  return trace;
}
inline bool plan_only() { return launch_trace().plan_only; }
// Appends "name[threads];" with blanks and the outer parentheses of `spelling` removed.
inline void note_launch(const char* spelling, dim3 block) {
  LaunchTrace& t = launch_trace();
  if (!t.recording) return;
  const size_t cap = sizeof(t.text) - 24;
  int depth = 0;
  for (const char* c = spelling; *c && t.used < cap; ++c) {
    if (*c == ' ' || *c == '\t' || *c == '\n') continue;
    if (*c == '(' && depth++ == 0 && c == spelling) continue;
    if (*c == ')' && --depth == 0 && c[1] == 0 && spelling[0] == '(') continue;
    t.text[t.used++] = *c;
  }
  char tail[24];
  const int n = snprintf(tail, sizeof(tail), "[%u];", block.x * block.y * block.z);
  for (int i = 0; i < n && t.used + 1 < sizeof(t.text); ++i) t.text[t.used++] = tail[i];
  t.text[t.used] = 0;
}
// A launcher that holds its kernel in a variable names the flavour itself.
inline void note_flavour(const char* name) {
  LaunchTrace& t = launch_trace();
  if (!t.recording) return;
  for (const char* c = name; *c && t.used + 2 < sizeof(t.text); ++c) t.text[t.used++] = *c;
  t.text[t.used++] = ':';
  t.text[t.used] = 0;
}

// A number that a plan depends on (slices per unit, rows per chunk ...): "key=value:".
inline void note_number(const char* key, long long value) {
  LaunchTrace& t = launch_trace();
  if (!t.recording) return;
  char item[64];
  const int n = snprintf(item, sizeof(item), "%s=%lld:", key, value);
  for (int i = 0; i < n && t.used + 1 < sizeof(t.text); ++i) t.text[t.used++] = item[i];
  t.text[t.used] = 0;
}

// Where a kernel that can record its phases leaves them for the calling thread's next launch
// (null: nothing is recorded). Set only by the *_timeline entry points of the C ABI, which
// exist for measurement: a handful of device clock reads per workgroup.
struct TimelineTarget {
  unsigned long long* stamps = nullptr;  // device memory, kTimelineWords words per workgroup
  size_t workgroups = 0;                 // how many workgroups it has room for
};
constexpr int kTimelineWords = 6;  // start, first data, loop end, end, XCD, rows done
inline TimelineTarget& timeline_target() {
  static thread_local TimelineTarget target;
  return target;
}

#undef hipLaunchKernelGGL
#define hipLaunchKernelGGL(kernelName, numBlocks, numThreads, memPerBlock, streamId, ...)       \
  do {                                                                                         \
    ::dragon_hip::note_launch(#kernelName, dim3(numThreads));                                  \
    if (!::dragon_hip::plan_only()) {                                                          \
      hipLaunchKernelGGLInternal((kernelName), (numBlocks), (numThreads), (memPerBlock),       \
                                 (streamId), __VA_ARGS__);                                     \
    }                                                                                          \
  } while (0)

// 16-bit storage types: same bit layout as dragon::float16 / dragon::bfloat16
// (dragon/core/types.h:36-42), a bare unsigned short.
struct f16_t {
  uint16_t x;
};
struct bf16_t {
  uint16_t x;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));

// IO<T>: how a tensor element type travels through HBM.
//   Acc    accumulator type (math::Traits<T>::accumulator_type,
//          dragon/utils/math/types.h:69-152)
//   kVec   elements per 16-byte packet
//   unpack / pack  one 16-byte packet (four dwords) <-> kVec accumulators
//   load1 / store1 one element (tails and unaligned tensors)
// Rounding on store is round-to-nearest-even in hardware, which is what the
// reference's software conversion implements (dragon/utils/conversions.h:42-106).
template <typename T>
struct IO;

template <>
struct IO<float> {
  using Acc = float;
  static constexpr int kVec = 4;
  // Vector elements are copied to scalars before any bit cast: a bit cast
  // applied directly to an element expression (t.x, t[i]) reads element 0.
  static __device__ __forceinline__ void unpack(const u32x4 t, float (&v)[4]) {
    const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_bit_cast(float, w[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) {
    const u32x4 t = {__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]),
                     __builtin_bit_cast(uint32_t, v[2]), __builtin_bit_cast(uint32_t, v[3])};
    return t;
  }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};

template <>
struct IO<double> {
  using Acc = double;
  static constexpr int kVec = 2;
  static __device__ __forceinline__ void unpack(const u32x4 t, double (&v)[2]) {
    const f64x2 d = __builtin_bit_cast(f64x2, t);
    v[0] = d.x, v[1] = d.y;
  }
  static __device__ __forceinline__ u32x4 pack(const double (&v)[2]) {
    const f64x2 d = {v[0], v[1]};
    return __builtin_bit_cast(u32x4, d);
  }
  static __device__ __forceinline__ double load1(const double* p) { return *p; }
  static __device__ __forceinline__ void store1(double* p, double v) { *p = v; }
};

template <>
struct IO<f16_t> {
  using Acc = float;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ void unpack(const u32x4 t, float (&v)[8]) {
    const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const h16x2 h = __builtin_bit_cast(h16x2, w[i]);
      v[2 * i] = static_cast<float>(h.x);
      v[2 * i + 1] = static_cast<float>(h.y);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2 f = {v[2 * i], v[2 * i + 1]};
      w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, h16x2));
    }
    const u32x4 t = {w[0], w[1], w[2], w[3]};
    return t;
  }
  static __device__ __forceinline__ float load1(const f16_t* p) {
    return static_cast<float>(__builtin_bit_cast(_Float16, p->x));
  }
  static __device__ __forceinline__ void store1(f16_t* p, float v) {
    p->x = __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
  }
};

template <>
struct IO<bf16_t> {
  using Acc = float;
  static constexpr int kVec = 8;
  static __device__ __forceinline__ void unpack(const u32x4 t, float (&v)[8]) {
    const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2 f = {v[2 * i], v[2 * i + 1]};
      w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, b16x2));
    }
    const u32x4 t = {w[0], w[1], w[2], w[3]};
    return t;
  }
  static __device__ __forceinline__ float load1(const bf16_t* p) {
    return __builtin_bit_cast(float, static_cast<uint32_t>(p->x) << 16);
  }
  static __device__ __forceinline__ void store1(bf16_t* p, float v) {
    p->x = __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
  }
};

// The sample that shifted sums are taken relative to (sum(x - s), sum((x - s)^2):
// no cancellation against a large mean). A sample that is not finite would turn
// every difference into inf or nan, so zero takes its place: the plain sums then
// carry inf and nan into the mean and the variance as the CPU kernels' sums do.
template <typename A>
__device__ __forceinline__ A finite_or_zero(const A v) {
  return __builtin_isfinite(v) ? v : A(0);
}
template <typename T>
__device__ __forceinline__ typename IO<T>::Acc load_shift(const T* p) {
  return finite_or_zero(IO<T>::load1(p));
}

// One aligned 16-byte packet to and from HBM. Outputs are written once and not
// read again by the same kernel, so stores carry the non-temporal hint.
// Loads come in two flavours. `load_packet` is for a tensor that the kernel
// reads exactly once and that nothing re-reads soon (the fused single-read
// kernels, the last pass of a multi-pass structure): non-temporal. Measured on
// MI355X with inputs that are not in the 256 MB last-level cache, streaming
// kernels gain 5-10% from it (a read-only stream 7.1 TB/s against 6.3, two reads
// and a write 6.2 against 5.7; SoftmaxGrad [262144, 512] fp16 124 us against
// 134). The lines it fetches are not kept, so a kernel that is re-run on the
// same 100 MB finds nothing of it in the cache. `load_packet_keep` is the plain
// load for what is read again: the first pass of a two-pass structure, the
// statistics kernel that a normalisation pass follows, parameters.
typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), may_alias));
template <typename T>
__device__ __forceinline__ u32x4 load_packet(const T* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4_any*>(p));
}
template <typename T>
__device__ __forceinline__ u32x4 load_packet_keep(const T* p) {
  return *reinterpret_cast<const u32x4_any*>(p);
}
template <typename T>
__device__ __forceinline__ void store_packet(T* p, const u32x4 t) {
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4_any*>(p));
}
// The same packet at an address that is only element-aligned (rows whose byte
// length is not a multiple of 16): still one 128-bit access, the memory system
// splits it where it straddles a cache line.
typedef uint32_t u32x4_unaligned __attribute__((ext_vector_type(4), may_alias, aligned(2)));
template <typename T>
__device__ __forceinline__ u32x4 load_packet_unaligned(const T* p) {
  return *reinterpret_cast<const u32x4_unaligned*>(p);
}
template <typename T>
__device__ __forceinline__ void store_packet_unaligned(T* p, const u32x4 t) {
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4_unaligned*>(p));
}

template <typename T>
__device__ __forceinline__ void load_unpack(const T* p, typename IO<T>::Acc (&v)[IO<T>::kVec]) {
  IO<T>::unpack(load_packet(p), v);
}
template <typename T>
__device__ __forceinline__ void load_unpack_keep(const T* p, typename IO<T>::Acc (&v)[IO<T>::kVec]) {
  IO<T>::unpack(load_packet_keep(p), v);
}
template <typename T>
__device__ __forceinline__ void pack_store(T* p, const typename IO<T>::Acc (&v)[IO<T>::kVec]) {
  store_packet(p, IO<T>::pack(v));
}

// kVec consecutive accumulator-typed parameters (gamma, beta, ...), 16-byte
// aligned at p.
template <int kVec>
__device__ __forceinline__ void load_params(const float* p, float (&v)[kVec]) {
  static_assert(kVec % 4 == 0, "float parameters travel in packets of four");
#pragma unroll
  for (int i = 0; i < kVec / 4; ++i) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p + 4 * i);
    v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
  }
}
template <int kVec>
__device__ __forceinline__ void load_params(const double* p, double (&v)[kVec]) {
  static_assert(kVec == 2, "double parameters travel in packets of two");
  const f64x2 t = *reinterpret_cast<const f64x2*>(p);
  v[0] = t.x, v[1] = t.y;
}

// The same for parameters at an element-aligned address, of which only the
// first n (n <= kVec) exist: whole groups as one unaligned access, the rest
// element by element, absent ones as zero.
template <int kVec, typename A>
__device__ __forceinline__ void load_params_ragged(const A* p, int n, A (&v)[kVec]) {
  constexpr int kPer = 16 / sizeof(A);
  if (n >= kVec) {
#pragma unroll
    for (int i = 0; i < kVec / kPer; ++i) {
      const u32x4 t = load_packet_unaligned(p + kPer * i);
      A w[kPer];
      IO<A>::unpack(t, w);
#pragma unroll
      for (int e = 0; e < kPer; ++e) v[kPer * i + e] = w[e];
    }
  } else {
#pragma unroll
    for (int e = 0; e < kVec; ++e) v[e] = e < n ? p[e] : A(0);
  }
}

// ---------------------------------------------------------------------------
// Reductions
// ---------------------------------------------------------------------------
struct SumOp {
  template <typename A>
  __device__ __forceinline__ A operator()(A a, A b) const {
    return a + b;
  }
};
// The hardware maximum (one instruction; a compare-and-select costs two).
struct MaxOp {
  __device__ __forceinline__ float operator()(float a, float b) const {
    return __builtin_fmaxf(a, b);
  }
  __device__ __forceinline__ double operator()(double a, double b) const {
    return __builtin_fmax(a, b);
  }
};

// One data-parallel-primitive step: every lane combines its value with the
// value of the lane the DPP control selects (the cross-lane move happens in the
// VALU operand path, without the LDS crossbar a shuffle would use).
template <int kCtrl, typename Op>
__device__ __forceinline__ float dpp_step(float v, Op op) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, 0xf, 0xf, false);
  return op(v, __builtin_bit_cast(float, moved));
}

// All-reduce over the 64 lanes of a wavefront: every lane ends up with the
// result. fp32: four DPP steps reduce each row of 16 lanes (swap within pairs,
// swap pairs within quads, mirror within 8, mirror within 16), then the four
// row results are read into scalar registers and combined. fp64 uses the
// butterfly of shuffles.
template <typename Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
  v = dpp_step<0xB1>(v, op);   // quad_perm [1,0,3,2]
  v = dpp_step<0x4E>(v, op);   // quad_perm [2,3,0,1]
  v = dpp_step<0x141>(v, op);  // row_half_mirror
  v = dpp_step<0x140>(v, op);  // row_mirror
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  return op(op(r0, r1), op(r2, r3));
}
template <typename Op>
__device__ __forceinline__ double wave_allreduce(double v, Op op) {
#pragma unroll
  for (int o = kWaveSize / 2; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, kWaveSize));
  return v;
}

// All-reduce over a workgroup of kWaves wavefronts through kWaves LDS slots.
// `slots` must not be reused by another reduction before the next barrier.
template <int kWaves, typename A, typename Op>
__device__ __forceinline__ A block_allreduce(A v, Op op, A* slots) {
  v = wave_allreduce(v, op);
  if (kWaves == 1) return v;
  const int wave = threadIdx.x / kWaveSize;
  if ((threadIdx.x & (kWaveSize - 1)) == 0) slots[wave] = v;
  __syncthreads();
  A r = slots[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) r = op(r, slots[i]);
  return r;
}

// ---------------------------------------------------------------------------
// Scalar math in the accumulator type
// ---------------------------------------------------------------------------
__device__ __forceinline__ float acc_rsqrt_exact(float v) { return 1.0f / sqrtf(v); }
__device__ __forceinline__ double acc_rsqrt_exact(double v) { return 1.0 / sqrt(v); }
__device__ __forceinline__ float acc_exp(float v) { return expf(v); }
__device__ __forceinline__ double acc_exp(double v) { return exp(v); }
__device__ __forceinline__ float acc_log(float v) { return logf(v); }
__device__ __forceinline__ double acc_log(double v) { return log(v); }
template <typename A>
__device__ __forceinline__ A acc_neg_inf();
template <>
__device__ __forceinline__ float acc_neg_inf<float>() { return -__builtin_inff(); }
template <>
__device__ __forceinline__ double acc_neg_inf<double>() { return -__builtin_inf(); }

// ---------------------------------------------------------------------------
// Host-side helpers
// ---------------------------------------------------------------------------
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// The same offset from a 16-byte boundary: the aligned packets of one tensor line up with the other's.
inline bool congruent16(const void* a, const void* b) {
  return ((reinterpret_cast<uintptr_t>(a) ^ reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
}
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int status_of_launch() {
  if (plan_only()) {  // nothing was launched; a host without a device has nothing to report
    (void)hipGetLastError();
    return DRAGON_HIP_OK;
  }
  const hipError_t e = hipGetLastError();
  return e == hipSuccess ? DRAGON_HIP_OK : static_cast<int>(e);
}

// Runs FN<T>(args...) for the element type a dtype tag names.
#define DRAGON_HIP_DISPATCH_DTYPE(dtype, FN, ...)                       \
  switch (dtype) {                                                      \
    case DRAGON_HIP_F16: return FN<dragon_hip::f16_t>(__VA_ARGS__);     \
    case DRAGON_HIP_BF16: return FN<dragon_hip::bf16_t>(__VA_ARGS__);   \
    case DRAGON_HIP_F32: return FN<float>(__VA_ARGS__);                 \
    case DRAGON_HIP_F64: return FN<double>(__VA_ARGS__);                \
    default: return DRAGON_HIP_EDTYPE;                                  \
  }

} // namespace dragon_hip
