// Single-read reductions over units that do not fit one workgroup.
//
// A reduction unit (a BatchNorm channel of an NCHW tensor, a GroupNorm group)
// whose statistics must be complete before any of its elements can be written
// normally costs two passes over the input. Here a unit is cut into K slices;
// a 256-thread workgroup keeps its slice in registers as raw packets (up to 16
// per thread, 64 KB per slice), writes the slice's two partial sums into the
// unit's K pairs in HBM and waits until the unit's other K-1 slices have done
// the same. Every workgroup of the unit then forms the same totals from the K
// pairs in a fixed order and finishes its slice out of registers, so every
// tensor is read once.
//
// Work item w = u*K + k is taken by workgroup w % grid, and a workgroup walks
// its items in ascending order. All `grid` workgroups are resident at once
// (the grid is never larger than the occupancy query reports), so a workgroup
// that waits for the peers of its item waits for workgroups that are running:
// each of them holds a slice of the same unit or an item of an earlier unit,
// which by induction completes. The wait is bounded all the same (a thread
// that runs out of patience goes on with what it has read), so every wavefront
// reaches the end of the kernel whatever happens.
//
// A small kernel fills the pairs with the "unset" pattern before every launch.
//
// The arithmetic is a policy Op:
//   kIn                              tensors held (x; x and dy)
//   Merge                            how two partial pairs combine (PairSum, or the
//                                    Op's own merge / identity)
//   begin(u, base, in0)              per-item setup (base = first element of the unit)
//   accumulate(u, j, x, dy, a, b)    the terms of packet j of unit u in the two sums
//   finish(u, leader, a, b)          coefficients from the unit's totals; the thread
//                                    with `leader` set (one per unit) writes the
//                                    per-unit outputs
//   transform(u, j, x, dy)           overwrites x with the outputs of packet j
// A slice is a whole number of wavefronts of packets, and so is a unit whenever
// its packet count is a multiple of 64: accumulate / transform are then entered
// by whole wavefronts and may reduce across the wavefront.
#pragma once

#include <type_traits>

#include "reduce.h"
#include "row_tile.h"

namespace dragon_hip {

constexpr int kCoopThreads = 256;

// A wait that gave up is reported through one word of pinned host memory that
// the kernels write and the host reads without synchronising: the outputs of
// that launch are invalid, and every later single-read launch is refused with
// DRAGON_HIP_ETIMEOUT until the word is cleared. Allocated on first use (once
// per process; before any stream capture, like the cached launch plans).
struct ExchangeState {
  uint32_t* host_word = nullptr;
  uint32_t* device_word = nullptr;
  uint32_t patience = 0;  // 0: the default
};
inline ExchangeState& exchange_state() {
  static ExchangeState st = [] {
    ExchangeState e;
    void* p = nullptr;
    if (hipHostMalloc(&p, sizeof(uint32_t), hipHostMallocMapped | hipHostMallocPortable) ==
        hipSuccess) {
      e.host_word = static_cast<uint32_t*>(p);
      *e.host_word = 0u;
      void* dp = nullptr;
      if (hipHostGetDevicePointer(&dp, p, 0) == hipSuccess) e.device_word = static_cast<uint32_t*>(dp);
    }
    (void)hipGetLastError();
    return e;
  }();
  return st;
}
constexpr uint32_t kCoopPatience = 1u << 20;  // polls of about 1 us each (s_sleep 32 between them)

struct CoopPlan {
  bool ok;
  uint32_t K;      // slices per channel
  uint32_t slice;  // packets per slice
  int r;           // packets per thread and tensor
};

// kIn tensors are held at once (1 forward, 2 backward).
// Packets per thread and tensor, and the workgroups resident per compute unit
// at that size: 16 forward (128 registers, four workgroups), 12 + 12 backward
// (up to 168 registers, three workgroups). Measured at [64,256,56,56] fp32:
// smaller slices lose more to the per-item exchange than the extra residency
// gains (8 packets: 81 us forward against 61; 4 + 4: 166 us backward against 125).
inline int coop_rmax(int kIn) { return kIn == 1 ? 16 : 12; }
inline uint32_t coop_grid(int r, int kIn) { return r * kIn > 16 ? kNumCUs * 3 : kNumCUs * 4; }

// What is reduced: `units` reduction units (BatchNorm channels, GroupNorm
// groups), each `nseg` runs of `seglen` contiguous elements; run s of unit u
// starts at element u * unit_stride + s * seg_stride.
struct SliceUnits {
  uint32_t units, nseg, seglen, unit_stride, seg_stride;
};

template <typename T>
CoopPlan plan_coop(const SliceUnits& u, int kIn) {
  constexpr int kVec = IO<T>::kVec;
  CoopPlan p = {false, 0, 0, 0};
  if (u.seglen % kVec != 0) return p;
  const uint32_t pps = u.seglen / kVec;
  if (pps < 16) return p;  // runs shorter than 256 bytes: left to the split reduction
  const int64_t P = static_cast<int64_t>(u.nseg) * pps;  // packets per unit
  const int rmax = coop_rmax(kIn);
  const int64_t grid = coop_grid(rmax, kIn);
  const int64_t kmin = ceil_div(P, static_cast<int64_t>(rmax) * kCoopThreads);
  if (kmin > 1024) return p;
  // Slices of at least four packets per thread, unless the unit is smaller.
  int64_t kmax = P / (4 * kCoopThreads);
  if (kmax < kmin) kmax = kmin;
  if (kmax > 1024) kmax = 1024;
  if (kmax > kmin + 64) kmax = kmin + 64;
  // The K whose units*K items fill whole rounds of the resident grid best.
  int64_t best = kmin;
  double best_util = 0;
  for (int64_t k = kmin; k <= kmax; ++k) {
    const int64_t items = static_cast<int64_t>(u.units) * k;
    const double util = static_cast<double>(items) / (ceil_div(items, grid) * grid);
    if (util > best_util + 1e-9) best = k, best_util = util;
    if (util >= 0.96) break;
  }
  p.K = static_cast<uint32_t>(best);
  // whole wavefronts of packets per slice, so that a wavefront never straddles two slices
  p.slice = static_cast<uint32_t>(ceil_div(ceil_div(P, best), kWaveSize) * kWaveSize);
  p.r = static_cast<int>(ceil_div(p.slice, kCoopThreads));
  p.ok = p.r <= rmax;
  return p;
}

// Scratch of the single-read path for `units`: the larger of the one- and the two-tensor plan.
template <typename T>
size_t coop_scratch_bytes(const SliceUnits& u) {
  using A = typename IO<T>::Acc;
  size_t need = 0;
  for (int in = 1; in <= 2; ++in) {
    const CoopPlan p = plan_coop<T>(u, in);
    if (!p.ok) continue;
    const size_t bytes = static_cast<size_t>(u.units) * p.K * 2 * sizeof(A);
    if (bytes > need) need = bytes;
  }
  return need;
}

struct CoopShape {
  uint32_t unit_stride, K, slice;
  uint32_t pps;          // packets per run
  uint32_t P;            // packets per unit
  uint32_t seg_stride;   // elements between two runs of a unit
  uint32_t step_seg, step_p;  // kCoopThreads packets further on = step_seg segments and step_p packets
  uint32_t items;        // units * K
  uint32_t patience;     // polls of a slot before a thread gives up
  uint32_t* timed_out;   // set to 1 by a thread that gave up (may be null)
};

template <typename T>
CoopShape make_coop_shape(const SliceUnits& u, const CoopPlan& p) {
  constexpr int kVec = IO<T>::kVec;
  CoopShape d;
  d.unit_stride = u.unit_stride, d.K = p.K, d.slice = p.slice;
  d.pps = u.seglen / kVec;
  d.P = u.nseg * d.pps;
  d.seg_stride = u.seg_stride;
  d.step_seg = kCoopThreads / d.pps, d.step_p = kCoopThreads % d.pps;
  d.items = u.units * p.K;
  const ExchangeState& ex = exchange_state();
  d.patience = ex.patience ? ex.patience : kCoopPatience;
  d.timed_out = ex.device_word;
  return d;
}

// The packets of one slice that a thread owns: packet i of the thread is packet
// j0 + threadIdx.x + i * kCoopThreads of the channel.
struct CoopCursor {
  uint32_t seg, p;
  __device__ __forceinline__ CoopCursor(const CoopShape& d, uint32_t j0) {
    const uint32_t jp = j0 + threadIdx.x;
    seg = jp / d.pps;
    p = jp - seg * d.pps;
  }
  template <int kVec>
  __device__ __forceinline__ uint32_t offset(const CoopShape& d, uint32_t base) const {
    return base + seg * d.seg_stride + p * kVec;
  }
  __device__ __forceinline__ void advance(const CoopShape& d) {
    seg += d.step_seg;
    p += d.step_p;
    if (p >= d.pps) p -= d.pps, ++seg;
  }
};

// Bit pattern of a partial sum that has not been published yet (a NaN that no
// arithmetic here produces; the slots are filled with it before every launch).
template <typename A>
struct Unset;
template <>
struct Unset<float> {
  using Bits = uint32_t;
  static constexpr Bits kValue = 0xffffffffu;
};
template <>
struct Unset<double> {
  using Bits = unsigned long long;
  static constexpr Bits kValue = ~0ull;
};

template <typename Bits>
__global__ __launch_bounds__(256) void fill_words(Bits* p, uint32_t n, Bits value) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = value;
}

// Publishes this slice's pair, waits for the channel's K pairs and returns
// their sums (the same bits in every workgroup of the channel). The pairs are
// written and read with device-scope atomic accesses, which go past the
// per-XCD L2 caches without flushing or invalidating them; a slot is complete
// as soon as it no longer holds the unset pattern, so no counter or fence
// orders the exchange.
// How two partial pairs combine: sums (the default policy of an Op), or an
// Op's own associative, symmetric merge (with its identity), e.g. the running
// (maximum, scaled sum) of a softmax.
struct PairSum {
  static constexpr bool kIsSum = true;
  template <typename A>
  static __device__ __forceinline__ void identity(A& a, A& b) {
    a = A(0), b = A(0);
  }
  template <typename A>
  static __device__ __forceinline__ void merge(A& a, A& b, A a2, A b2) {
    a += a2, b += b2;
  }
};

// All-reduce of a pair over the workgroup with Merge; every thread returns the
// same bits (the per-wavefront results are merged in wavefront order).
template <typename Merge, typename A>
__device__ __forceinline__ void block_merge_pair(A& a, A& b, A* lds /*2*kReduceWaves*/) {
  if constexpr (Merge::kIsSum) {
    block_reduce_pair(a, b, lds);
  } else {
#pragma unroll
    for (int o = 1; o < kWaveSize; o <<= 1) {
      const A a2 = __shfl_xor(a, o, kWaveSize), b2 = __shfl_xor(b, o, kWaveSize);
      Merge::merge(a, b, a2, b2);
    }
    const int wave = threadIdx.x / kWaveSize;
    if ((threadIdx.x & (kWaveSize - 1)) == 0) {
      lds[2 * wave] = a;
      lds[2 * wave + 1] = b;
    }
    __syncthreads();
    a = lds[0], b = lds[1];
#pragma unroll
    for (int i = 1; i < kReduceWaves; ++i) Merge::merge(a, b, lds[2 * i], lds[2 * i + 1]);
  }
}

template <typename Merge, typename A>
__device__ __forceinline__ void coop_channel_totals(const CoopShape& d, uint32_t c, uint32_t w,
                                                    A& a, A& b, A* partial, A* lds_a, A* lds_b) {
  using Bits = typename Unset<A>::Bits;
  block_merge_pair<Merge>(a, b, lds_a);
  Bits* slots = reinterpret_cast<Bits*>(partial);
  if (threadIdx.x == 0) {
    __hip_atomic_store(slots + 2 * static_cast<size_t>(w), __builtin_bit_cast(Bits, a),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(slots + 2 * static_cast<size_t>(w) + 1, __builtin_bit_cast(Bits, b),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  A ta, tb;
  Merge::identity(ta, tb);
  const Bits* pairs = slots + 2 * static_cast<size_t>(c) * d.K;
  for (uint32_t q = threadIdx.x; q < d.K; q += kCoopThreads) {
    Bits ua, ub;
    uint32_t patience = d.patience;
    for (;;) {
      ua = __hip_atomic_load(pairs + 2 * q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ub = __hip_atomic_load(pairs + 2 * q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (ua != Unset<A>::kValue && ub != Unset<A>::kValue) break;
      if (--patience == 0) {
        if (d.timed_out) {
          __hip_atomic_store(d.timed_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        break;
      }
      __builtin_amdgcn_s_sleep(32);
    }
    Merge::merge(ta, tb, __builtin_bit_cast(A, ua), __builtin_bit_cast(A, ub));
  }
  block_merge_pair<Merge>(ta, tb, lds_b);
  a = ta, b = tb;
}

// Optional parts of an Op, both off unless it declares them:
//   kScanFirst  op.scan(x) sees every packet of the item before the first
//               accumulate (a thread-wide maximum, say);
//   kRewrites   op.accumulate_rewrite(x, a, b) replaces the elements it is
//               given, and the second pass reads those instead of the input
//               (exact only where a packet holds accumulator-typed elements).
template <typename Op, typename = void>
struct OpScansFirst : std::false_type {};
template <typename Op>
struct OpScansFirst<Op, std::void_t<decltype(Op::kScanFirst)>> : std::bool_constant<Op::kScanFirst> {};
template <typename Op, typename = void>
struct OpRewrites : std::false_type {};
template <typename Op>
struct OpRewrites<Op, std::void_t<decltype(Op::kRewrites)>> : std::bool_constant<Op::kRewrites> {};

template <typename T, int kR, int kIn>
struct CoopSlice {  // the raw packets of one item
  u32x4 p0[kR];
  u32x4 p1[kIn == 2 ? kR : 1];
};

struct CoopItem {
  uint32_t c, k, j0, len, base;
  __device__ __forceinline__ CoopItem(const CoopShape& d, uint32_t w) {
    c = w / d.K;
    k = w - c * d.K;
    j0 = k * d.slice;
    const uint32_t j1 = j0 + d.slice < d.P ? j0 + d.slice : d.P;
    len = j1 > j0 ? j1 - j0 : 0u;
    base = c * d.unit_stride;
  }
  __device__ __forceinline__ bool has(int i) const { return i * kCoopThreads + threadIdx.x < len; }
};

template <typename T, int kR, int kIn>
__device__ __forceinline__ void coop_load(const CoopShape& d, uint32_t w, const T* in0, const T* in1,
                                          CoopSlice<T, kR, kIn>& s) {
  constexpr int kVec = IO<T>::kVec;
  const CoopItem it(d, w);
  CoopCursor cur(d, it.j0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const uint32_t off = it.has(i) ? cur.template offset<kVec>(d, it.base) : it.base;
    s.p0[i] = load_packet(in0 + off);
    if constexpr (kIn == 2) s.p1[i] = load_packet(in1 + off);
    cur.advance(d);
  }
}

// `next` is the item this workgroup takes after w (>= d.items: none): its
// packets are requested one by one into the registers the second pass has just
// written out, so they travel while the rest of this item is stored.
template <typename T, int kR, typename Op>
__device__ __forceinline__ void coop_process(const CoopShape& d, uint32_t w, uint32_t next,
                                             const T* in0, const T* in1, T* out, Op op,
                                             CoopSlice<T, kR, Op::kIn>& s,
                                             typename IO<T>::Acc* partial,
                                             typename IO<T>::Acc* lds_a,
                                             typename IO<T>::Acc* lds_b) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const CoopItem it(d, w);
  op.begin(it.c, it.base, in0);
  A a, b;
  Op::Merge::identity(a, b);
  if constexpr (OpScansFirst<Op>::value) {
#pragma unroll
    for (int i = 0; i < kR; ++i) {
      if (it.has(i)) {
        A xv[kVec];
        IO<T>::unpack(s.p0[i], xv);
        op.scan(xv);
      }
    }
    // convert the packets again instead of keeping every converted element
#pragma unroll
    for (int i = 0; i < kR; ++i) asm volatile("" : "+v"(s.p0[i]));
  }
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    if (it.has(i)) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
      if constexpr (OpRewrites<Op>::value) {
        static_assert(sizeof(T) == sizeof(A), "rewritten elements must survive the packet");
        op.accumulate_rewrite(xv, a, b);
        s.p0[i] = IO<T>::pack(xv);
      } else {
        op.accumulate(it.c, it.j0 + i * kCoopThreads + threadIdx.x, xv, dv, a, b);
      }
    }
  }
  coop_channel_totals<typename Op::Merge>(d, it.c, w, a, b, partial, lds_a, lds_b);
  op.finish(it.c, it.k == 0 && threadIdx.x == 0, a, b);
  // convert the packets again instead of keeping every converted element
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    asm volatile("" : "+v"(s.p0[i]));
    if constexpr (Op::kIn == 2) asm volatile("" : "+v"(s.p1[i]));
  }
  const bool more = next < d.items;  // uniform over the workgroup
  const CoopItem nit(d, more ? next : w);
  CoopCursor cur(d, it.j0), ncur(d, nit.j0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    if (it.has(i)) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
      op.transform(it.c, it.j0 + i * kCoopThreads + threadIdx.x, xv, dv);
      store_packet(out + cur.template offset<kVec>(d, it.base), IO<T>::pack(xv));
    }
    cur.advance(d);
    if (more) {
      const uint32_t off = nit.has(i) ? ncur.template offset<kVec>(d, nit.base) : nit.base;
      s.p0[i] = load_packet(in0 + off);
      if constexpr (Op::kIn == 2) s.p1[i] = load_packet(in1 + off);
      ncur.advance(d);
    }
  }
}

// One item at a time per workgroup, as large as the registers allow: the
// exchange costs a few microseconds per item whatever its size. Four
// workgroups per compute unit, or three with up to 168 registers for the
// widest slices.
template <typename T, int kR, typename Op>
__global__ __launch_bounds__(kCoopThreads, kR * Op::kIn > 16 ? 3 : 4) void channel_slices(
    const CoopShape d, const T* __restrict__ in0, const T* __restrict__ in1, T* __restrict__ out,
    const Op op, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds_a[2 * kReduceWaves];
  __shared__ A lds_b[2 * kReduceWaves];
  CoopSlice<T, kR, Op::kIn> s;
  if (blockIdx.x < d.items) coop_load<T, kR, Op::kIn>(d, blockIdx.x, in0, in1, s);
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    coop_process<T, kR, Op>(d, w, w + gridDim.x, in0, in1, out, op, s, partial, lds_a, lds_b);
  }
}

template <typename A>
inline void fill_unset(A* pairs, const CoopShape& d, hipStream_t stream) {
  using Bits = typename Unset<A>::Bits;
  const uint32_t n = d.items * 2;
  hipLaunchKernelGGL((fill_words<Bits>), dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0,
                     stream, reinterpret_cast<Bits*>(pairs), n, Unset<A>::kValue);
}

// DRAGON_HIP_OK when the single-read kernel was launched, kNotApplicable when
// the shape or alignment leaves the call to the split path, or an error.
constexpr int kNotApplicable = 1;
template <typename T, typename Op>
int try_channel_slices(const SliceUnits& sh, const Op& op, const T* in0, const T* in1, T* out,
                       typename IO<T>::Acc* scratch, hipStream_t stream) {
  const CoopPlan p = plan_coop<T>(sh, Op::kIn);
  if (!p.ok || !aligned16(in0) || !aligned16(in1) || !aligned16(out)) return kNotApplicable;
  const ExchangeState& ex = exchange_state();
  if (ex.host_word && *static_cast<volatile uint32_t*>(ex.host_word) != 0u) {
    return DRAGON_HIP_ETIMEOUT;
  }
  const CoopShape d = make_coop_shape<T>(sh, p);
  fill_unset(scratch, d, stream);
#define LAUNCH(R)                                                                              \
  {                                                                                            \
    auto kernel = channel_slices<T, R, Op>;                                                    \
    const unsigned resident = resident_grid(kernel, kCoopThreads, 0);                          \
    const unsigned want = coop_grid(coop_rmax(Op::kIn), Op::kIn);                              \
    const unsigned cap = resident < want ? resident : want;                                    \
    hipLaunchKernelGGL(kernel, dim3(d.items < cap ? d.items : cap), dim3(kCoopThreads), 0,     \
                       stream, d, in0, in1, out, op, scratch);                                 \
  }
  constexpr int kIn = Op::kIn;
  if (p.r * kIn <= 4) LAUNCH(4 / kIn)
  else if (p.r * kIn <= 8) LAUNCH(8 / kIn)
  else if (p.r * kIn <= 16) LAUNCH(16 / kIn)
  else if constexpr (kIn == 2) LAUNCH(12)  // one tensor: never more than 16 packets
#undef LAUNCH
  return status_of_launch();
}


} // namespace dragon_hip
