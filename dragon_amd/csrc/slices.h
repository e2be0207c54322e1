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
// (the grid is never larger than the occupancy query reports) and a unit never
// has more slices than the grid has workgroups, so the K items of a unit are
// held by K different workgroups, each of which is at that item or at an item
// of an earlier unit, which by induction completes: a workgroup that waits for
// the peers of its item waits for workgroups that are running.
//
// The wait is bounded all the same (other work on the device can keep part of
// the grid from becoming resident, e.g. a second such kernel on another
// stream). A workgroup whose wait runs out leaves its item alone: it writes no
// output for it, the unit's leader writes no per-unit output, and the item is
// flagged in the launch's own scratch. A second launch of the same code
// (`channel_slices_repair`, enqueued right behind the first) ends at once when
// nothing is flagged; otherwise it finishes every flagged item. By then every
// slice of every unit has published its pair (a workgroup publishes before it
// waits), so the repair needs no waiting and forms the same totals, bit for
// bit, as the workgroups that did not give up. The outputs of a call are
// therefore always complete in stream order, in place or not.
//
// A small kernel fills the pairs with the "unset" pattern and clears the flags
// before every launch. Units of a single slice (K = 1) exchange nothing: the
// workgroup's own pair is the unit's, and neither the fill nor the repair is
// launched.
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
//
// Runs that are not whole aligned packets (a 57x57 or 15x15 feature map, a
// tensor at an element-aligned address) go through the same kernel in its
// window flavour, for an Op that declares kWindows: a run of seglen elements is
// read as the aligned 16-byte packets that cover it, seglen / kVec + 2 packet
// slots of which the last may lie behind the run and is skipped. A packet
// wholly inside the run is accumulated, transformed and stored as a packet; of
// a packet at either end only the run's own elements count (the others are
// replaced by the Op's neutral element before they are accumulated) and are
// stored (one element store each), the neighbouring run's elements in it
// belonging to another unit and another workgroup. All
// tensors of a call must then be congruent modulo 16 bytes. An aligned packet
// that holds a byte of a tensor lies in that byte's page, so a packet that
// reaches beyond either end of a tensor may be read whole.
#pragma once

#include <type_traits>

#include "reduce.h"
#include "row_tile.h"

namespace dragon_hip {

constexpr int kCoopThreads = 256;

// Process-wide settings and diagnostics of the exchange (defined in
// context.hip). `exchange_patience` is how many polls of a slot a thread makes
// before it gives up (0: the default). `exchange_gave_up_counter` is the address,
// on the current device, of a word that counts the items whose wait ran out
// (a diagnostic: such items are repaired, see above); null when it cannot be
// resolved. Neither allocates.
uint32_t exchange_patience();
uint32_t* exchange_gave_up_counter();
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
inline uint32_t coop_grid(int r, int kIn) {
  return static_cast<uint32_t>(r * kIn > 16 ? num_cus() * 3 : num_cus() * 4);
}

// What is reduced: `units` reduction units (BatchNorm channels, GroupNorm
// groups), each `nseg` runs of `seglen` contiguous elements; run s of unit u
// starts at element u * unit_stride + s * seg_stride.
struct SliceUnits {
  uint32_t units, nseg, seglen, unit_stride, seg_stride;
};

template <typename T>
CoopPlan plan_coop(const SliceUnits& u, int kIn, bool windows = false) {
  constexpr int kVec = IO<T>::kVec;
  CoopPlan p = {false, 0, 0, 0};
  if (!windows && u.seglen % kVec != 0) return p;
  // Runs shorter than 256 bytes are left to the split reduction, and so are window
  // runs under 384 bytes: two of their packets are stored element by element,
  // and the gathered 200-byte runs of a channel use their cache lines worse than
  // the split path's contiguous rows (7x7 fp32 maps, single-slice channels, which
  // need no exchange: 49 us against 33; 9x9: 15 against 23 the other way).
  if (u.seglen / kVec < (windows ? 24u : 16u)) return p;
  const uint32_t pps = u.seglen / kVec + (windows ? 2 : 0);
  const int64_t P = static_cast<int64_t>(u.nseg) * pps;  // packets per unit
  const int rmax = coop_rmax(kIn);
  const int64_t grid = coop_grid(rmax, kIn);
  const int64_t kmin = ceil_div(P, static_cast<int64_t>(rmax) * kCoopThreads);
  // The K slices of a unit must be held by K different workgroups (see the
  // head of this file): never more slices than the grid has workgroups.
  const int64_t klimit = grid < 1024 ? grid : 1024;
  if (kmin > klimit) return p;
  // Slices of at least four packets per thread, unless the unit is smaller.
  int64_t kmax = P / (4 * kCoopThreads);
  if (kmax < kmin) kmax = kmin;
  if (kmax > klimit) kmax = klimit;
  if (kmax > kmin + 64) kmax = kmin + 64;
  // The K with the least estimated time: the resident grid works through units*K items in
  // rounds, and a round costs its slice (packets per workgroup) plus the exchange, which is
  // worth about 800 packets of streaming (4 us at a workgroup's share of the bandwidth).
  // More, smaller slices fill the last round better but pay the exchange more often
  // (GroupNorm bf16 [55,384,56,56] in 16 groups: 8 slices 75 us, 3 slices 60 us).
  constexpr int64_t kExchangePackets = 800;
  int64_t best = kmin, best_cost = INT64_MAX;
  for (int64_t k = kmin; k <= kmax; ++k) {
    const int64_t items = static_cast<int64_t>(u.units) * k;
    const int64_t cost = ceil_div(items, grid) * (kExchangePackets + ceil_div(P, k));
    if (cost < best_cost) best = k, best_cost = cost;
  }
  p.K = static_cast<uint32_t>(best);
  // whole wavefronts of packets per slice, so that a wavefront never straddles two slices
  p.slice = static_cast<uint32_t>(ceil_div(ceil_div(P, best), kWaveSize) * kWaveSize);
  p.r = static_cast<int>(ceil_div(p.slice, kCoopThreads));
  p.ok = p.r <= rmax;
  return p;
}

// Scratch of one launch over `items` work items: the pairs, then one flag word
// per item (set when the item's wait ran out) and one for the launch as a whole;
// a multiple of 256 bytes, so that whatever a caller places behind it stays aligned.
inline size_t coop_exchange_bytes(size_t items, size_t acc_size) {
  const size_t bytes = items * 2 * acc_size + (items + 1) * sizeof(uint32_t);
  return (bytes + 255) / 256 * 256;
}

// Scratch of the single-read path for `units`: the larger of the one- and the
// two-tensor plan (`windows_too`: and of their window flavours, which the
// addresses of a call may select).
template <typename T>
size_t coop_scratch_bytes(const SliceUnits& u, bool windows_too = false) {
  using A = typename IO<T>::Acc;
  size_t need = 0;
  for (int in = 1; in <= 2; ++in) {
    for (int win = 0; win <= (windows_too ? 1 : 0); ++win) {
      const CoopPlan p = plan_coop<T>(u, in, win != 0);
      if (!p.ok) continue;
      const size_t bytes = coop_exchange_bytes(static_cast<size_t>(u.units) * p.K, sizeof(A));
      if (bytes > need) need = bytes;
    }
  }
  return need;
}

struct CoopShape {
  uint32_t unit_stride, K, slice;
  uint32_t pps;          // packets (window flavour: packet slots) per run
  uint32_t seglen;       // elements per run
  uint32_t P;            // packets per unit
  uint32_t seg_stride;   // elements between two runs of a unit
  uint32_t step_seg, step_p;  // a workgroup's threads further on = step_seg segments and step_p packets
  uint32_t items;        // units * K
  uint32_t patience;     // polls of a slot before a thread gives up
  uint32_t* flags;       // flags[w] = 1: item w gave up; flags[items] = 1: some item did
  uint32_t* gave_up_count;  // device-wide count of such items (a diagnostic; may be null)
};

template <typename T>
CoopShape make_coop_shape(const SliceUnits& u, const CoopPlan& p, typename IO<T>::Acc* scratch,
                          bool windows = false, uint32_t threads = kCoopThreads) {
  constexpr int kVec = IO<T>::kVec;
  CoopShape d;
  d.unit_stride = u.unit_stride, d.K = p.K, d.slice = p.slice;
  d.pps = u.seglen / kVec + (windows ? 2 : 0);
  d.seglen = u.seglen;
  d.P = u.nseg * d.pps;
  d.seg_stride = u.seg_stride;
  d.step_seg = threads / d.pps, d.step_p = threads % d.pps;
  d.items = u.units * p.K;
  const uint32_t patience = exchange_patience();
  d.patience = patience ? patience : kCoopPatience;
  d.flags = reinterpret_cast<uint32_t*>(scratch + static_cast<size_t>(d.items) * 2);
  d.gave_up_count = exchange_gave_up_counter();
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

// Where the cursor's packet lies, as an element offset from the tensors' bases
// (window flavour: below zero for the packet that holds the tensor's first
// elements at an unaligned base), and which of its elements [lo, hi) belong to
// the run; hi <= lo for the slot behind a run, whose packet is not touched.
struct CoopSlot {
  int32_t off;
  int lo, hi;
  template <int kVec>
  __device__ __forceinline__ bool whole() const { return lo == 0 && hi == kVec; }
};
template <typename T, bool kWin>
__device__ __forceinline__ CoopSlot coop_slot(const CoopShape& d, const CoopCursor& cur,
                                              uint32_t base, const T* in0) {
  constexpr int kVec = IO<T>::kVec;
  const uint32_t run = base + cur.seg * d.seg_stride;
  CoopSlot s;
  if constexpr (!kWin) {
    s.off = static_cast<int32_t>(run + cur.p * kVec), s.lo = 0, s.hi = kVec;
  } else {
    const int lead = static_cast<int>((reinterpret_cast<uintptr_t>(in0 + run) & 15u) / sizeof(T));
    const int pe = static_cast<int>(cur.p * kVec) - lead;  // the packet's first element, in the run
    const int rest = static_cast<int>(d.seglen) - pe;
    s.off = static_cast<int32_t>(run) + pe;
    s.lo = pe < 0 ? -pe : 0;
    s.hi = rest < kVec ? rest : kVec;
  }
  return s;
}
// An aligned packet that may always be read: the one that holds the unit's first element.
template <typename T, bool kWin>
__device__ __forceinline__ int32_t coop_safe_offset(uint32_t base, const T* in0) {
  if constexpr (!kWin) return static_cast<int32_t>(base);
  return static_cast<int32_t>(base) -
      static_cast<int32_t>((reinterpret_cast<uintptr_t>(in0 + base) & 15u) / sizeof(T));
}
// Keeps the compiler from carrying every slot of one pass over an item to the
// next pass in registers: the slots are recomputed from the cursor instead.
__device__ __forceinline__ void coop_forget(CoopCursor& cur) {
  asm volatile("" : "+v"(cur.seg), "+v"(cur.p));
}

// Bit pattern of a partial sum that has not been published yet; the slots are
// filled with it before every launch. It is a NaN, and the hardware carries the
// payload of an input NaN into a sum, so a partial that is any NaN is published
// as the canonical quiet NaN instead: no published value equals the pattern.
template <typename A>
struct Unset;
template <>
struct Unset<float> {
  using Bits = uint32_t;
  static constexpr Bits kValue = 0xffffffffu;
  static constexpr Bits kQuietNaN = 0x7fc00000u;
};
template <>
struct Unset<double> {
  using Bits = unsigned long long;
  static constexpr Bits kValue = ~0ull;
  static constexpr Bits kQuietNaN = 0x7ff8000000000000ull;
};
template <typename A>
__device__ __forceinline__ typename Unset<A>::Bits publishable_bits(const A v) {
  return v != v ? Unset<A>::kQuietNaN : __builtin_bit_cast(typename Unset<A>::Bits, v);
}

// Before a launch: the n pair words take the unset pattern, the nflags flag words zero.
template <typename Bits>
__global__ __launch_bounds__(256) void fill_exchange(Bits* p, uint32_t n, Bits value,
                                                     uint32_t* flags, uint32_t nflags) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = value;
  if (i < nflags) flags[i] = 0u;
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
template <typename Merge, int kWaves = kReduceWaves, typename A>
__device__ __forceinline__ void block_merge_pair(A& a, A& b, A* lds /*2*kWaves*/) {
  if constexpr (Merge::kIsSum && kWaves == kReduceWaves) {
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
    for (int i = 1; i < kWaves; ++i) Merge::merge(a, b, lds[2 * i], lds[2 * i + 1]);
  }
}

// Returns false when a wait ran out (the same answer in every thread of the
// workgroup): a and b are then meaningless and the item has been flagged.
// kRepair: the second launch; every pair has been published, nothing is
// published or waited for.
template <typename Merge, bool kRepair, typename A>
__device__ __forceinline__ bool coop_channel_totals(const CoopShape& d, uint32_t c, uint32_t w,
                                                    A& a, A& b, A* partial, A* lds_a, A* lds_b) {
  using Bits = typename Unset<A>::Bits;
  Bits* slots = reinterpret_cast<Bits*>(partial);
  if constexpr (!kRepair) {
    block_merge_pair<Merge>(a, b, lds_a);
    if (threadIdx.x == 0) {
      __hip_atomic_store(slots + 2 * static_cast<size_t>(w), publishable_bits(a), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slots + 2 * static_cast<size_t>(w) + 1, publishable_bits(b),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  A ta, tb;
  Merge::identity(ta, tb);
  int gave_up = 0;
  const Bits* pairs = slots + 2 * static_cast<size_t>(c) * d.K;
  for (uint32_t q = threadIdx.x; q < d.K; q += kCoopThreads) {
    Bits ua, ub;
    uint32_t patience = kRepair ? 1u : d.patience;
    for (;;) {
      ua = __hip_atomic_load(pairs + 2 * q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ub = __hip_atomic_load(pairs + 2 * q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (ua != Unset<A>::kValue && ub != Unset<A>::kValue) break;
      if (--patience == 0) {
        gave_up = 1;
        break;
      }
      __builtin_amdgcn_s_sleep(32);
    }
    Merge::merge(ta, tb, __builtin_bit_cast(A, ua), __builtin_bit_cast(A, ub));
  }
  if constexpr (!kRepair) {
    if (__syncthreads_or(gave_up)) {
      if (threadIdx.x == 0) {
        __hip_atomic_store(d.flags + w, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(d.flags + d.items, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d.gave_up_count) {
          __hip_atomic_fetch_add(d.gave_up_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      return false;
    }
  }
  block_merge_pair<Merge>(ta, tb, lds_b);
  a = ta, b = tb;
  return true;
}

// Optional parts of an Op, both off unless it declares them:
//   kScanFirst  op.scan(x) sees every packet of the item before the first
//               accumulate (a thread-wide maximum, say);
//   kRewrites   op.accumulate_rewrite(x, a, b) replaces the elements it is
//               given, and the second pass reads those instead of the input
//               (exact only where a packet holds accumulator-typed elements);
template <typename Op, typename = void>
struct OpScansFirst : std::false_type {};
template <typename Op>
struct OpScansFirst<Op, std::void_t<decltype(Op::kScanFirst)>> : std::bool_constant<Op::kScanFirst> {};
template <typename Op, typename = void>
struct OpRewrites : std::false_type {};
template <typename Op>
struct OpRewrites<Op, std::void_t<decltype(Op::kRewrites)>> : std::bool_constant<Op::kRewrites> {};
//   kBeginReadsInput  op.begin reads elements of the unit from memory (the sample
//               a shifted sum is taken relative to). A repaired item must see
//               the value the first launch saw, so such an Op is kept off
//               calls whose output overwrites that input.
template <typename Op, typename = void>
struct OpBeginReadsInput : std::false_type {};
template <typename Op>
struct OpBeginReadsInput<Op, std::void_t<decltype(Op::kBeginReadsInput)>>
    : std::bool_constant<Op::kBeginReadsInput> {};

//   kWindows    the Op's accumulate and transform do not depend on the packet
//               index j, and op.neutral(x, dy) replaces an element by one that
//               adds nothing to its sums: the window flavour may serve it.
template <typename Op, typename = void>
struct OpTakesWindows : std::false_type {};
template <typename Op>
struct OpTakesWindows<Op, std::void_t<decltype(Op::kWindows)>> : std::bool_constant<Op::kWindows> {};

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
  template <int kThreads = kCoopThreads>
  __device__ __forceinline__ bool has(int i) const { return i * kThreads + threadIdx.x < len; }
};

template <typename T, int kR, int kIn, bool kWin, int kThreads = kCoopThreads>
__device__ __forceinline__ void coop_load(const CoopShape& d, uint32_t w, const T* in0, const T* in1,
                                          CoopSlice<T, kR, kIn>& s) {
  const CoopItem it(d, w);
  CoopCursor cur(d, it.j0);
  const int32_t safe = coop_safe_offset<T, kWin>(it.base, in0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const CoopSlot at = coop_slot<T, kWin>(d, cur, it.base, in0);
    const int32_t off = it.template has<kThreads>(i) && at.hi > at.lo ? at.off : safe;
    s.p0[i] = load_packet(in0 + off);
    if constexpr (kIn == 2) s.p1[i] = load_packet(in1 + off);
    cur.advance(d);
  }
}

// `next` is the item this workgroup takes after w (>= d.items: none): its
// packets are requested one by one into the registers the second pass has just
// written out, so they travel while the rest of this item is stored.
// kRepair: the second launch, which finishes the items whose wait ran out.
template <typename T, int kR, typename Op, bool kRepair, bool kWin, int kThreads = kCoopThreads>
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
  static_assert(!kWin || (!OpScansFirst<Op>::value && !OpRewrites<Op>::value),
                "the window flavour serves plain accumulate / transform Ops");
  if constexpr (OpScansFirst<Op>::value) {
#pragma unroll
    for (int i = 0; i < kR; ++i) {
      if (it.template has<kThreads>(i)) {
        A xv[kVec];
        IO<T>::unpack(s.p0[i], xv);
        op.scan(xv);
      }
    }
    // convert the packets again instead of keeping every converted element
#pragma unroll
    for (int i = 0; i < kR; ++i) asm volatile("" : "+v"(s.p0[i]));
  }
  CoopCursor acur(d, it.j0);
  if constexpr (kWin) coop_forget(acur);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const CoopSlot at = coop_slot<T, kWin>(d, acur, it.base, in0);
    if (it.template has<kThreads>(i) && at.hi > at.lo) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
      if constexpr (OpRewrites<Op>::value) {
        static_assert(sizeof(T) == sizeof(A), "rewritten elements must survive the packet");
        op.accumulate_rewrite(xv, a, b);
        s.p0[i] = IO<T>::pack(xv);
      } else {
        if constexpr (kWin) {
          // what the packet holds of the neighbouring runs is replaced by values
          // that add nothing to the Op's sums (no branch: short runs have such a
          // packet in every wavefront)
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (e < at.lo || e >= at.hi) op.neutral(xv[e], dv[e]);
          }
        }
        op.accumulate(it.c, it.j0 + i * kThreads + threadIdx.x, xv, dv, a, b);
      }
    }
    if constexpr (kWin) acur.advance(d);
  }
  // false (for the whole workgroup): the wait ran out, the item is left to the repair launch
  bool complete = true;
  if (d.K == 1) {
    // a unit in one slice: its totals are this workgroup's own, nothing is
    // exchanged (the host launches neither the fill nor the repair). Items take
    // the two LDS buffers by turns: the barrier of one item's reduction lies
    // between another's reads and writes of the same buffer.
    block_merge_pair<typename Op::Merge, kThreads / kWaveSize>(a, b, ((w / gridDim.x) & 1u) ? lds_b : lds_a);
  } else if constexpr (kThreads == kCoopThreads) {
    complete = coop_channel_totals<typename Op::Merge, kRepair>(d, it.c, w, a, b, partial, lds_a,
                                                                lds_b);
  }
  if (complete) op.finish(it.c, it.k == 0 && threadIdx.x == 0, a, b);
  // convert the packets again instead of keeping every converted element
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    asm volatile("" : "+v"(s.p0[i]));
    if constexpr (Op::kIn == 2) asm volatile("" : "+v"(s.p1[i]));
  }
  const bool more = !kRepair && next < d.items;  // uniform over the workgroup
  const CoopItem nit(d, more ? next : w);
  CoopCursor cur(d, it.j0), ncur(d, nit.j0);
  if constexpr (kWin) coop_forget(cur), coop_forget(ncur);
  const int32_t nsafe = coop_safe_offset<T, kWin>(nit.base, in0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const CoopSlot at = coop_slot<T, kWin>(d, cur, it.base, in0);
    if (complete && it.template has<kThreads>(i) && at.hi > at.lo) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
      op.transform(it.c, it.j0 + i * kThreads + threadIdx.x, xv, dv);
      if (!kWin || at.template whole<kVec>()) {
        store_packet(out + at.off, IO<T>::pack(xv));
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (e >= at.lo && e < at.hi) IO<T>::store1(out + at.off + e, xv[e]);
        }
      }
    }
    cur.advance(d);
    if (more) {
      const CoopSlot nat = coop_slot<T, kWin>(d, ncur, nit.base, in0);
      const int32_t off = nit.template has<kThreads>(i) && nat.hi > nat.lo ? nat.off : nsafe;
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
template <typename T, int kR, typename Op, bool kWin>
__global__ __launch_bounds__(kCoopThreads, kR * Op::kIn > 16 ? 3 : 4) void channel_slices(
    const CoopShape d, const T* __restrict__ in0, const T* __restrict__ in1, T* __restrict__ out,
    const Op op, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds_a[2 * kReduceWaves];
  __shared__ A lds_b[2 * kReduceWaves];
  CoopSlice<T, kR, Op::kIn> s;
  if (blockIdx.x < d.items) coop_load<T, kR, Op::kIn, kWin>(d, blockIdx.x, in0, in1, s);
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    coop_process<T, kR, Op, false, kWin>(d, w, w + gridDim.x, in0, in1, out, op, s, partial, lds_a,
                                         lds_b);
  }
}

// The launch behind it: nothing to do unless a wait of the first launch ran
// out; then every flagged item is finished from the pairs, which by now are all
// published. Inputs of a flagged item are intact even when the call runs in
// place: the workgroup that gave up wrote nothing for it.
template <typename T, int kR, typename Op, bool kWin>
__global__ __launch_bounds__(kCoopThreads, kR * Op::kIn > 16 ? 3 : 4) void channel_slices_repair(
    const CoopShape d, const T* __restrict__ in0, const T* __restrict__ in1, T* __restrict__ out,
    const Op op, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds_a[2 * kReduceWaves];
  __shared__ A lds_b[2 * kReduceWaves];
  if (d.flags[d.items] == 0u) return;
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    if (d.flags[w] == 0u) continue;  // the same word in every thread
    CoopSlice<T, kR, Op::kIn> s;
    coop_load<T, kR, Op::kIn, kWin>(d, w, in0, in1, s);
    coop_process<T, kR, Op, true, kWin>(d, w, d.items, in0, in1, out, op, s, partial, lds_a,
                                        lds_b);
    __syncthreads();  // the next item reuses the LDS words of the reductions
  }
}

// What a launcher returns when the shape or the addresses leave the call to another path.
constexpr int kNotApplicable = 1;

// Units that a workgroup of 512 or 1024 threads holds whole (K = 1: nothing is exchanged, and
// nothing waits, so the workgroups need not be resident together: one per unit, handed out by
// the hardware as workgroups finish). Two or one per compute unit at 128 registers.
template <typename T, int kR, int kThreads, typename Op, bool kWin>
__global__ __launch_bounds__(kThreads, 4) void channel_whole(
    const CoopShape d, const T* __restrict__ in0, const T* __restrict__ in1, T* __restrict__ out,
    const Op op) {
  using A = typename IO<T>::Acc;
  __shared__ A lds_a[2 * (kThreads / kWaveSize)];
  __shared__ A lds_b[2 * (kThreads / kWaveSize)];
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    CoopSlice<T, kR, Op::kIn> s;
    coop_load<T, kR, Op::kIn, kWin, kThreads>(d, w, in0, in1, s);
    coop_process<T, kR, Op, false, kWin, kThreads>(d, w, d.items, in0, in1, out, op, s, nullptr,
                                                   lds_a, lds_b);
  }
}

// Whether an Op's units may take channel_whole (BatchNorm's: plain accumulate / transform).
template <typename Op, typename = void>
struct OpTakesWholeUnits : std::false_type {};
template <typename Op>
struct OpTakesWholeUnits<Op, std::void_t<decltype(Op::kWholeUnits)>>
    : std::bool_constant<Op::kWholeUnits> {};

// Threads (512 or 1024) that hold a unit of P packets whole at sixteen packets per thread (one
// tensor) or eight each (two), 0 where neither does or 256 threads do. (Every such unit needs
// more than half of those packets, so there is one flavour per workgroup size.)
inline int whole_unit_threads(int64_t P, int kIn) {
  const int rmax = 16 / kIn;
  if (P <= static_cast<int64_t>(kCoopThreads) * rmax) return 0;  // a slice of the 256-thread kernel
  for (const int threads : {512, 1024}) {
    if (P <= static_cast<int64_t>(threads) * rmax) return threads;
  }
  return 0;
}

template <typename T, typename Op, bool kWin>
int launch_channel_whole(const SliceUnits& sh, const Op& op, const T* in0, const T* in1, T* out,
                         hipStream_t stream) {
  constexpr int kIn = Op::kIn;
  constexpr int kVec = IO<T>::kVec;
  // (short runs are left to the split reduction, as in plan_coop)
  if (sh.seglen / kVec < (kWin ? 24u : 16u)) return kNotApplicable;
  // Fewer units than compute units: slices spread them over more workgroups.
  if (sh.units < static_cast<uint32_t>(num_cus())) return kNotApplicable;
  const uint32_t pps = sh.seglen / kVec + (kWin ? 2 : 0);
  const int64_t P = static_cast<int64_t>(sh.nseg) * pps;
  const int threads = whole_unit_threads(P, kIn);
  if (threads == 0) return kNotApplicable;
  CoopPlan p = {true, 1u, static_cast<uint32_t>(ceil_div(P, kWaveSize) * kWaveSize), 16 / kIn};
  typename IO<T>::Acc* none = nullptr;  // no pairs, no flags: nothing is exchanged
  CoopShape d = make_coop_shape<T>(sh, p, none, kWin, static_cast<uint32_t>(threads));
  d.flags = nullptr;
  const unsigned grid = d.items < (1u << 21) ? d.items : 1u << 21;
  if (kWin) note_flavour("windows");
  if (threads == 512) {
    hipLaunchKernelGGL((channel_whole<T, 16 / kIn, 512, Op, kWin>), dim3(grid), dim3(512), 0, stream,
                       d, in0, in1, out, op);
  } else {
    hipLaunchKernelGGL((channel_whole<T, 16 / kIn, 1024, Op, kWin>), dim3(grid), dim3(1024), 0,
                       stream, d, in0, in1, out, op);
  }
  return status_of_launch();
}

template <typename A>
inline void fill_unset(A* pairs, const CoopShape& d, hipStream_t stream) {
  using Bits = typename Unset<A>::Bits;
  const uint32_t n = d.items * 2;
  hipLaunchKernelGGL((fill_exchange<Bits>), dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256),
                     0, stream, reinterpret_cast<Bits*>(pairs), n, Unset<A>::kValue, d.flags,
                     d.items + 1);
}

// DRAGON_HIP_OK when the single-read kernel was launched, kNotApplicable when
// the shape or alignment leaves the call to the split path, or an error.
// `scratch` holds coop_scratch_bytes<T>(sh) bytes.
constexpr unsigned kCoopRepairGrid = 256;
template <typename T, typename Op, bool kWin>
int launch_channel_slices(const SliceUnits& sh, const CoopPlan& p, const Op& op, const T* in0,
                          const T* in1, T* out, typename IO<T>::Acc* scratch, hipStream_t stream) {
  constexpr int kIn = Op::kIn;
  const CoopShape d = make_coop_shape<T>(sh, p, scratch, kWin);
  // Workgroups launched: all of them resident at once, and at least as many as a unit has slices.
#define DRAGON_HIP_COOP_GRID(R)                                                                \
  [&] {                                                                                        \
    const unsigned resident = resident_grid(channel_slices<T, R, Op, kWin>, kCoopThreads, 0);  \
    const unsigned want = coop_grid(coop_rmax(kIn), kIn);                                      \
    return resident < want ? resident : want;                                                  \
  }()
#define DRAGON_HIP_COOP_LAUNCH(R)                                                              \
  {                                                                                            \
    const unsigned cap = DRAGON_HIP_COOP_GRID(R);                                              \
    if (p.K > cap) return kNotApplicable;                                                      \
    note_number("slices", p.K);                                                                \
    if (kWin) note_flavour("windows");                                                         \
    if (p.K > 1) fill_unset(scratch, d, stream);                                               \
    hipLaunchKernelGGL((channel_slices<T, R, Op, kWin>), dim3(d.items < cap ? d.items : cap),  \
                       dim3(kCoopThreads), 0, stream, d, in0, in1, out, op, scratch);          \
  }
  if (p.r * kIn <= 4) DRAGON_HIP_COOP_LAUNCH(4 / kIn)
  else if (p.r * kIn <= 8) DRAGON_HIP_COOP_LAUNCH(8 / kIn)
  else if (p.r * kIn <= 16) DRAGON_HIP_COOP_LAUNCH(16 / kIn)
  else if constexpr (kIn == 2) DRAGON_HIP_COOP_LAUNCH(12)  // one tensor: never more than 16 packets
#undef DRAGON_HIP_COOP_LAUNCH
#undef DRAGON_HIP_COOP_GRID
  if (p.K == 1) return status_of_launch();  // nothing was exchanged: nothing to repair
  // the widest slice serves every plan: a repair is rare and its speed does not matter
  constexpr int kRepairR = kIn == 2 ? 12 : 16;
  hipLaunchKernelGGL((channel_slices_repair<T, kRepairR, Op, kWin>),
                     dim3(d.items < kCoopRepairGrid ? d.items : kCoopRepairGrid), dim3(kCoopThreads),
                     0, stream, d, in0, in1, out, op, scratch);
  return status_of_launch();
}

template <typename T, typename Op>
int try_channel_slices(const SliceUnits& sh, const Op& op, const T* in0, const T* in1, T* out,
                       typename IO<T>::Acc* scratch, hipStream_t stream) {
  constexpr int kIn = Op::kIn;
  // In place, a repair launch could re-read what another slice of the unit has already
  // overwritten; a unit of one slice exchanges nothing and is never repaired.
  const bool in_place_hazard = OpBeginReadsInput<Op>::value && static_cast<const void*>(out) == in0;
  const bool packets = sh.seglen % IO<T>::kVec == 0 && sh.unit_stride % IO<T>::kVec == 0 &&
      sh.seg_stride % IO<T>::kVec == 0 && aligned16(in0) && aligned16(in1) && aligned16(out);
  if (packets) {
    if constexpr (OpTakesWholeUnits<Op>::value) {
      // units of 64-256 KB per tensor (64-128 KB each for two): whole, instead of 2-4 slices
      // that exchange their sums
      const int st = launch_channel_whole<T, Op, false>(sh, op, in0, in1, out, stream);
      if (st != kNotApplicable) return st;
    }
    const CoopPlan p = plan_coop<T>(sh, kIn);
    if (!p.ok || (in_place_hazard && p.K > 1)) return kNotApplicable;
    return launch_channel_slices<T, Op, false>(sh, p, op, in0, in1, out, scratch, stream);
  }
  if constexpr (OpTakesWindows<Op>::value) {
    if (sizeof(T) > 4 || !congruent16(in0, in1) || !congruent16(in0, out)) return kNotApplicable;
    if constexpr (OpTakesWholeUnits<Op>::value) {
      const int st = launch_channel_whole<T, Op, true>(sh, op, in0, in1, out, stream);
      if (st != kNotApplicable) return st;
    }
    const CoopPlan p = plan_coop<T>(sh, kIn, true);
    if (!p.ok || (in_place_hazard && p.K > 1)) return kNotApplicable;
    return launch_channel_slices<T, Op, true>(sh, p, op, in0, in1, out, scratch, stream);
  }
  return kNotApplicable;
}


} // namespace dragon_hip
