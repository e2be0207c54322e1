// GroupNorm forward over NHWC samples that do not fit one workgroup: x is read once.
//
// A sample is S rows of C channels. It is cut into K slices of whole rows; a
// workgroup of 256 (or 512) threads keeps its slice in registers as raw packets
// (thread (r, cp) holds packet cp of rows r, r + R, r + 2R, ... of the slice,
// R = threads / (C / kVec) rows at a time), so a thread's channels, their group
// and their parameters are the same for every item it sees. A slice holds a share
// of every group of the sample, so an item has G partial pairs to exchange, not
// one. If every slice read every other slice's G pairs, a sample would cost
// G * K * K uncached reads; instead the groups are dealt out over the sample's
// slices, and the exchange has two steps:
//   1. a slice publishes its G partial pairs (before it waits for anything);
//   2. slice k, the combiner of groups k, k + K, k + 2K, ..., waits for the K
//      partial pairs of each of them (one wavefront per group, a pair or a
//      few per lane), forms the group's totals in a fixed order and publishes
//      them as one pair per group (and writes the group's mean and rsig);
//   3. every slice waits for the sample's G total pairs and finishes its rows
//      out of registers.
// A combiner waits only for partial pairs, which every workgroup publishes
// before its first wait; totals wait only for combiners. Items are dealt out
// and walked as in slices.h (item w = n*K + k on workgroup w % grid, ascending;
// the whole grid resident; K never above the grid), so the same induction
// shows that every wait is for a workgroup that is running.
//
// A pair is two fp32 words, published and read as one 64-bit word with
// device-scope atomic accesses; a pair is complete when neither half holds the
// unset pattern (slices.h).
//
// The waits are bounded, and an item whose wait runs out is flagged and
// finished by a second launch behind the first, exactly as in slices.h. By then
// every partial pair is published, so the repair forms the totals of all G
// groups itself with the combiner's arithmetic (contraction off: the same bits)
// and, for the groups its slice combines, writes the mean and rsig the
// combiner did not. A flagged item wrote no output, so a call may run in place.
//
// A group is at least a packet wide. Where it is not whole packets (10, 12, 20
// channels in 16-bit types) a packet may lie in two groups, never three; the
// kTwo flavour then keeps two shares per thread (the elements below k0 belong to
// group g, the others to g + 1) and picks mean and rsig per element.
//
// Partials are (mean, sum of squared deviations) of the slice's share of the
// group, formed in two passes over the registers; the combiner adds them up with
// the counts the slice geometry gives (slice_group_moments). Nothing depends on an element outside
// the slice.
//
// Every item pays the two steps of the exchange, about 10 us on MI355X during
// which its workgroup moves nothing, so the kernel reaches 4-4.7 TB/s where a
// plain copy reaches 5.5. Measured cold on MI355X against the two-pass path
// (column statistics, then the map) on tensors of the same size: [32, 64*64,
// 512] bf16 65 us against 84, fp32 123 against 141; [64, 32*32, 512] bf16 27.5
// against 46. A backward built the same way (x and dy in registers, ds / db
// exchanged) holds half as many rows per item and pays the exchange twice as
// often: 143 us against 122 for the five-pass path at the first shape, so the
// backward keeps the five passes.
#pragma once

#include "slices.h"

namespace dragon_hip {

// Workgroup size: 256 threads, four workgroups per compute unit, or 512, two, for rows whose
// packets would leave too many of 256 threads without a row (C = 1280 in 16-bit types). Either
// way four wavefronts per SIMD, i.e. 128 registers (the second launch bound counts wavefronts
// per SIMD, not workgroups).
constexpr int kMaxSliceThreads = 512;
constexpr int kSlicePackets = 16;  // per thread: a slice is up to 64 KB
constexpr uint32_t kMaxSampleSlices = 1024;  // slices per sample (a resident grid holds no more workgroups)
constexpr uint32_t kMaxSampleGroups = 256;  // groups: one owner thread each

struct SampleSlices {
  uint32_t N, S, C, G, D;
  uint32_t threads;   // workgroup size
  uint32_t K;         // slices per sample
  uint32_t rows;      // rows per slice (the last slice of a sample may hold fewer)
  uint32_t items;     // N * K
  uint32_t patience;  // polls of a slot before a thread gives up
  uint32_t* flags;    // flags[w] = 1: item w gave up; flags[items] = 1: some item did
  uint32_t* gave_up_count;
};

// How a packet's channels lie in groups.
enum SliceSplit {
  kSplitNone = 0,  // groups of whole packets: a packet lies in one group
  kSplitTwo = 1,   // groups of at least a packet that are not whole packets: in at most two
  kSplitEach = 2   // groups of less than a packet: every channel of a packet finds its own group
};

struct SampleSlicePlan {
  bool ok;
  int split;  // SliceSplit
  uint32_t threads, K, rows;
  int vpt;  // packets per thread and tensor
};

// Up to 16 packets per thread, four workgroups per compute unit (128 registers).
template <typename T>
SampleSlicePlan plan_sample_slices(uint32_t S, uint32_t C, uint32_t G, uint32_t D) {
  constexpr uint32_t kVec = IO<T>::kVec;
  SampleSlicePlan p{false, kSplitNone, 0u, 0u, 0u, 0};
  if (sizeof(T) > 4 || S <= 1 || C % kVec != 0) return p;
  p.split = D % kVec == 0 ? kSplitNone : D > kVec ? kSplitTwo : kSplitEach;
  const uint32_t cps = C / kVec;
  if (G > kMaxSampleGroups) return p;
  // most of the workgroup's threads must have a row to hold
  auto fits = [&](uint32_t threads) {
    return cps <= threads && cps * (threads / cps) * 4 >= threads * 3;
  };
  for (const uint32_t threads : {256u, 512u}) {
    if (fits(threads)) {
      p.threads = threads;
      break;
    }
  }
  if (p.threads == 0) return p;
  // A sample that 512 threads hold as one slice and 256 as two takes the one slice: nothing to
  // exchange (bf16 [1024, 16*16, 256] 61 -> 49 us, [2048, 14*14, 256] 93 -> 79 us). A workgroup of
  // 1024 (one per compute unit) loses to either: 75 and 125 us on those shapes.
  if (p.threads == 256 && fits(512u) && S > 256 / cps * kSlicePackets &&
      S <= 512 / cps * kSlicePackets) {
    p.threads = 512;
  }
  const uint32_t rows_at_a_time = p.threads / cps;
  const uint32_t vmax = kSlicePackets;
  const uint32_t k0 = static_cast<uint32_t>(ceil_div(S, rows_at_a_time * vmax));
  // slices of about the same size
  const uint32_t vpt = static_cast<uint32_t>(ceil_div(ceil_div(S, k0), rows_at_a_time));
  p.rows = rows_at_a_time * vpt;
  p.K = static_cast<uint32_t>(ceil_div(S, p.rows));
  p.vpt = static_cast<int>(vpt);
  p.ok = p.K <= kMaxSampleSlices;
  return p;
}

// Scratch words of a call, in accumulator words: G pairs per item, G pairs per
// sample, then the flags (a 32-bit word each, one more than there are items).
inline size_t sample_slices_exchange_words(uint32_t N, uint32_t G, uint32_t K) {
  return (static_cast<size_t>(N) * K * G + static_cast<size_t>(N) * G) * 2;
}
inline size_t sample_slices_exchange_bytes(uint32_t N, uint32_t G, uint32_t K, size_t acc_size) {
  const size_t bytes = sample_slices_exchange_words(N, G, K) * acc_size +
      (static_cast<size_t>(N) * K + 1) * sizeof(uint32_t);
  return (bytes + 255) / 256 * 256;
}

template <typename T>
SampleSlices make_sample_slices(uint32_t N, uint32_t S, uint32_t C, uint32_t G, uint32_t D,
                                const SampleSlicePlan& p, typename IO<T>::Acc* exchange) {
  SampleSlices d;
  d.N = N, d.S = S, d.C = C, d.G = G, d.D = D;
  d.threads = p.threads, d.K = p.K, d.rows = p.rows, d.items = N * p.K;
  const uint32_t patience = exchange_patience();
  d.patience = patience ? patience : kCoopPatience;
  d.flags = exchange ? reinterpret_cast<uint32_t*>(exchange + sample_slices_exchange_words(N, G, p.K))
                     : nullptr;  // (a sample in one slice: no exchange)
  d.gave_up_count = exchange_gave_up_counter();
  return d;
}

// Threads that add up one group's shares together (a power of two, adjacent lanes of one
// wavefront): the team size for G groups, `rows` rows at a time and a workgroup of `threads`.
__host__ __device__ inline uint32_t team_size(uint32_t G, uint32_t rows, uint32_t threads) {
  uint32_t team = kWaveSize;
  while (team > 1 && (team * G > threads || team > rows)) team >>= 1;
  return team;
}

// Where a thread sits in its workgroup's slice.
template <int kVec>
struct SliceSeat {
  uint32_t cps, rows_at_a_time, r, cp, g, lanes_per_group;
  uint32_t g1;  // where groups are not whole packets: the group of the packet's last channels,
  int k0;       // and how many of its channels lie in g (the first group)
  uint32_t team;  // adjacent threads that add up one group's shares (a power of two, <= 64)
  bool on;
  __device__ explicit SliceSeat(const SampleSlices& d) {
    cps = d.C / kVec;
    rows_at_a_time = d.threads / cps;
    r = threadIdx.x / cps, cp = threadIdx.x - r * cps;
    on = r < rows_at_a_time;
    lanes_per_group = d.D / kVec;
    g = on ? cp * kVec / d.D : 0u;
    k0 = static_cast<int>(min(static_cast<uint32_t>(kVec), (g + 1) * d.D - (on ? cp : 0u) * kVec));
    g1 = g + 1 < d.G ? g + 1 : g;
    team = team_size(d.G, rows_at_a_time, d.threads);
  }
};

struct SliceItem {
  uint32_t n, k, row0, nrows;
  __device__ SliceItem(const SampleSlices& d, uint32_t w) {
    n = w / d.K, k = w - n * d.K;
    row0 = k * d.rows;
    nrows = min(d.rows, d.S - row0);
  }
};

// Element offset of the thread's first packet of the item, and between its packets.
template <int kVec>
__device__ __forceinline__ uint32_t slice_first(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                const SliceItem& it) {
  return (it.n * d.S + it.row0 + at.r) * d.C + at.cp * kVec;
}

// Packet i of a thread exists while i * R < room. The loops over a thread's packets count
// `room` down and an offset up, one register each: sixteen row numbers and sixteen offsets per
// thread, which the unrolled loops would otherwise keep across the whole item loop, do not fit.
template <int kVec>
__device__ __forceinline__ int slice_room(const SliceSeat<kVec>& at, const SliceItem& it) {
  return at.on ? static_cast<int>(it.nrows) - static_cast<int>(at.r) : 0;
}

template <typename T, int kVPT>
__device__ __forceinline__ void slice_load(const SampleSlices& d, const SliceSeat<IO<T>::kVec>& at,
                                           const SliceItem& it, const T* in, u32x4 (&raw)[kVPT]) {
  const uint32_t step = at.rows_at_a_time * d.C;
  int room = slice_room(at, it);
  uint32_t off = slice_first(d, at, it);
#pragma unroll
  for (int i = 0; i < kVPT; ++i) {
    raw[i] = load_packet(in + (room > 0 ? off : 0u));
    room -= static_cast<int>(at.rows_at_a_time), off += step;
    asm volatile("" : "+v"(room), "+v"(off));
  }
}

// A pair of fp32 words is published and read as one 64-bit word: one request, and
// both halves arrive together.
__device__ __forceinline__ unsigned long long pair_bits(const float a, const float b) {
  return static_cast<unsigned long long>(publishable_bits(a)) |
      (static_cast<unsigned long long>(publishable_bits(b)) << 32);
}
__device__ __forceinline__ void publish_pair(float* slot, const float a, const float b) {
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(slot), pair_bits(a, b), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long peek_pair(const float* slot) {
  return __hip_atomic_load(reinterpret_cast<const unsigned long long*>(slot), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool pair_set(unsigned long long u) {
  return static_cast<uint32_t>(u) != 0xffffffffu && static_cast<uint32_t>(u >> 32) != 0xffffffffu;
}
// false: the pair was still unset after `patience` polls (a and b are then meaningless);
// `u` is what a first look has already seen
__device__ __forceinline__ bool await_pair(const float* slot, uint32_t patience, unsigned long long u,
                                           float& a, float& b) {
  for (;;) {
    a = __builtin_bit_cast(float, static_cast<uint32_t>(u));
    b = __builtin_bit_cast(float, static_cast<uint32_t>(u >> 32));
    if (pair_set(u)) return true;
    if (--patience == 0) return false;
    __builtin_amdgcn_s_sleep(8);
    u = peek_pair(slot);
  }
}
__device__ __forceinline__ bool await_pair(const float* slot, uint32_t patience, float& a, float& b) {
  return await_pair(slot, patience, peek_pair(slot), a, b);
}

// The group's totals of the threads' shares, one LDS word per thread and share. A team of
// `at.team` adjacent threads adds up group t: member j takes rows j, j + team, ... of the rows
// the workgroup holds at a time (`row_sum(g, rr)`: what row rr adds to group g, in a fixed
// order), the members' sums meet in a butterfly of shuffles, and the team's first thread
// leaves the total in total[j][t]. The order of the additions depends on the geometry alone.
// Every thread may read total[j][*] afterwards; the barrier of the next call (or of the
// exchange) lies between those reads and the next writes.
template <int kN, typename A, typename Total, typename RowSum>
__device__ __forceinline__ void team_sums(uint32_t G, uint32_t rows_at_a_time, uint32_t team,
                                          Total total, RowSum row_sum) {
  const uint32_t t = threadIdx.x;
  const uint32_t g = t / team, j = t - g * team;
  A acc[kN];
#pragma unroll
  for (int k = 0; k < kN; ++k) acc[k] = A(0);
  if (g < G) {
    for (uint32_t rr = j; rr < rows_at_a_time; rr += team) row_sum(g, rr, acc);
  }
  for (uint32_t o = 1; o < team; o <<= 1) {
#pragma unroll
    for (int k = 0; k < kN; ++k) acc[k] += __shfl_xor(acc[k], static_cast<int>(o), kWaveSize);
  }
  if (g < G && j == 0) {
#pragma unroll
    for (int k = 0; k < kN; ++k) total[k][g] = acc[k];
  }
  __syncthreads();
}
template <int kN, int kVec, typename A, typename RowSum>
__device__ __forceinline__ void slice_team_sums(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                A (*total)[kMaxSliceThreads], RowSum row_sum) {
  team_sums<kN, A>(d.G, at.rows_at_a_time, at.team, total, row_sum);
}

// Groups of whole packets: kN values per thread, all for the group of its packet.
template <int kN, int kVec, typename A>
__device__ __forceinline__ void slice_group_sums(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                 const A (&v)[kN], A (*part)[kMaxSliceThreads],
                                                 A (*total)[kMaxSliceThreads]) {
  const uint32_t t = threadIdx.x;
#pragma unroll
  for (int j = 0; j < kN; ++j) part[j][t] = at.on ? v[j] : A(0);
  __syncthreads();
  slice_team_sums<kN, kVec>(d, at, total, [&](uint32_t g, uint32_t rr, A (&acc)[kN]) {
    const uint32_t first = rr * at.cps + g * at.lanes_per_group;
    for (uint32_t c = 0; c < at.lanes_per_group; ++c) {
#pragma unroll
      for (int j = 0; j < kN; ++j) acc[j] += part[j][first + c];
    }
  });
}

// The same where a packet may lie in two groups: v0 is the thread's share for the group of its
// packet's first channel, v1 for the next group; group g takes the shares of the packets that
// touch it (packet c starts in group g, or, only the first of them, before it).
template <int kVec, typename A>
__device__ __forceinline__ void slice_group_sums_two(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                     const A v0, const A v1,
                                                     A (*part)[kMaxSliceThreads],
                                                     A (*total)[kMaxSliceThreads]) {
  const uint32_t t = threadIdx.x;
  part[0][t] = at.on ? v0 : A(0);
  part[1][t] = at.on ? v1 : A(0);
  __syncthreads();
  slice_team_sums<1, kVec>(d, at, total, [&](uint32_t g, uint32_t rr, A (&acc)[1]) {
    const uint32_t lo = g * d.D / kVec, hi = ((g + 1) * d.D - 1) / kVec;
    for (uint32_t c = lo; c <= hi; ++c) {
      const int share = c * kVec < g * d.D ? 1 : 0;
      acc[0] += part[share][rr * at.cps + c];
    }
  });
}

// The same where groups are narrower than a packet: a share per channel of the packet; group g
// takes the shares of its D channels.
template <int kVec, typename A>
__device__ __forceinline__ void slice_group_sums_each(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                      const A (&v)[kVec],
                                                      A (*each)[kMaxSliceThreads],
                                                      A (*total)[kMaxSliceThreads]) {
  const uint32_t t = threadIdx.x;
#pragma unroll
  for (int e = 0; e < kVec; ++e) each[e][t] = at.on ? v[e] : A(0);
  __syncthreads();
  slice_team_sums<1, kVec>(d, at, total, [&](uint32_t g, uint32_t rr, A (&acc)[1]) {
    for (uint32_t ch = g * d.D; ch < (g + 1) * d.D; ++ch) {
      acc[0] += each[ch % kVec][rr * at.cps + ch / kVec];
    }
  });
}

// The groups of the kVec channels of the thread's packet (kSplitEach).
template <int kVec>
__device__ __forceinline__ void slice_channel_groups(const SampleSlices& d, const SliceSeat<kVec>& at,
                                                     uint32_t (&ge)[kVec]) {
  uint32_t g = at.g, r = (at.on ? at.cp : 0u) * kVec - at.g * d.D;  // r < D
#pragma unroll
  for (int e = 0; e < kVec; ++e) {
    if (r >= d.D) r -= d.D, ++g;
    ge[e] = g < d.G ? g : d.G - 1;
    ++r;
  }
}

// The sum of v over the wavefront, the same bits in every lane (each step adds
// the two halves of a pair of lanes, which commutes).
template <typename A>
__device__ __forceinline__ A wave_total(A v) {
#pragma unroll
  for (int o = 1; o < kWaveSize; o <<= 1) v += __shfl_xor(v, o, kWaveSize);
  return v;
}

template <typename A>
struct SliceLds {
  A part[2][kMaxSliceThreads];
  A total[2][kMaxSliceThreads];
};

__device__ __forceinline__ void slice_flag(const SampleSlices& d, uint32_t w) {
  if (threadIdx.x == 0) {
    __hip_atomic_store(d.flags + w, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(d.flags + d.items, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (d.gave_up_count) {
      __hip_atomic_fetch_add(d.gave_up_count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// One wavefront: the K partial (mean, squared deviations) pairs of group g of
// sample n become the group's mean and rsig, the same bits in every lane, with
// two plain sums: the count-weighted mean of the slices' means, then the slices'
// squared deviations plus what the distances of their means from the total mean
// add. Lane l takes slices l, l + 64, ...; it keeps its first pair for the
// second sum and reads any further ones (K > 64) again. Contraction is off so
// that the combiner and the repair launch, which reach this code through
// different callers, round alike. false (the same in every lane): a pair was
// still unset.
template <typename A>
__device__ __forceinline__ bool slice_group_moments(const SampleSlices& d, const A* partials,
                                                    uint32_t n, uint32_t g, uint32_t patience,
                                                    const A eps, A& o0, A& o1) {
#pragma clang fp contract(off)
  const uint32_t lane = threadIdx.x & (kWaveSize - 1);
  const A* pairs = partials + (static_cast<size_t>(n) * d.K * d.G + g) * 2;
  const A inv_l = A(1) / A(static_cast<int64_t>(d.D) * d.S);
  int gave_up = 0;
  A a0 = A(0), b0 = A(0), c0 = A(0), sum = A(0);
  for (uint32_t q = lane; q < d.K; q += kWaveSize) {
    A a, b;
    if (!await_pair(pairs + static_cast<size_t>(q) * d.G * 2, patience, a, b)) gave_up = 1;
    const A cnt = A(min(d.rows, d.S - q * d.rows) * d.D);
    sum += cnt * a;
    if (q == lane) a0 = a, b0 = b, c0 = cnt;
  }
  const A mean = wave_total(sum) * inv_l;
  const A d0 = a0 - mean;
  A m2 = b0 + (c0 * d0) * d0;
  for (uint32_t q = lane + kWaveSize; q < d.K; q += kWaveSize) {
    A a, b;
    (void)await_pair(pairs + static_cast<size_t>(q) * d.G * 2, 1u, a, b);  // seen set above
    const A cnt = A(min(d.rows, d.S - q * d.rows) * d.D);
    const A dq = a - mean;
    m2 += b + (cnt * dq) * dq;
  }
  o0 = mean;
  o1 = acc_rsqrt_exact(wave_total(m2) * inv_l + eps);
  return !__any(gave_up);
}

// Step 1 for item w: the owner threads (t < G) publish the item's G partial pairs.
template <typename A>
__device__ __forceinline__ void slice_publish(const SampleSlices& d, uint32_t w, const A pa,
                                              const A pb, A* exchange) {
  const uint32_t t = threadIdx.x;
  if (t < d.G) publish_pair(exchange + (static_cast<size_t>(w) * d.G + t) * 2, pa, pb);
}

// Steps 2 and 3 for item w. Afterwards lds.total[0 / 1][g] hold group g's total
// pair in every thread's view; out0 / out1 (per (n, g)) have been written for
// the groups this slice combines. false (for the whole workgroup): a wait ran
// out and the item has been flagged. kRepair: nothing is published or waited
// for.
template <bool kRepair, typename A>
__device__ __forceinline__ bool slice_totals(const SampleSlices& d, const SliceItem& it, uint32_t w,
                                             const A eps, A* exchange, A* out0, A* out1,
                                             SliceLds<A>& lds) {
  const uint32_t t = threadIdx.x;
  const uint32_t wave = t / kWaveSize, lane = t & (kWaveSize - 1), waves = d.threads / kWaveSize;
  if (d.K == 1) {  // the owner threads have left the sample's own statistics in LDS
    __syncthreads();
    return true;
  }
  A* partials = exchange;
  A* totals = exchange + static_cast<size_t>(d.items) * d.G * 2;
  if constexpr (kRepair) {
    for (uint32_t g = wave; g < d.G; g += waves) {
      A o0, o1;
      (void)slice_group_moments(d, partials, it.n, g, 1u, eps, o0, o1);
      if (lane == 0) {
        lds.total[0][g] = o0, lds.total[1][g] = o1;
        if (g % d.K == it.k) {
          out0[static_cast<size_t>(it.n) * d.G + g] = o0;
          out1[static_cast<size_t>(it.n) * d.G + g] = o1;
        }
      }
    }
    __syncthreads();
    return true;
  } else {
    // the groups this slice combines: k, k + K, ..., a wavefront each
    int gave_up = 0;
    for (uint32_t g = it.k + wave * d.K; g < d.G; g += waves * d.K) {
      A o0, o1;
      if (!slice_group_moments(d, partials, it.n, g, d.patience, eps, o0, o1)) {
        gave_up = 1;  // the group's totals stay unset: every slice of the sample will be flagged
      } else if (lane == 0) {
        publish_pair(totals + (static_cast<size_t>(it.n) * d.G + g) * 2, o0, o1);
        out0[static_cast<size_t>(it.n) * d.G + g] = o0;
        out1[static_cast<size_t>(it.n) * d.G + g] = o1;
      }
    }
    if (t < d.G) {
      A a, b;
      if (!await_pair(totals + (static_cast<size_t>(it.n) * d.G + t) * 2, d.patience, a, b)) {
        gave_up = 1;
      }
      lds.total[0][t] = a, lds.total[1][t] = b;
    }
    if (__syncthreads_or(gave_up)) {
      slice_flag(d, w);
      return false;
    }
    return true;
  }
}

// ---------------------------------------------------------------- forward
// The slice's share of each group: its mean, then its squared deviations from
// that mean; the owner threads publish them.
template <typename T, int kVPT, int kSplit>
__device__ __forceinline__ void slice_forward_stats(
    const SampleSlices& d, const SliceSeat<IO<T>::kVec>& at, uint32_t w,
    const typename IO<T>::Acc eps, typename IO<T>::Acc* mu, typename IO<T>::Acc* rsig,
    typename IO<T>::Acc* exchange, u32x4 (&raw)[kVPT], SliceLds<typename IO<T>::Acc>& lds,
    typename IO<T>::Acc (*each)[kMaxSliceThreads]) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr bool kTwo = kSplit == kSplitTwo, kEach = kSplit == kSplitEach;
  constexpr int kShares = kEach ? kVec : 2;
  const SliceItem it(d, w);
  const uint32_t t = threadIdx.x;
  const A inv_cnt = A(1) / A(it.nrows * d.D);
  // (kTwo: s[0] for the group of the packet's first channel, s[1] for the next one; kEach: a
  // share per channel)
  A s[kShares];
#pragma unroll
  for (int j = 0; j < kShares; ++j) s[j] = A(0);
  int room = slice_room(at, it);
#pragma unroll
  for (int i = 0; i < kVPT; ++i) {
    const bool has = room > 0;
    room -= static_cast<int>(at.rows_at_a_time);
    asm volatile("" : "+v"(room));
    if (has) {
      A v[kVec];
      IO<T>::unpack(raw[i], v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if constexpr (kEach) {
          s[e] += v[e];
        } else {
          if (!kTwo || e < at.k0) s[0] += v[e]; else s[1] += v[e];
        }
      }
    }
  }
  auto group_sums = [&]() {
    if constexpr (kEach) {
      slice_group_sums_each<kVec>(d, at, s, each, lds.total);
    } else if constexpr (kTwo) {
      slice_group_sums_two<kVec>(d, at, s[0], s[1], lds.part, lds.total);
    } else {
      const A one[1] = {s[0]};
      slice_group_sums<1, kVec>(d, at, one, lds.part, lds.total);
    }
  };
  group_sums();
  A pa = A(0), pb = A(0);
  if (t < d.G) pa = lds.total[0][t] * inv_cnt;
  // the slice's mean of each share's group
  A mean_k[kShares];
  if constexpr (kEach) {
    uint32_t ge[kVec];
    slice_channel_groups<kVec>(d, at, ge);
#pragma unroll
    for (int e = 0; e < kVec; ++e) mean_k[e] = lds.total[0][ge[e]] * inv_cnt;
  } else {
    mean_k[0] = lds.total[0][at.g] * inv_cnt;
    mean_k[1] = kTwo ? lds.total[0][at.g1] * inv_cnt : A(0);
  }
  // convert the packets again in each pass instead of keeping every converted element
#pragma unroll
  for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
#pragma unroll
  for (int j = 0; j < kShares; ++j) s[j] = A(0);
  room = slice_room(at, it);
#pragma unroll
  for (int i = 0; i < kVPT; ++i) {
    const bool has = room > 0;
    room -= static_cast<int>(at.rows_at_a_time);
    asm volatile("" : "+v"(room));
    if (has) {
      A v[kVec];
      IO<T>::unpack(raw[i], v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if constexpr (kEach) {
          const A dv = v[e] - mean_k[e];
          s[e] += dv * dv;
        } else if (!kTwo || e < at.k0) {
          const A dv = v[e] - mean_k[0];
          s[0] += dv * dv;
        } else {
          const A dv = v[e] - mean_k[1];
          s[1] += dv * dv;
        }
      }
    }
  }
  group_sums();
  if (t < d.G) pb = lds.total[0][t];
#pragma unroll
  for (int i = 0; i < kVPT; ++i) asm volatile("" : "+v"(raw[i]));
  if (d.K == 1) {
    // a sample in one slice: its statistics are this workgroup's own, nothing is exchanged
    if (t < d.G) {
      const A rs = acc_rsqrt_exact(pb * inv_cnt + eps);
      lds.total[0][t] = pa, lds.total[1][t] = rs;
      mu[static_cast<size_t>(it.n) * d.G + t] = pa;
      rsig[static_cast<size_t>(it.n) * d.G + t] = rs;
    }
  } else {
    slice_publish(d, w, pa, pb, exchange);
  }
}

// Totals of item w, its rows out of `raw`, and item `reload` (if below d.items) into `raw`.
template <typename T, int kVPT, bool kRepair, int kSplit>
__device__ __forceinline__ void slice_forward_finish(
    const SampleSlices& d, const SliceSeat<IO<T>::kVec>& at, uint32_t w, uint32_t reload,
    const typename IO<T>::Acc eps, const T* x, const typename IO<T>::Acc* gamma,
    const typename IO<T>::Acc* beta, typename IO<T>::Acc* mu, typename IO<T>::Acc* rsig, T* y,
    typename IO<T>::Acc* exchange, u32x4 (&raw)[kVPT], SliceLds<typename IO<T>::Acc>& lds) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr bool kTwo = kSplit == kSplitTwo, kEach = kSplit == kSplitEach;
  const SliceItem it(d, w);
  const bool complete = slice_totals<kRepair>(d, it, w, eps, exchange, mu, rsig, lds);
  const A mean = lds.total[0][at.g], rs = lds.total[1][at.g];
  const A mean1 = kTwo ? lds.total[0][at.g1] : A(0), rs1 = kTwo ? lds.total[1][at.g1] : A(0);
  const bool more = !kRepair && reload < d.items;  // uniform over the workgroup
  const SliceItem nit(d, more ? reload : w);
  const uint32_t first = slice_first(d, at, it), step = at.rows_at_a_time * d.C;
  const uint32_t nfirst = slice_first(d, at, nit);
  {
    // One path whether the item is complete or not (an incomplete item only skips its
    // stores): with a second path that also loads the next item the register allocator
    // spilled 120-300 bytes per thread at sixteen packets and 128 registers.
    // The thread's channels are the same for every item, but their parameters are
    // fetched per item so that they do not occupy registers while the slice is reduced.
    const A* gp = gamma + (at.on ? at.cp * kVec : 0u);
    const A* bp = beta + (at.on ? at.cp * kVec : 0u);
    asm volatile("" : "+v"(gp), "+v"(bp));
    A gam[kVec], bet[kVec];
    load_params_ragged<kVec>(gp, kVec, gam);
    load_params_ragged<kVec>(bp, kVec, bet);
    A mean_e[kEach ? kVec : 1];  // kEach: the mean of each channel's group
    if constexpr (kEach) {
      uint32_t ge[kVec];
      slice_channel_groups<kVec>(d, at, ge);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        mean_e[e] = lds.total[0][ge[e]];
        gam[e] *= lds.total[1][ge[e]];
      }
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) gam[e] *= !kTwo || e < at.k0 ? rs : rs1;
    }
    int room = complete ? slice_room(at, it) : 0, nroom = slice_room(at, nit);
    uint32_t off = first, noff = nfirst;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (room > 0) {
        A v[kVec];
        IO<T>::unpack(raw[i], v);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if constexpr (kEach) {
            v[e] = (v[e] - mean_e[e]) * gam[e] + bet[e];
          } else {
            v[e] = (v[e] - (!kTwo || e < at.k0 ? mean : mean1)) * gam[e] + bet[e];
          }
        }
        store_packet(y + off, IO<T>::pack(v));
      }
      if (more) raw[i] = load_packet(x + (nroom > 0 ? noff : 0u));
      room -= static_cast<int>(at.rows_at_a_time), nroom -= static_cast<int>(at.rows_at_a_time);
      off += step, noff += step;
      asm volatile("" : "+v"(room), "+v"(nroom), "+v"(off), "+v"(noff));
    }
  }
}

// One item at a time per workgroup; the next item's packets are requested while
// this one's are stored.
template <typename T, int kVPT, int kThreads, int kSplit>
__global__ __launch_bounds__(kThreads, 4) void group_norm_nhwc_slices(
    const SampleSlices d, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y, typename IO<T>::Acc* __restrict__ exchange) {
  using A = typename IO<T>::Acc;
  __shared__ SliceLds<A> lds;
  // (a word per thread and channel of its packet where groups are narrower than a packet)
  __shared__ A each[kSplit == kSplitEach ? IO<T>::kVec : 1][kMaxSliceThreads];
  const SliceSeat<IO<T>::kVec> at(d);
  const uint32_t step = gridDim.x;
  uint32_t w = blockIdx.x;
  u32x4 one[kVPT];
  if (w < d.items) slice_load<T, kVPT>(d, at, SliceItem(d, w), x, one);
  for (; w < d.items; w += step) {
    slice_forward_stats<T, kVPT, kSplit>(d, at, w, eps, mu, rsig, exchange, one, lds, each);
    slice_forward_finish<T, kVPT, false, kSplit>(d, at, w, w + step, eps, x, gamma, beta, mu, rsig,
                                                 y, exchange, one, lds);
  }
}

// The launch behind it: nothing to do unless a wait of the first launch ran out.
template <typename T, int kVPT, int kThreads, int kSplit>
__global__ __launch_bounds__(kThreads, 4) void group_norm_nhwc_slices_repair(
    const SampleSlices d, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y, typename IO<T>::Acc* __restrict__ exchange) {
  using A = typename IO<T>::Acc;
  __shared__ SliceLds<A> lds;
  if (d.flags[d.items] == 0u) return;
  const SliceSeat<IO<T>::kVec> at(d);
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    if (d.flags[w] == 0u) continue;  // the same word in every thread
    u32x4 raw[kVPT];
    slice_load<T, kVPT>(d, at, SliceItem(d, w), x, raw);
    slice_forward_finish<T, kVPT, true, kSplit>(d, at, w, d.items, eps, x, gamma, beta, mu, rsig, y,
                                                exchange, raw, lds);
    __syncthreads();  // the next item rewrites the totals in LDS
  }
}

// ---------------------------------------------------------------- host
constexpr unsigned kSliceRepairGrid = 256;

// The most workgroups the kernel is launched with.
inline uint32_t sample_slices_max_grid() { return static_cast<uint32_t>(num_cus()) * 4u; }

template <typename A>
inline void fill_sample_exchange(A* exchange, const SampleSlices& d, hipStream_t stream) {
  using Bits = typename Unset<A>::Bits;
  const size_t words = sample_slices_exchange_words(d.N, d.G, d.K);
  const uint32_t n = static_cast<uint32_t>(words), nflags = d.items + 1;
  const uint32_t most = n > nflags ? n : nflags;
  hipLaunchKernelGGL((fill_exchange<Bits>), dim3(static_cast<unsigned>(ceil_div(most, 256))),
                     dim3(256), 0, stream, reinterpret_cast<Bits*>(exchange), n, Unset<A>::kValue,
                     d.flags, nflags);
}

// DRAGON_HIP_OK when the kernels were launched, kNotApplicable when the shape
// or the addresses leave the call to the other paths. `scratch` holds
// sample_slices_exchange_bytes(...) bytes (none is needed for samples of one slice).
template <typename T>
int try_group_norm_forward_nhwc_slices(uint32_t N, uint32_t S, uint32_t C, uint32_t G, uint32_t D,
                                       float eps, const void* x, const void* gamma, const void* beta,
                                       void* mu, void* rsig, void* y, void* scratch,
                                       size_t scratch_bytes, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  if constexpr (sizeof(T) > 4) {
    return kNotApplicable;
  } else {
    const SampleSlicePlan p = plan_sample_slices<T>(S, C, G, D);
    if (!p.ok || !aligned16(x) || !aligned16(y)) return kNotApplicable;
    if (static_cast<uint64_t>(N) * p.K * G * 2 + static_cast<uint64_t>(N) * G * 2 > 0x7fffffffull) {
      return kNotApplicable;
    }
    // a sample in one slice exchanges nothing: no scratch, no fill, no repair launch
    if (p.K > 1 && (!scratch || scratch_bytes < sample_slices_exchange_bytes(N, G, p.K, sizeof(A)))) {
      return kNotApplicable;
    }
    A* exchange = p.K > 1 ? static_cast<A*>(scratch) : nullptr;
    const SampleSlices d = make_sample_slices<T>(N, S, C, G, D, p, exchange);
#define LAUNCH_T(VPT, THREADS, SPLIT)                                                             \
  {                                                                                               \
    auto kernel = group_norm_nhwc_slices<T, VPT, THREADS, SPLIT>;                                 \
    unsigned cap = resident_grid(kernel, THREADS, 0);                                             \
    if (cap > sample_slices_max_grid()) cap = sample_slices_max_grid();                           \
    if (p.K > cap) return kNotApplicable;                                                         \
    /* Samples of one slice wait for nobody, so they need not be resident together: from     */ \
    /* four per resident workgroup on, a workgroup per sample, handed out by the hardware as */ \
    /* workgroups finish, is ahead of workgroups that walk the samples and request one ahead */ \
    /* (bf16 [8192, 7*7, 256] 77.6 -> 71.2 us; with two per workgroup 48.9 against 50.6 us). */ \
    const bool walk = p.K > 1 || d.items < 4u * num_cus() * (THREADS == 256 ? 4u : 2u);          \
    if (!walk) cap = 1u << 21; /* (a launch holds fewer than 2^32 threads) */                     \
    note_flavour(SPLIT == kSplitEach ? "group_norm_nhwc_slices<" #VPT "," #THREADS ",each>"       \
                 : SPLIT == kSplitTwo ? "group_norm_nhwc_slices<" #VPT "," #THREADS ",two>"       \
                                      : "group_norm_nhwc_slices<" #VPT "," #THREADS ">");         \
    note_number("slices", p.K);                                                                   \
    if (p.K == 1) note_number("walk", walk ? 1 : 0);                                              \
    if (p.K > 1) fill_sample_exchange(exchange, d, stream);                                       \
    hipLaunchKernelGGL(kernel, dim3(d.items < cap ? d.items : cap), dim3(THREADS), 0, stream, d,  \
                       A(eps), static_cast<const T*>(x), static_cast<const A*>(gamma),            \
                       static_cast<const A*>(beta), static_cast<A*>(mu), static_cast<A*>(rsig),   \
                       static_cast<T*>(y), exchange);                                             \
    if (p.K > 1) {                                                                                \
      /* (the widest flavour serves every plan: a repair is rare, its speed does not matter) */   \
      hipLaunchKernelGGL((group_norm_nhwc_slices_repair<T, kSlicePackets, THREADS, SPLIT>),       \
                         dim3(d.items < kSliceRepairGrid ? d.items : kSliceRepairGrid),           \
                         dim3(THREADS), 0, stream, d, A(eps), static_cast<const T*>(x),           \
                         static_cast<const A*>(gamma), static_cast<const A*>(beta),               \
                         static_cast<A*>(mu), static_cast<A*>(rsig), static_cast<T*>(y),          \
                         exchange);                                                               \
    }                                                                                             \
  }
#define LAUNCH(VPT, THREADS)                                                   \
  {                                                                            \
    if (p.split == kSplitEach) LAUNCH_T(VPT, THREADS, kSplitEach)              \
    else if (p.split == kSplitTwo) LAUNCH_T(VPT, THREADS, kSplitTwo)           \
    else LAUNCH_T(VPT, THREADS, kSplitNone)                                    \
  }
    if (p.threads == 256) {
      if (p.vpt <= 8) LAUNCH(8, 256) else LAUNCH(16, 256)
    } else {
      if (p.vpt <= 8) LAUNCH(8, 512) else LAUNCH(16, 512)
    }
#undef LAUNCH
#undef LAUNCH_T
    return status_of_launch();
  }
}

} // namespace dragon_hip
