// Register-resident row tiles: a row of C elements is split into 16-byte
// packets, packet p of the row is owned by thread p % kTPR of the row's
// thread group in slot p / kTPR, so consecutive lanes touch consecutive
// packets (fully coalesced 128-bit accesses) and the whole row is read from
// HBM exactly once.
//
//   kTPR == 64   one wavefront per row, four rows per 256-thread workgroup,
//                reductions by wave64 shuffles only
//   kTPR == 256 / 1024   one workgroup per row, wave shuffles plus one LDS
//                exchange between the wavefronts
//
// A tile covers rows of up to kTPR * kVPT packets; slots beyond the row's
// packet count are masked off, which is how widths that are not a multiple of
// the tile (e.g. 1000 = 125 packets of 8) are handled.
//
// Ragged tiles (kRagged) take rows of any width and alignment: packets are
// counted from the row's first element, so a packet may sit at an address that
// is only element-aligned, and the last packet of a row may be partial (it is
// then read and written element by element). Their `extent` argument is the
// row's element count; for regular tiles it is the row's packet count.
#pragma once

#include <map>
#include <mutex>
#include <tuple>

#include "common.h"

namespace dragon_hip {

// Workgroup size of a row kernel: wave-per-row tiles share a 256-thread group.
constexpr int row_threads(int tpr) { return tpr == kWaveSize ? 256 : tpr; }

// A row of any width at any element-aligned address, as the aligned 16-byte
// packets that cover it (its window): the window starts `lead` elements before
// the row and its last packet holds `tail_valid` elements of the row. Where a
// kernel does not care which column an element is (softmax and its gradient;
// the fused loss adds `lead` to the target's column), a row can be read,
// reduced and written window packet by window packet: every access to HBM
// is an aligned packet except the element-wise stores of a row's first and last
// packet, whose other elements belong to the neighbouring rows. An aligned
// packet that holds one byte of a tensor lies in the same page as that byte, so
// reading all of it is safe at the tensor's ends too.
template <typename T>
struct RowWindow {
  static constexpr int kVec = IO<T>::kVec;
  int lead, packets, tail_valid;
  __device__ __forceinline__ RowWindow(const T* row, int C) {
    lead = static_cast<int>((reinterpret_cast<uintptr_t>(row) & 15u) / sizeof(T));
    packets = (lead + C + kVec - 1) / kVec;
    tail_valid = lead + C - (packets - 1) * kVec;  // 1 .. kVec
  }
};

// kThreads is the workgroup size; a workgroup runs kThreads / kTPR rows at a
// time. Kernels whose rows span several wavefronts and that run more than one
// row per workgroup must keep their row loop uniform across the workgroup
// (reductions contain a barrier).
template <typename T, int kTPR, int kVPT, int kThreadsT = row_threads(kTPR), bool kRagged = false>
struct RowTile {
  using A = typename IO<T>::Acc;
  static constexpr int kVec = IO<T>::kVec;
  static constexpr int kThreads = kThreadsT;
  static constexpr int kRowsPerBlock = kThreads / kTPR;
  static constexpr int kWavesPerRow = kTPR / kWaveSize;
  static constexpr int kMaxPackets = kTPR * kVPT;
  // LDS words one reduction needs (pairs need twice that).
  static constexpr int kSlots = kRowsPerBlock * kWavesPerRow;

  A v[kVPT][kVec];

  static __device__ __forceinline__ int lane() { return threadIdx.x % kTPR; }
  // kTPR is a whole number of wavefronts, so the row-group index is uniform
  // over a wavefront: reading it from the first lane keeps it, and every row
  // base address derived from it, in scalar registers.
  static __device__ __forceinline__ int sub_row() {
    return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / kTPR));
  }
  // Whether slot `slot` of this thread holds any element of the row.
  static __device__ __forceinline__ bool active(int slot, int extent) {
    return kRagged ? (slot * kTPR + lane()) * kVec < extent : slot * kTPR + lane() < extent;
  }
  // Whether element `e` of slot `slot` lies inside the row (always true for a
  // regular tile's active slot).
  static __device__ __forceinline__ bool elem_active(int slot, int e, int extent) {
    return kRagged ? (slot * kTPR + lane()) * kVec + e < extent : true;
  }
  // The extent argument of this tile flavour for a row of C elements.
  static __host__ __device__ __forceinline__ int extent_of(int C) { return kRagged ? C : C / kVec; }

  // Loads are unconditional (a masked slot reads packet 0 of the row and is
  // then overwritten with `fill`): with no branch around a load the number of
  // loads in flight is static, and the compiler can wait for exactly the ones a
  // computation needs instead of draining the queue. `row` must point to
  // readable memory even when `valid` is false.
  // Rows that fill the tile exactly (npackets == kMaxPackets): no slot is masked,
  // so no select is spent on the fill value.
  __device__ __forceinline__ void load_full(const T* row) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      load_unpack<T>(row + static_cast<int64_t>(s * kTPR + lane()) * kVec, v[s]);
    }
  }

  __device__ __forceinline__ void load(const T* row, int npackets, A fill, bool valid = true) {
    if constexpr (kRagged) {
      load_ragged(row, npackets, fill, valid);
      return;
    }
    // every packet is requested before the first one is converted and masked
    u32x4 raw[kVPT];
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const bool on = valid && active(s, npackets);
      const int packet = on ? s * kTPR + lane() : 0;
      raw[s] = load_packet(row + static_cast<int64_t>(packet) * kVec);
    }
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const bool on = valid && active(s, npackets);
      IO<T>::unpack(raw[s], v[s]);
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[s][e] = on ? v[s][e] : fill;
    }
  }

  __device__ __forceinline__ void store(T* row, int npackets, bool valid = true) const {
    if constexpr (kRagged) {
      store_ragged(row, npackets, valid);
      return;
    }
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      if (valid && active(s, npackets)) {
        pack_store<T>(row + static_cast<int64_t>(s * kTPR + lane()) * kVec, v[s]);
      }
    }
  }

  // The row through its window (regular tiles only): aligned packets, and what the
  // window's first and last packet hold of the neighbouring rows replaced by `fill`.
  // `row` is the row's own (element-aligned) address.
  __device__ __forceinline__ void load_window(const T* row, const RowWindow<T>& w, A fill,
                                              bool valid = true) {
    static_assert(!kRagged, "windows use the regular tile");
    load(row - w.lead, w.packets, fill, valid);
    const int tail_slot = (w.packets - 1) / kTPR, tail_lane = (w.packets - 1) % kTPR;
    if (w.lead > 0 && lane() == 0) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < w.lead) v[0][e] = fill;
      }
    }
    if (w.tail_valid < kVec && lane() == tail_lane) {
#pragma unroll
      for (int s = 0; s < kVPT; ++s) {
        if (s == tail_slot) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            if (e >= w.tail_valid) v[s][e] = fill;
          }
        }
      }
    }
  }
  // Whole packets of the row as aligned packets; the elements of the row in the
  // window's first and last packet one by one (the others belong to its neighbours).
  __device__ __forceinline__ void store_window(T* row, const RowWindow<T>& w,
                                               bool valid = true) const {
    static_assert(!kRagged, "windows use the regular tile");
    T* base = row - w.lead;
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int idx = s * kTPR + lane();
      if (!valid || idx >= w.packets) continue;
      const int first = idx == 0 ? w.lead : 0;
      const int last = idx == w.packets - 1 ? w.tail_valid : kVec;
      if (first == 0 && last == kVec) {
        pack_store<T>(base + static_cast<int64_t>(idx) * kVec, v[s]);
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (e >= first && e < last) IO<T>::store1(base + static_cast<int64_t>(idx) * kVec + e, v[s][e]);
        }
      }
    }
  }

  __device__ __forceinline__ void load_ragged(const T* row, int ncols, A fill, bool valid) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int col = (s * kTPR + lane()) * kVec;
      if (valid && col + kVec <= ncols) {
        IO<T>::unpack(load_packet_unaligned(row + col), v[s]);
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          v[s][e] = (valid && col + e < ncols) ? IO<T>::load1(row + col + e) : fill;
        }
      }
    }
  }

  __device__ __forceinline__ void store_ragged(T* row, int ncols, bool valid) const {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int col = (s * kTPR + lane()) * kVec;
      if (!valid) continue;
      if (col + kVec <= ncols) {
        store_packet_unaligned(row + col, IO<T>::pack(v[s]));
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (col + e < ncols) IO<T>::store1(row + col + e, v[s][e]);
        }
      }
    }
  }

  // All-reduce of one value per thread over the row's thread group. `slots`
  // holds kSlots words and must not be reused before the next barrier.
  template <typename Op>
  static __device__ __forceinline__ A reduce(A x, Op op, A* slots) {
    x = wave_allreduce(x, op);
    if (kWavesPerRow == 1) return x;
    const int wave_in_row = (threadIdx.x % kTPR) / kWaveSize;
    A* mine = slots + sub_row() * kWavesPerRow;
    if ((threadIdx.x & (kWaveSize - 1)) == 0) mine[wave_in_row] = x;
    __syncthreads();
    A r = mine[0];
#pragma unroll
    for (int i = 1; i < kWavesPerRow; ++i) r = op(r, mine[i]);
    return r;
  }

  // Sum all-reduce of two values with a single barrier; `slots` holds 2*kSlots words.
  static __device__ __forceinline__ void reduce_sum_pair(A& a, A& b, A* slots) {
    a = wave_allreduce(a, SumOp());
    b = wave_allreduce(b, SumOp());
    if (kWavesPerRow == 1) return;
    const int wave_in_row = (threadIdx.x % kTPR) / kWaveSize;
    A* mine = slots + sub_row() * kWavesPerRow * 2;
    if ((threadIdx.x & (kWaveSize - 1)) == 0) {
      mine[2 * wave_in_row] = a;
      mine[2 * wave_in_row + 1] = b;
    }
    __syncthreads();
    a = mine[0], b = mine[1];
#pragma unroll
    for (int i = 1; i < kWavesPerRow; ++i) {
      a += mine[2 * i];
      b += mine[2 * i + 1];
    }
  }
};

// The same tile kept as raw packets (four dwords each): half the registers of
// the unpacked form for 16-bit types, at the price of converting again on
// every pass over the tile. Used where several tiles are live at once or the
// next row is prefetched while the current one is processed.
template <typename T, int kTPR, int kVPT, int kThreadsT = row_threads(kTPR)>
struct RawRowTile {
  using A = typename IO<T>::Acc;
  static constexpr int kVec = IO<T>::kVec;
  u32x4 p[kVPT];

  static __device__ __forceinline__ int lane() { return threadIdx.x % kTPR; }
  static __device__ __forceinline__ bool active(int slot, int npackets) {
    return slot * kTPR + lane() < npackets;
  }
  // Inactive slots hold zero bits, i.e. +0.0 in every element type. The load
  // itself is unconditional (see RowTile::load); `row` must be readable even
  // when `valid` is false.
  __device__ __forceinline__ void load(const T* row, int npackets, bool valid = true) {
    // every packet is requested before the first one is masked
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const bool on = valid && active(s, npackets);
      const int packet = on ? s * kTPR + lane() : 0;
      p[s] = load_packet(row + static_cast<int64_t>(packet) * kVec);
    }
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const bool on = valid && active(s, npackets);
      const u32x4 z = {0u, 0u, 0u, 0u};
      p[s] = on ? p[s] : z;
    }
  }
  // Rows of any width at element-aligned addresses, read in whole (unaligned)
  // packets: the row's last packet may reach up to kVec - 1 elements past the
  // row, so the caller guarantees that those are readable (another row follows)
  // and masks them itself.
  __device__ __forceinline__ void load_over(const T* row, int ncols, bool valid = true) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int col = (s * kTPR + lane()) * kVec;
      const bool on = valid && col < ncols;
      const u32x4 t = load_packet_unaligned(row + (on ? col : 0));
      const u32x4 z = {0u, 0u, 0u, 0u};
      p[s] = on ? t : z;
    }
  }
  // load() without the zero fill: inactive slots (and every slot when `valid`
  // is false) hold packet 0 of `row`, for kernels that mask at the point of use.
  __device__ __forceinline__ void load_unmasked(const T* row, int npackets) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int packet = active(s, npackets) ? s * kTPR + lane() : 0;
      p[s] = load_packet(row + static_cast<int64_t>(packet) * kVec);
    }
  }
  // One slot of load_unmasked(): a slot beyond the row holds the row's first
  // packet, and no select touches the loaded registers (a select would wait
  // for the load where it stands, which defeats a request made ahead of use).
  __device__ __forceinline__ void load_slot_unmasked(const T* row, int s, int npackets) {
    const int packet = active(s, npackets) ? s * kTPR + lane() : 0;
    p[s] = load_packet(row + static_cast<int64_t>(packet) * kVec);
  }
  // Rows of any width at element-aligned addresses: whole packets with one
  // unaligned access, the row's last partial packet element by element.
  // Elements beyond the row hold zero bits.
  __device__ __forceinline__ void load_any(const T* row, int ncols, bool valid = true) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      const int col = (s * kTPR + lane()) * kVec;
      const u32x4 z = {0u, 0u, 0u, 0u};
      if (valid && col + kVec <= ncols) {
        p[s] = load_packet_unaligned(row + col);
      } else if (valid && col < ncols) {
        A v[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = col + e < ncols ? IO<T>::load1(row + col + e) : A(0);
        p[s] = IO<T>::pack(v);
      } else {
        p[s] = z;
      }
    }
  }
  __device__ __forceinline__ void unpack(int s, A (&v)[kVec]) const { IO<T>::unpack(p[s], v); }
  // Called between two passes over the tile: makes the compiler treat the
  // packets as new values, so it converts them again in the next pass instead
  // of keeping every converted element of the previous pass in registers.
  __device__ __forceinline__ void refresh() {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) asm volatile("" : "+v"(p[s]));
  }
  // For a prefetched tile: pins the point where its loads must have landed.
  // Placed after the current row's arithmetic and before the current row's
  // stores, it makes the wait cover only loads (and the previous row's, by
  // then old, stores), so the new stores stay in flight across the next row.
  __device__ __forceinline__ void wait_ready() {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) asm volatile("" : "+v"(p[s])::"memory");
  }
  __device__ __forceinline__ void store_slot(T* row, int s, const A (&v)[kVec]) const {
    pack_store<T>(row + static_cast<int64_t>(s * kTPR + lane()) * kVec, v);
  }
};

// How many neighbouring rows a forward row kernel holds per thread group at a
// time. A wavefront that holds a whole row in one or two packets per lane takes
// two: the dependent cross-lane reduction steps of the two rows interleave
// instead of each waiting out the latency of the one before, and twice the
// loads are in flight per wavefront.
template <int kTPR, int kVPT>
constexpr int wave_rows_at_a_time() {
  return kTPR == kWaveSize && kVPT <= 2 ? 2 : 1;
}

// Picks the tile for a row of `npackets` packets: the fewest threads per row
// whose tile still holds it, because short rows on few threads leave many rows
// in flight per compute unit (wave-per-row up to 4 packets per lane, then a
// 256-thread workgroup, then 1024 threads). `max_vpt` bounds the packets a
// thread of a multi-wave tile may hold (kernels with two live tiles pass 4).
// Returns false when the row is too long for registers.
struct RowConfig {
  int tpr, vpt;
};
inline bool pick_row_config(int64_t npackets, int max_vpt, RowConfig* cfg) {
  static const RowConfig table[] = {{64, 1},  {64, 2},  {64, 4},   {256, 2},  {256, 4},
                                    {256, 8}, {1024, 2}, {1024, 4}, {1024, 8}};
  for (const RowConfig& c : table) {
    if (c.vpt > max_vpt) continue;
    if (npackets <= static_cast<int64_t>(c.tpr) * c.vpt) {
      *cfg = c;
      return true;
    }
  }
  return false;
}

// Instantiates LAUNCH(tpr, vpt) for the tile pick_row_config chose.
#define DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH)                  \
  if (cfg.tpr == 64 && cfg.vpt == 1) LAUNCH(64, 1)          \
  else if (cfg.tpr == 64 && cfg.vpt == 2) LAUNCH(64, 2)     \
  else if (cfg.tpr == 64 && cfg.vpt == 4) LAUNCH(64, 4)     \
  else if (cfg.tpr == 256 && cfg.vpt == 2) LAUNCH(256, 2)   \
  else if (cfg.tpr == 256 && cfg.vpt == 4) LAUNCH(256, 4)   \
  else if (cfg.tpr == 256 && cfg.vpt == 8) LAUNCH(256, 8)   \
  else if (cfg.tpr == 1024 && cfg.vpt == 2) LAUNCH(1024, 2) \
  else if (cfg.tpr == 1024 && cfg.vpt == 4) LAUNCH(1024, 4) \
  else LAUNCH(1024, 8)

// Workgroups of `kernel` (block size `threads`, `dynamic_lds` bytes of dynamic
// LDS) that can be resident on the whole device at once: the grid of a
// persistent kernel. Also raises the kernel's dynamic-LDS limit when needed.
// The answer is cached per (device, kernel, LDS size): the queries cost
// microseconds of host time, and a launch path that a caller captures into a
// graph should not depend on them after its first use.
template <typename Kernel>
inline unsigned resident_grid(Kernel kernel, int threads, size_t dynamic_lds) {
  struct Key {
    int device;
    const void* fn;
    size_t lds;
    bool operator<(const Key& o) const {
      return std::tie(device, fn, lds) < std::tie(o.device, o.fn, o.lds);
    }
  };
  static std::mutex lock;
  static std::map<Key, unsigned> cache;
  static std::map<Key, size_t> lds_limit;  // per (device, kernel): the limit set so far
  int device = 0;
  (void)hipGetDevice(&device);
  const void* fn = reinterpret_cast<const void*>(kernel);
  const Key key{device, fn, dynamic_lds};
  {
    std::lock_guard<std::mutex> guard(lock);
    const auto hit = cache.find(key);
    if (hit != cache.end()) return hit->second;
    size_t& limit = lds_limit[Key{device, fn, 0}];
    if (dynamic_lds > 48 * 1024 && dynamic_lds > limit) {  // only ever raised
      (void)hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                static_cast<int>(dynamic_lds));
      limit = dynamic_lds;
    }
  }
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, dynamic_lds) !=
          hipSuccess ||
      per_cu < 1) {
    (void)hipGetLastError();
    per_cu = 1;
  }
  const unsigned grid = static_cast<unsigned>(per_cu) * num_cus();
  std::lock_guard<std::mutex> guard(lock);
  cache[key] = grid;
  return grid;
}

// LDS a workgroup may use for staged parameters (of 160 KB per compute unit).
constexpr size_t kMaxStagedParamBytes = 144 * 1024;

// Workgroups for a row kernel: enough to cover every row once, capped so a
// grid-stride loop picks up the rest.
inline unsigned row_grid(int64_t rows, int rows_per_block) {
  const int64_t want = ceil_div(rows, rows_per_block);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 2048;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

} // namespace dragon_hip
