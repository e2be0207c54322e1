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
#pragma once

#include "common.h"

namespace dragon_hip {

// Workgroup size of a row kernel: wave-per-row tiles share a 256-thread group.
constexpr int row_threads(int tpr) { return tpr == kWaveSize ? 256 : tpr; }

// kThreads is the workgroup size; a workgroup runs kThreads / kTPR rows at a
// time. Kernels whose rows span several wavefronts and that run more than one
// row per workgroup must keep their row loop uniform across the workgroup
// (reductions contain a barrier).
template <typename T, int kTPR, int kVPT, int kThreadsT = row_threads(kTPR)>
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
  static __device__ __forceinline__ int sub_row() { return threadIdx.x / kTPR; }
  static __device__ __forceinline__ bool active(int slot, int npackets) {
    return slot * kTPR + lane() < npackets;
  }

  __device__ __forceinline__ void load(const T* row, int npackets, A fill, bool valid = true) {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      if (valid && active(s, npackets)) {
        IO<T>::load(row + static_cast<int64_t>(s * kTPR + lane()) * kVec, v[s]);
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[s][e] = fill;
      }
    }
  }

  __device__ __forceinline__ void store(T* row, int npackets, bool valid = true) const {
#pragma unroll
    for (int s = 0; s < kVPT; ++s) {
      if (valid && active(s, npackets)) {
        IO<T>::store(row + static_cast<int64_t>(s * kTPR + lane()) * kVec, v[s]);
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

// Picks the smallest tile that holds `npackets` packets. Returns false when
// the row is too long for registers (the caller then uses its looping kernel).
// Order: wave-per-row while a lane holds at most 4 packets, then a 256-thread
// workgroup, then 1024 threads.
struct RowConfig {
  int tpr, vpt;
};
inline bool pick_row_config(int64_t npackets, RowConfig* cfg) {
  static const RowConfig table[] = {{64, 1},  {64, 2},  {64, 4},   {256, 2},
                                    {256, 4}, {1024, 2}, {1024, 4}, {1024, 8}};
  for (const RowConfig& c : table) {
    if (npackets <= static_cast<int64_t>(c.tpr) * c.vpt) {
      *cfg = c;
      return true;
    }
  }
  return false;
}

// Instantiates LAUNCH(T, tpr, vpt) for the tile pick_row_config chose.
#define DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH)                 \
  if (cfg.tpr == 64 && cfg.vpt == 1) LAUNCH(64, 1)         \
  else if (cfg.tpr == 64 && cfg.vpt == 2) LAUNCH(64, 2)    \
  else if (cfg.tpr == 64 && cfg.vpt == 4) LAUNCH(64, 4)    \
  else if (cfg.tpr == 256 && cfg.vpt == 2) LAUNCH(256, 2)  \
  else if (cfg.tpr == 256 && cfg.vpt == 4) LAUNCH(256, 4)  \
  else if (cfg.tpr == 1024 && cfg.vpt == 2) LAUNCH(1024, 2) \
  else if (cfg.tpr == 1024 && cfg.vpt == 4) LAUNCH(1024, 4) \
  else LAUNCH(1024, 8)

// Workgroups for a row kernel: enough to cover every row once, capped so a
// grid-stride loop picks up the rest.
inline unsigned row_grid(int64_t rows, int rows_per_block) {
  const int64_t want = ceil_div(rows, rows_per_block);
  const int64_t cap = static_cast<int64_t>(kNumCUs) * 2048;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

} // namespace dragon_hip
