// Register tiles for reductions along a strided axis: a tensor viewed as
// [N, C, S] is reduced along C with S > 1 (channel softmax of an NCHW tensor,
// L2 normalisation across channels).
//
// A 256-thread workgroup owns a tile of all C rows by kTW * kVec adjacent
// columns of one n. Thread (tc, tw) holds the 16-byte packet of columns
// [tw * kVec, (tw + 1) * kVec) of the rows c = tc, tc + kTC, tc + 2 kTC, ...
// (kTC = 256 / kTW rows in flight, up to kR packets per thread), as raw packets.
// Every tensor is therefore read from HBM once; a row segment of the tile is
// kTW * 16 contiguous bytes (1 KiB for kTW = 64, 64 bytes for kTW = 4).
//
//   kTW = 64   C <= 4 * kR     (kR = 16: 64)     widest segments, few channels
//   kTW = 16   C <= 16 * kR    (256)
//   kTW = 4    C <= 64 * kR    (1024)            many channels, narrow segments
//
// Per-column reductions over the kTC threads of a column group go through
// wave shuffles (threads of one wavefront) and one LDS exchange (its four
// wavefronts). Rows sit at arbitrary element-aligned addresses (S need not be
// a multiple of a packet); the last packet of a row may be partial.
#pragma once

#include "common.h"

namespace dragon_hip {

constexpr int kColThreads = 256;

template <typename T, int kTW, int kR>
struct ColTile {
  using A = typename IO<T>::Acc;
  static constexpr int kVec = IO<T>::kVec;
  static constexpr int kTC = kColThreads / kTW;
  static constexpr int kCols = kTW * kVec;   // columns per tile
  static constexpr int kMaxC = kTC * kR;     // rows a tile can hold
  static constexpr int kLdsWords = 4 * kTW * kVec;  // one reduction's exchange

  u32x4 p[kR];

  static __device__ __forceinline__ int tw() { return threadIdx.x % kTW; }
  static __device__ __forceinline__ int tc() { return threadIdx.x / kTW; }

  // base = first element of row c = 0 at this thread's first column; nvalid =
  // how many of the thread's kVec columns exist (0 .. kVec).
  __device__ __forceinline__ void load(const T* base, int64_t S, int C, int nvalid, A fill) {
    A f[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) f[e] = fill;
    const u32x4 fill_bits = IO<T>::pack(f);
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      const int c = r * kTC + tc();
      if (c < C && nvalid == kVec) {
        p[r] = load_packet_unaligned(base + c * S);
      } else if (c < C && nvalid > 0) {
        A v[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e) v[e] = e < nvalid ? IO<T>::load1(base + c * S + e) : fill;
        p[r] = IO<T>::pack(v);
      } else {
        p[r] = fill_bits;
      }
    }
  }

  __device__ __forceinline__ void unpack(int r, A (&v)[kVec]) const { IO<T>::unpack(p[r], v); }
  __device__ __forceinline__ void set(int r, const A (&v)[kVec]) { p[r] = IO<T>::pack(v); }
  // Between two passes over the tile: makes the compiler convert the packets
  // again in the next pass instead of keeping every converted element live.
  __device__ __forceinline__ void refresh() {
#pragma unroll
    for (int r = 0; r < kR; ++r) asm volatile("" : "+v"(p[r]));
  }
  // Packets per thread that hold rows of a C-row tensor (the others are padding).
  static __device__ __forceinline__ int rows_used(int C) { return (C + kTC - 1) / kTC; }

  static __device__ __forceinline__ void store(T* base, int64_t S, int C, int nvalid, int r,
                                               const A (&v)[kVec]) {
    const int c = r * kTC + tc();
    if (c >= C || nvalid <= 0) return;
    if (nvalid == kVec) {
      store_packet_unaligned(base + c * S, IO<T>::pack(v));
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < nvalid) IO<T>::store1(base + c * S + e, v[e]);
      }
    }
  }

  // All-reduce of kVec per-column values over the kTC threads that share this
  // thread's columns. `lds` holds kLdsWords words; a barrier separates two uses.
  template <typename Op>
  static __device__ __forceinline__ void reduce_rows(A (&v)[kVec], Op op, A* lds) {
#pragma unroll
    for (int o = kTW; o < kWaveSize; o <<= 1) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = op(v[e], __shfl_xor(v[e], o, kWaveSize));
    }
    const int wave = threadIdx.x / kWaveSize;
    const int lane = threadIdx.x & (kWaveSize - 1);
    __syncthreads();  // the previous use of lds is over
    if (lane < kTW) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) lds[(wave * kTW + lane) * kVec + e] = v[e];
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      const A a = lds[(0 * kTW + tw()) * kVec + e], b = lds[(1 * kTW + tw()) * kVec + e];
      const A c = lds[(2 * kTW + tw()) * kVec + e], d = lds[(3 * kTW + tw()) * kVec + e];
      v[e] = op(op(a, b), op(c, d));
    }
  }
};

// Tile geometry shared by the kernels: tile index -> (n, first column).
struct ColGrid {
  int64_t N, S;
  int C;
  int64_t strips;  // tiles per n
  int64_t tiles;
};
inline ColGrid make_col_grid(int64_t N, int64_t S, int64_t C, int cols_per_tile) {
  ColGrid g;
  g.N = N, g.S = S, g.C = static_cast<int>(C);
  g.strips = ceil_div(S, cols_per_tile);
  g.tiles = N * g.strips;
  return g;
}

// Threads along the columns for a strided reduction over C rows of S columns
// with at most `max_r` packets per thread: the widest tile that still holds C
// rows, not wider than the columns there are. 0 when no tile can hold C rows.
inline int pick_col_tw(int64_t N, int64_t C, int64_t S, int vec, int max_r) {
  // A tile never spans two n: where one n holds a few hundred elements at most
  // (a handful of classes over a handful of positions), a workgroup per n is
  // mostly idle and a thread per column does better. The same where S is less
  // than a packet (most of a tile's lanes along S have no column) and there are
  // enough columns in all to fill the device with a thread each.
  if (C * S <= 512) return 0;
  if (S < vec && C <= 256 && N * S >= 16384) return 0;
  const int64_t packets = ceil_div(S, vec);
  const int tw_cap = packets > 16 ? 64 : (packets > 4 ? 16 : 4);
  for (int tw : {64, 16, 4}) {
    if (tw > tw_cap) continue;
    if (C <= static_cast<int64_t>(kColThreads / tw) * max_r) return tw;
  }
  return 0;
}

inline unsigned col_launch_grid(int64_t tiles) {
  const int64_t cap = static_cast<int64_t>(num_cus()) * 64;
  return static_cast<unsigned>(tiles < cap ? (tiles > 0 ? tiles : 1) : cap);
}

} // namespace dragon_hip
