// Rows too long for the register tiles: a 1024-thread workgroup walks one row
// in 16-byte packets, several passes per row. Only the first pass reads HBM;
// a row of a few hundred KB stays in the 4 MB L2 of its XCD for the later
// ones. Packets are counted from the row's first element and may be
// element-aligned only; the row's last packet may be partial.
#pragma once

#include "common.h"

namespace dragon_hip {

constexpr int kLoopThreads = 1024;
constexpr int kLoopWaves = kLoopThreads / kWaveSize;

template <typename T>
struct RowLoop {
  using A = typename IO<T>::Acc;
  static constexpr int kVec = IO<T>::kVec;

  // f(col, v, n): kVec values starting at column `col`, of which the first n
  // are inside the row (the others hold `fill`).
  template <typename F>
  static __device__ __forceinline__ void visit(const T* row, int64_t C, A fill, F&& f) {
    const int64_t full = C / kVec;
#pragma unroll 4
    for (int64_t p = threadIdx.x; p < full; p += kLoopThreads) {
      A v[kVec];
      IO<T>::unpack(load_packet_unaligned(row + p * kVec), v);
      f(p * kVec, v, kVec);
    }
    const int tail = static_cast<int>(C - full * kVec);
    if (tail > 0 && full % kLoopThreads == threadIdx.x) {
      A v[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = e < tail ? IO<T>::load1(row + full * kVec + e) : fill;
      f(full * kVec, v, tail);
    }
  }

  // Two rows of the same shape walked together: f(col, a, b, n).
  template <typename F>
  static __device__ __forceinline__ void visit2(const T* row_a, const T* row_b, int64_t C, A fill,
                                                F&& f) {
    const int64_t full = C / kVec;
#pragma unroll 4
    for (int64_t p = threadIdx.x; p < full; p += kLoopThreads) {
      A a[kVec], b[kVec];
      IO<T>::unpack(load_packet_unaligned(row_a + p * kVec), a);
      IO<T>::unpack(load_packet_unaligned(row_b + p * kVec), b);
      f(p * kVec, a, b, kVec);
    }
    const int tail = static_cast<int>(C - full * kVec);
    if (tail > 0 && full % kLoopThreads == threadIdx.x) {
      A a[kVec], b[kVec];
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        a[e] = e < tail ? IO<T>::load1(row_a + full * kVec + e) : fill;
        b[e] = e < tail ? IO<T>::load1(row_b + full * kVec + e) : fill;
      }
      f(full * kVec, a, b, tail);
    }
  }

  // Writes the first n of kVec values at column `col` of `row`.
  static __device__ __forceinline__ void store(T* row, int64_t col, const A (&v)[kVec], int n) {
    if (n == kVec) {
      store_packet_unaligned(row + col, IO<T>::pack(v));
    } else {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < n) IO<T>::store1(row + col + e, v[e]);
      }
    }
  }
};

// Workgroups of a looped row kernel: one per row, capped at a few per compute unit.
inline unsigned loop_grid(int64_t rows) {
  const int64_t cap = static_cast<int64_t>(num_cus()) * 2;
  return static_cast<unsigned>(rows < cap ? (rows > 0 ? rows : 1) : cap);
}

} // namespace dragon_hip
