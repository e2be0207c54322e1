// Rows of any length at element-aligned addresses, one wavefront per row:
// NCHW feature maps whose S elements are not whole 16-byte packets and are too
// long for the LDS-staged short-row kernel (35x35, 71x71, 147x147 maps). A
// row's first elements up to a 16-byte boundary and its last ones past the
// final whole packet are moved element by element, everything between as
// aligned packets. The tensors must be congruent modulo 16 bytes, so that one
// split serves all of them.
//
// Op provides
//   static constexpr int kParams          per-row scalars
//   void row_params(int64_t row, A (&w)[kParams]) const
//   void add(const A* w, A x0, A x1, A& a, A& b) const      (long_rows_sums)
//   A apply(const A* w, A x0, A x1) const                   (long_rows_map)
#pragma once

#include "common.h"
#include "row_tile.h"

namespace dragon_hip {

constexpr int kLongThreads = 256;  // four rows at a time per workgroup

struct LongRowSplit {
  int head, body;  // leading elements, then whole packets; the rest is the tail
  template <typename T>
  __device__ __forceinline__ LongRowSplit(const T* row, int S) {
    constexpr int kVec = IO<T>::kVec;
    const int lead = static_cast<int>(
        ((16u - static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row) & 15u)) & 15u) / sizeof(T));
    head = lead < S ? lead : S;
    body = (S - head) / kVec;
  }
};

inline unsigned long_rows_grid(int64_t rows) {
  const int64_t want = ceil_div(rows, kLongThreads / kWaveSize);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 16;
  return static_cast<unsigned>(want < cap ? want : cap);
}

// pairs[2 * row + {0, 1}] = the row's (a, b).
template <typename T, int kIn, typename Op>
__global__ __launch_bounds__(kLongThreads) void long_rows_sums(
    const int64_t rows, const int S, const T* __restrict__ in0, const T* __restrict__ in1,
    const Op op, typename IO<T>::Acc* __restrict__ pairs) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kWaves = kLongThreads / kWaveSize;
  const int lane = threadIdx.x & (kWaveSize - 1);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWaveSize; row < rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    A w[Op::kParams];
    op.row_params(row, w);
    const T* r0 = in0 + row * S;
    const T* r1 = in1 + row * S;
    const LongRowSplit sp(r0, S);
    A a = A(0), b = A(0);
    if (lane < sp.head) {
      op.add(w, IO<T>::load1(r0 + lane), kIn == 2 ? IO<T>::load1(r1 + lane) : A(0), a, b);
    }
#pragma unroll 4
    for (int p = lane; p < sp.body; p += kWaveSize) {
      A x0[kVec], x1[kVec];
      load_unpack_keep<T>(r0 + sp.head + p * kVec, x0);
      if constexpr (kIn == 2) load_unpack_keep<T>(r1 + sp.head + p * kVec, x1);
#pragma unroll
      for (int e = 0; e < kVec; ++e) op.add(w, x0[e], kIn == 2 ? x1[e] : A(0), a, b);
    }
    const int t = sp.head + sp.body * kVec + lane;  // fewer than kVec elements remain
    if (t < S) op.add(w, IO<T>::load1(r0 + t), kIn == 2 ? IO<T>::load1(r1 + t) : A(0), a, b);
    a = wave_allreduce(a, SumOp());
    b = wave_allreduce(b, SumOp());
    if (lane == 0) {
      pairs[2 * row] = a;
      pairs[2 * row + 1] = b;
    }
  }
}

// out = op.apply(row's scalars, in0, in1), element by element.
template <typename T, int kIn, typename Op>
__global__ __launch_bounds__(kLongThreads) void long_rows_map(
    const int64_t rows, const int S, const T* in0, const T* in1, T* out, const Op op) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kWaves = kLongThreads / kWaveSize;
  const int lane = threadIdx.x & (kWaveSize - 1);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWaveSize; row < rows;
       row += static_cast<int64_t>(gridDim.x) * kWaves) {
    A w[Op::kParams];
    op.row_params(row, w);
    const T* r0 = in0 + row * S;
    const T* r1 = in1 + row * S;
    T* ro = out + row * S;
    const LongRowSplit sp(r0, S);
    if (lane < sp.head) {
      const A v = op.apply(w, IO<T>::load1(r0 + lane), kIn == 2 ? IO<T>::load1(r1 + lane) : A(0));
      IO<T>::store1(ro + lane, v);
    }
#pragma unroll 4
    for (int p = lane; p < sp.body; p += kWaveSize) {
      A x0[kVec], x1[kVec];
      load_unpack<T>(r0 + sp.head + p * kVec, x0);
      if constexpr (kIn == 2) load_unpack<T>(r1 + sp.head + p * kVec, x1);
#pragma unroll
      for (int e = 0; e < kVec; ++e) x0[e] = op.apply(w, x0[e], kIn == 2 ? x1[e] : A(0));
      pack_store<T>(ro + sp.head + p * kVec, x0);
    }
    const int t = sp.head + sp.body * kVec + lane;
    if (t < S) {
      const A v = op.apply(w, IO<T>::load1(r0 + t), kIn == 2 ? IO<T>::load1(r1 + t) : A(0));
      IO<T>::store1(ro + t, v);
    }
  }
}

} // namespace dragon_hip
