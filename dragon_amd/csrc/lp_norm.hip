// L1Norm / L2Norm forward and backward for gfx950.
//
// Replaces kernels::L1Norm, L2Norm, L1NormGrad, L2NormGrad
// (dragon/kernels/normalization/op_kernels.h:145-189; CPU
// dragon/kernels/normalization/cpu/lp_norm_kernel.cc:10-101, CUDA
// dragon/kernels/normalization/cuda/lp_norm_kernel.cu:11-134) over a tensor
// viewed as [N, C, S] with the reduction along C:
//   p = 1   norm = max(sum |x| / normalizer, eps)
//   p = 2   norm = max(sqrt(sum x^2 / normalizer), eps)
//   forward     y  = x / norm
//   backward    dx = dy / norm - g(x) * (sum(dy * x) / normalizer) / norm^(p+1)
//               with g(x) = sign(x) for p = 1 and g(x) = x for p = 2
//
// S == 1 keeps each row in registers (one read, one write per tensor), with
// the same tiles as the softmax kernels. S > 1 keeps a [C, columns] tile in
// the registers of a workgroup (col_tile.h) when C <= 1024; beyond that each
// thread owns a strip of adjacent (n, s) columns one 16-byte packet wide and
// walks it twice (reduce, write), the second walk re-reading what the first
// left in L2.
//
// 16-bit I/O accumulates in fp32 as the reference's CUDA kernels do; fp32 and
// fp64 I/O divide by the norm exactly as the reference's CPU expression does,
// 16-bit I/O multiplies by its reciprocal (error far below one 16-bit ulp).
#include "col_tile.h"
#include "row_loop.h"
#include "row_tile.h"
#include "short_rows.h"

namespace dragon_hip {
namespace {

template <typename A>
__device__ __forceinline__ A acc_sign(A v) {
  return A((A(0) < v) - (v < A(0)));
}
__device__ __forceinline__ float acc_abs(float v) { return __builtin_fabsf(v); }
__device__ __forceinline__ double acc_abs(double v) { return __builtin_fabs(v); }
__device__ __forceinline__ float acc_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double acc_sqrt(double v) { return sqrt(v); }

template <typename T, int kP>
struct LpMath {
  using A = typename IO<T>::Acc;
  static constexpr bool kFast = sizeof(T) == 2;
  static __device__ __forceinline__ A term(A v) { return kP == 1 ? acc_abs(v) : v * v; }
  static __device__ __forceinline__ A norm_of(A acc, A normalizer, A eps) {
    A n = acc / normalizer;
    if (kP == 2) n = acc_sqrt(n);
    return n > eps ? n : eps;
  }
  static __device__ __forceinline__ A forward(A x, A norm, A inv_norm) {
    if constexpr (kFast) {
      return x * inv_norm;
    } else {
      return x / norm;
    }
  }
  // coef = (sum(dy * x) / normalizer) / norm^(p+1)
  static __device__ __forceinline__ A coef_of(A dot, A normalizer, A norm) {
    const A powed = kP == 1 ? norm * norm : norm * norm * norm;
    return (dot / normalizer) / powed;
  }
  static __device__ __forceinline__ A backward(A dy, A x, A norm, A inv_norm, A coef) {
    const A g = kP == 1 ? acc_sign(x) : x;
    if constexpr (kFast) {
      return dy * inv_norm - g * coef;
    } else {
      return dy / norm - g * coef;
    }
  }
};

template <typename T, int kP, int kTPR, int kVPT, bool kRagged>
__global__ __launch_bounds__(row_threads(kTPR)) void lp_norm_rows(
    const int64_t N, const int C, const typename IO<T>::Acc normalizer,
    const typename IO<T>::Acc eps, const T* x, T* y) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  using M = LpMath<T, kP>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[Tile::kSlots];
  const int npackets = Tile::extent_of(C);

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < N; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile t;
    t.load(x + row * C, npackets, A(0));
    A acc = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) acc += M::term(t.v[i][e]);
    acc = Tile::reduce(acc, SumOp(), slots);
    const A norm = M::norm_of(acc, normalizer, eps);
    const A inv = A(1) / norm;
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) t.v[i][e] = M::forward(t.v[i][e], norm, inv);
    t.store(y + row * C, npackets);
    if (kTPR != kWaveSize) __syncthreads();
  }
}

template <typename T, int kP, int kTPR, int kVPT, bool kRagged>
__global__ __launch_bounds__(row_threads(kTPR)) void lp_norm_grad_rows(
    const int64_t N, const int C, const typename IO<T>::Acc normalizer,
    const typename IO<T>::Acc eps, const T* dy, const T* x, T* dx) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  using M = LpMath<T, kP>;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2 * Tile::kSlots];
  const int npackets = Tile::extent_of(C);

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < N; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile g, t;
    g.load(dy + row * C, npackets, A(0));
    t.load(x + row * C, npackets, A(0));
    A acc = A(0), dot = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        acc += M::term(t.v[i][e]);
        dot += g.v[i][e] * t.v[i][e];
      }
    Tile::reduce_sum_pair(acc, dot, slots);
    const A norm = M::norm_of(acc, normalizer, eps);
    const A inv = A(1) / norm;
    const A coef = M::coef_of(dot, normalizer, norm);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e)
        g.v[i][e] = M::backward(g.v[i][e], t.v[i][e], norm, inv, coef);
    g.store(dx + row * C, npackets);
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// S == 1 rows too long for the register tiles: two passes per row.
template <typename T, int kP, bool kGrad>
__global__ __launch_bounds__(kLoopThreads) void lp_norm_rows_looped(
    const int64_t N, const int64_t C, const typename IO<T>::Acc normalizer,
    const typename IO<T>::Acc eps, const T* dy, const T* x, T* out) {
  using A = typename IO<T>::Acc;
  using M = LpMath<T, kP>;
  using Loop = RowLoop<T>;
  constexpr int kVec = Loop::kVec;
  __shared__ A slots[2][kLoopWaves];
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const T* xr = x + row * C;
    const T* gr = kGrad ? dy + row * C : xr;
    T* outr = out + row * C;
    A acc = A(0), dot = A(0);
    if constexpr (kGrad) {
      Loop::visit2(gr, xr, C, A(0), [&](int64_t, const A(&g)[kVec], const A(&v)[kVec], int) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          acc += M::term(v[e]);
          dot += g[e] * v[e];
        }
      });
    } else {
      Loop::visit(xr, C, A(0), [&](int64_t, const A(&v)[kVec], int) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) acc += M::term(v[e]);
      });
    }
    acc = block_allreduce<kLoopWaves>(acc, SumOp(), slots[0]);
    if (kGrad) dot = block_allreduce<kLoopWaves>(dot, SumOp(), slots[1]);
    const A norm = M::norm_of(acc, normalizer, eps);
    const A inv = A(1) / norm;
    const A coef = kGrad ? M::coef_of(dot, normalizer, norm) : A(0);
    if constexpr (kGrad) {
      Loop::visit2(gr, xr, C, A(0), [&](int64_t col, const A(&g)[kVec], const A(&v)[kVec], int n) {
        A o[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e) o[e] = M::backward(g[e], v[e], norm, inv, coef);
        Loop::store(outr, col, o, n);
      });
    } else {
      Loop::visit(xr, C, A(0), [&](int64_t col, const A(&v)[kVec], int n) {
        A o[kVec];
#pragma unroll
        for (int e = 0; e < kVec; ++e) o[e] = M::forward(v[e], norm, inv);
        Loop::store(outr, col, o, n);
      });
    }
    __syncthreads();  // slots are reused by the next row
  }
}

// S > 1 with the whole reduced axis in one register tile (col_tile.h): one
// read of every tensor.
template <typename T, int kP, bool kGrad, int kTW, int kR>
__global__ __launch_bounds__(kColThreads) void lp_norm_col_tiles(
    const ColGrid g, const typename IO<T>::Acc normalizer, const typename IO<T>::Acc eps,
    const T* dy, const T* x, T* out) {
  using Tile = ColTile<T, kTW, kR>;
  using A = typename Tile::A;
  using M = LpMath<T, kP>;
  constexpr int kVec = Tile::kVec;
  __shared__ A lds[Tile::kLdsWords];
  const int nr = Tile::rows_used(g.C);  // uniform: later packets are padding
  for (int64_t tile = blockIdx.x; tile < g.tiles; tile += gridDim.x) {
    const int64_t n = tile / g.strips;
    const int64_t s0 = (tile - n * g.strips) * Tile::kCols + Tile::tw() * kVec;
    const int64_t left = g.S - s0;
    const int nvalid = left >= kVec ? kVec : (left > 0 ? static_cast<int>(left) : 0);
    const int64_t base = n * g.C * g.S + (nvalid > 0 ? s0 : 0);
    Tile tx, tg;
    tx.load(x + base, g.S, g.C, nvalid, A(0));
    if (kGrad) tg.load(dy + base, g.S, g.C, nvalid, A(0));
    A acc[kVec], dot[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) acc[e] = dot[e] = A(0);
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A v[kVec], gv[kVec];
        tx.unpack(r, v);
        if (kGrad) tg.unpack(r, gv);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          acc[e] += M::term(v[e]);
          if (kGrad) dot[e] += gv[e] * v[e];
        }
      }
    }
    Tile::reduce_rows(acc, SumOp(), lds);
    if (kGrad) Tile::reduce_rows(dot, SumOp(), lds);
    tx.refresh();
    if (kGrad) tg.refresh();
    A norm[kVec], inv[kVec], coef[kVec];
#pragma unroll
    for (int e = 0; e < kVec; ++e) {
      norm[e] = M::norm_of(acc[e], normalizer, eps);
      inv[e] = A(1) / norm[e];
      coef[e] = kGrad ? M::coef_of(dot[e], normalizer, norm[e]) : A(0);
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      if (r < nr) {
        A v[kVec], gv[kVec];
        tx.unpack(r, v);
        if (kGrad) tg.unpack(r, gv);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          v[e] = kGrad ? M::backward(gv[e], v[e], norm[e], inv[e], coef[e])
                       : M::forward(v[e], norm[e], inv[e]);
        }
        Tile::store(out + base, g.S, g.C, nvalid, r, v);
      }
    }
  }
}

// Reduction along a strided axis: a thread owns kW adjacent columns of one n
// (kW = 1, or one 16-byte packet when S is a multiple of it and the tensors are
// aligned) and walks its C elements S apart.
template <typename T, int kP, bool kGrad, int kW>
__global__ __launch_bounds__(256) void lp_norm_columns(
    const int64_t N, const int64_t S, const int64_t C, const typename IO<T>::Acc normalizer,
    const typename IO<T>::Acc eps, const T* dy, const T* x, T* out) {
  using A = typename IO<T>::Acc;
  using M = LpMath<T, kP>;
  const int64_t strips = S / kW;
  const int64_t total = N * strips;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t base = (i / strips) * C * S + (i % strips) * kW;
    A acc[kW], dot[kW];
#pragma unroll
    for (int e = 0; e < kW; ++e) acc[e] = dot[e] = A(0);
    for (int64_t k = 0; k < C; ++k) {
      A v[kW], g[kW];
      if constexpr (kW == 1) {
        v[0] = IO<T>::load1(x + base + k * S);
        if (kGrad) g[0] = IO<T>::load1(dy + base + k * S);
      } else {
        load_unpack_keep<T>(x + base + k * S, v);
        if (kGrad) load_unpack_keep<T>(dy + base + k * S, g);
      }
#pragma unroll
      for (int e = 0; e < kW; ++e) {
        acc[e] += M::term(v[e]);
        if (kGrad) dot[e] += g[e] * v[e];
      }
    }
    A norm[kW], inv[kW], coef[kW];
#pragma unroll
    for (int e = 0; e < kW; ++e) {
      norm[e] = M::norm_of(acc[e], normalizer, eps);
      inv[e] = A(1) / norm[e];
      coef[e] = kGrad ? M::coef_of(dot[e], normalizer, norm[e]) : A(0);
    }
    for (int64_t k = 0; k < C; ++k) {
      A v[kW], g[kW];
      if constexpr (kW == 1) {
        v[0] = IO<T>::load1(x + base + k * S);
        if (kGrad) g[0] = IO<T>::load1(dy + base + k * S);
      } else {
        load_unpack<T>(x + base + k * S, v);
        if (kGrad) load_unpack<T>(dy + base + k * S, g);
      }
#pragma unroll
      for (int e = 0; e < kW; ++e) {
        v[e] = kGrad ? M::backward(g[e], v[e], norm[e], inv[e], coef[e])
                     : M::forward(v[e], norm[e], inv[e]);
      }
      if constexpr (kW == 1) {
        IO<T>::store1(out + base + k * S, v[0]);
      } else {
        pack_store<T>(out + base + k * S, v);
      }
    }
  }
}

inline unsigned flat_grid(int64_t threads_needed) {
  const int64_t want = ceil_div(threads_needed, 256);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 64;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

// Short rows (embedding-sized, odd widths): policies of the LDS-staged kernel
// (short_rows.h).
template <typename T, int kP, int kE>
struct LpNormShortForwardOp {
  using A = typename IO<T>::Acc;
  using M = LpMath<T, kP>;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  A normalizer, eps;
  __device__ __forceinline__ void set_packed(bool) {}  // no per-element state: any order
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A*, int, int, A (&v)[kE], const A (&)[kE]) const {
    A acc = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) acc += M::term(v[j]);
    const A norm = M::norm_of(group_allreduce<kL>(acc, SumOp()), normalizer, eps);
    const A inv = A(1) / norm;
#pragma unroll
    for (int j = 0; j < kE; ++j) v[j] = M::forward(v[j], norm, inv);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename T, int kE>
using L1NormShortForward = LpNormShortForwardOp<T, 1, kE>;
template <typename T, int kE>
using L2NormShortForward = LpNormShortForwardOp<T, 2, kE>;

// in0 = dy (overwritten with dx), in1 = x.
template <typename T, int kP, int kE>
struct LpNormShortBackwardOp {
  using A = typename IO<T>::Acc;
  using M = LpMath<T, kP>;
  static constexpr int kIn = 2;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  A normalizer, eps;
  __device__ __forceinline__ void set_packed(bool) {}  // no per-element state: any order
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A*, int, int, A (&g)[kE], const A (&x)[kE]) const {
    A acc = A(0), dot = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      acc += M::term(x[j]);
      dot += g[j] * x[j];
    }
    acc = group_allreduce<kL>(acc, SumOp());
    dot = group_allreduce<kL>(dot, SumOp());
    const A norm = M::norm_of(acc, normalizer, eps);
    const A inv = A(1) / norm;
    const A coef = M::coef_of(dot, normalizer, norm);
#pragma unroll
    for (int j = 0; j < kE; ++j) g[j] = M::backward(g[j], x[j], norm, inv, coef);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename T, int kE>
using L1NormShortBackward = LpNormShortBackwardOp<T, 1, kE>;
template <typename T, int kE>
using L2NormShortBackward = LpNormShortBackwardOp<T, 2, kE>;

// Rows of up to 512 bytes in both directions; longer rows (up to 1024 elements)
// that are not whole aligned packets forward only, as for softmax.
inline bool lp_norm_short_rows(int64_t C, size_t elem_bytes, bool grad, const void* a,
                               const void* b, const void* out) {
  if (C > 1024 || !congruent16(a, out) || (grad && !congruent16(a, b))) return false;
  const size_t row_bytes = static_cast<size_t>(C) * elem_bytes;
  if (row_bytes <= 512) return true;
  return !grad && (row_bytes % 16 != 0 || !aligned16(a));
}

template <typename T, int kP, bool kGrad>
int launch_lp_norm(int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                   const void* dy, const void* x, void* out, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* gp = static_cast<const T*>(dy);
  const T* xp = static_cast<const T*>(x);
  T* op = static_cast<T*>(out);
  const A nrm = static_cast<A>(normalizer), eps = static_cast<A>(epsilon);
  const bool packets_ok = aligned16(x) && aligned16(out) && (!kGrad || aligned16(dy));
  ShortPlan sp;
  if (S == 1 && lp_norm_short_rows(C, sizeof(T), kGrad, x, dy, out) &&
      plan_short_rows(C, sizeof(T), 4, aligned16(x), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * (kGrad ? 32 : 16);
    const unsigned grid = short_grid(N, sp.rows_per_chunk);
    if constexpr (kGrad && kP == 1) {
      DRAGON_HIP_SHORT_LAUNCH(T, L1NormShortBackward, sp, lds, grid, stream, N,
                              static_cast<int>(C), gp, xp, op, nrm, eps);
    } else if constexpr (kGrad) {
      DRAGON_HIP_SHORT_LAUNCH(T, L2NormShortBackward, sp, lds, grid, stream, N,
                              static_cast<int>(C), gp, xp, op, nrm, eps);
    } else if constexpr (kP == 1) {
      DRAGON_HIP_SHORT_LAUNCH(T, L1NormShortForward, sp, lds, grid, stream, N,
                              static_cast<int>(C), xp, xp, op, nrm, eps);
    } else {
      DRAGON_HIP_SHORT_LAUNCH(T, L2NormShortForward, sp, lds, grid, stream, N,
                              static_cast<int>(C), xp, xp, op, nrm, eps);
    }
    return status_of_launch();
  }
  RowConfig cfg;
  // The gradient holds two tiles at once: halve the packets a thread may hold.
  if (S == 1 && pick_row_config(ceil_div(C, kVec), kGrad ? 4 : 8, &cfg)) {
    const bool regular = C % kVec == 0 && packets_ok;  // else ragged tiles
#define LAUNCH_FLAVOUR(TPR, VPT, RAGGED)                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    if constexpr (kGrad) {                                                                      \
      hipLaunchKernelGGL((lp_norm_grad_rows<T, kP, TPR, VPT, RAGGED>),                          \
                         dim3(row_grid(N, Tile::kRowsPerBlock)), dim3(Tile::kThreads), 0,       \
                         stream, N, static_cast<int>(C), nrm, eps, gp, xp, op);                 \
    } else {                                                                                    \
      hipLaunchKernelGGL((lp_norm_rows<T, kP, TPR, VPT, RAGGED>),                               \
                         dim3(row_grid(N, Tile::kRowsPerBlock)), dim3(Tile::kThreads), 0,       \
                         stream, N, static_cast<int>(C), nrm, eps, xp, op);                     \
    }                                                                                           \
  }
#define LAUNCH(TPR, VPT)                                          \
  {                                                               \
    if (regular) LAUNCH_FLAVOUR(TPR, VPT, false)                  \
    else LAUNCH_FLAVOUR(TPR, VPT, true)                           \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
#undef LAUNCH_FLAVOUR
  } else if (S == 1) {
    hipLaunchKernelGGL((lp_norm_rows_looped<T, kP, kGrad>), dim3(loop_grid(N)), dim3(kLoopThreads),
                       0, stream, N, C, nrm, eps, gp, xp, op);
  } else if (const int tw = pick_col_tw(N, C, S, kVec, 16)) {
    // the gradient holds two tiles: 8 packets per thread each where that holds C rows
    const bool small = kGrad && C <= static_cast<int64_t>(kColThreads / tw) * 8;
#define LAUNCH(TW)                                                                            \
  {                                                                                           \
    const ColGrid g = make_col_grid(N, S, C, TW * kVec);                                      \
    const dim3 grid(col_launch_grid(g.tiles)), block(kColThreads);                            \
    if (small) {                                                                              \
      hipLaunchKernelGGL((lp_norm_col_tiles<T, kP, kGrad, TW, 8>), grid, block, 0, stream, g, \
                         nrm, eps, gp, xp, op);                                               \
    } else {                                                                                  \
      hipLaunchKernelGGL((lp_norm_col_tiles<T, kP, kGrad, TW, 16>), grid, block, 0, stream, g, \
                         nrm, eps, gp, xp, op);                                               \
    }                                                                                         \
  }
    if (tw == 64) LAUNCH(64) else if (tw == 16) LAUNCH(16) else LAUNCH(4)
#undef LAUNCH
  } else if (kVec > 1 && S % kVec == 0 && packets_ok) {
    hipLaunchKernelGGL((lp_norm_columns<T, kP, kGrad, kVec>), dim3(flat_grid(N * (S / kVec))),
                       dim3(256), 0, stream, N, S, C, nrm, eps, gp, xp, op);
  } else {
    hipLaunchKernelGGL((lp_norm_columns<T, kP, kGrad, 1>), dim3(flat_grid(N * S)), dim3(256), 0,
                       stream, N, S, C, nrm, eps, gp, xp, op);
  }
  return status_of_launch();
}

template <typename T>
int lp_norm_fwd(int p, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                const void* x, void* y, hipStream_t s) {
  return p == 1 ? launch_lp_norm<T, 1, false>(N, S, C, normalizer, epsilon, nullptr, x, y, s)
                : launch_lp_norm<T, 2, false>(N, S, C, normalizer, epsilon, nullptr, x, y, s);
}
template <typename T>
int lp_norm_bwd(int p, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                const void* dy, const void* x, void* dx, hipStream_t s) {
  return p == 1 ? launch_lp_norm<T, 1, true>(N, S, C, normalizer, epsilon, dy, x, dx, s)
                : launch_lp_norm<T, 2, true>(N, S, C, normalizer, epsilon, dy, x, dx, s);
}

inline int check_lp_args(int64_t N, int64_t S, int64_t C, float normalizer, const void* a,
                         const void* b) {
  if (N < 0 || S < 0 || C <= 0 || !(normalizer > 0.f)) return DRAGON_HIP_EINVAL;
  if (N * S == 0) return 1;  // nothing to do
  if (!a || !b) return DRAGON_HIP_EINVAL;
  return 0;
}

} // namespace
} // namespace dragon_hip

extern "C" {

int dragon_hip_l1_norm(int dtype, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                       const void* x, void* y, void* stream) {
  const int c = dragon_hip::check_lp_args(N, S, C, normalizer, x, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::lp_norm_fwd, 1, N, S, C, normalizer, epsilon, x, y, s);
}

int dragon_hip_l2_norm(int dtype, int64_t N, int64_t S, int64_t C, float normalizer, float epsilon,
                       const void* x, void* y, void* stream) {
  const int c = dragon_hip::check_lp_args(N, S, C, normalizer, x, y);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::lp_norm_fwd, 2, N, S, C, normalizer, epsilon, x, y, s);
}

int dragon_hip_l1_norm_grad(int dtype, int64_t N, int64_t S, int64_t C, float normalizer,
                            float epsilon, const void* dy, const void* x, void* dx, void* stream) {
  const int c = dragon_hip::check_lp_args(N, S, C, normalizer, dy, x);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  if (!dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::lp_norm_bwd, 1, N, S, C, normalizer, epsilon, dy, x,
                            dx, s);
}

int dragon_hip_l2_norm_grad(int dtype, int64_t N, int64_t S, int64_t C, float normalizer,
                            float epsilon, const void* dy, const void* x, void* dx, void* stream) {
  const int c = dragon_hip::check_lp_args(N, S, C, normalizer, dy, x);
  if (c != 0) return c > 0 ? DRAGON_HIP_OK : c;
  if (!dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::lp_norm_bwd, 2, N, S, C, normalizer, epsilon, dy, x,
                            dx, s);
}

} // extern "C"
