// Softmax cross-entropy loss kernels for gfx950.
//
// Replaces, for float and double (dtypes::Loss, dragon/core/types.h:90):
//   kernels::CrossEntropy (dense and sparse targets), SoftmaxCrossEntropyGrad
//     dragon/kernels/loss/op_kernels.h:51-69,179-189;
//     CPU dragon/kernels/loss/cpu/cross_entropy_kernel.cc:10-42,80-108
//   kernels::ReduceLoss, ReduceLossGrad, BroadcastLossGrad
//     dragon/kernels/loss/op_kernels.h:25-32,95-113;
//     CPU dragon/kernels/loss/cpu/generic_loss_kernel.cc:10-73
// and fuses the bodies of SoftmaxCrossEntropyLossOp / ...GradientOp
// (dragon/operators/loss/cross_entropy_softmax_loss_op.cc:8-143) for sparse
// targets:
//   forward   one pass over the logits writes the probabilities (the op's
//             "X_norm" output), the per-position loss and the validity mask,
//             where the reference runs Softmax, then a gather kernel;
//   backward  one pass over the probabilities writes
//             dx = (p - onehot(target)) * mask * scale, where the reference
//             copies p, patches it per position and rescales it (three passes).
//
// A target outside [0, C) that is not ignore_index is treated as ignored
// (loss 0, mask 0, zero gradient); the reference would read out of bounds.
#include <cfloat>

#include "loss_math.h"
#include "row_tile.h"
#include "short_rows.h"

namespace dragon_hip {
namespace {

constexpr int kLossThreads = 256;
constexpr int kLossWaves = kLossThreads / kWaveSize;
constexpr int kMaxPartials = 1024;  // stage-one workgroups of a loss reduction

// ------------------------------------------------------------------ CrossEntropy

template <typename T>
__global__ __launch_bounds__(kLossThreads) void cross_entropy_dense(
    const int64_t N, const T* __restrict__ input, const T* __restrict__ target,
    T* __restrict__ loss) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < N;
       i += static_cast<int64_t>(gridDim.x) * kLossThreads) {
    loss[i] = target[i] * neg_log_clamped(input[i]);
  }
}

template <typename T, typename TargetT>
__global__ __launch_bounds__(kLossThreads) void cross_entropy_sparse(
    const int64_t NxS, const int64_t S, const int64_t C, const int64_t ignore_index,
    const T* __restrict__ input, const TargetT* __restrict__ target, T* __restrict__ loss,
    T* __restrict__ mask) {
  for (int64_t index = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x;
       index < NxS; index += static_cast<int64_t>(gridDim.x) * kLossThreads) {
    const int64_t i = index / S, j = index - i * S;
    const TargetT tgt = target[index];
    if (target_valid(tgt, ignore_index, C)) {
      loss[index] = neg_log_clamped(input[(i * C + static_cast<int64_t>(tgt)) * S + j]);
      mask[index] = T(1);
    } else {
      loss[index] = mask[index] = T(0);
    }
  }
}

// S > 1: a thread per (n, s) position, neighbouring threads neighbouring s.
template <typename T, typename TargetT>
__global__ __launch_bounds__(kLossThreads) void softmax_ce_grad_positions(
    const int64_t NxS, const int64_t S, const int64_t C, const int64_t ignore_index,
    const TargetT* __restrict__ target, T* __restrict__ dx, T* __restrict__ mask) {
  for (int64_t index = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x;
       index < NxS; index += static_cast<int64_t>(gridDim.x) * kLossThreads) {
    const int64_t i = index / S, j = index - i * S;
    const TargetT tgt = target[index];
    if (target_valid(tgt, ignore_index, C)) {
      dx[(i * C + static_cast<int64_t>(tgt)) * S + j] -= T(1);
      mask[index] = T(1);
    } else {
      T* col = dx + i * C * S + j;
      for (int64_t k = 0; k < C; ++k) col[k * S] = T(0);
      mask[index] = T(0);
    }
  }
}

// S == 1: a wavefront per row, so that an ignored row is cleared with
// coalesced stores.
template <typename T, typename TargetT>
__global__ __launch_bounds__(kLossThreads) void softmax_ce_grad_rows(
    const int64_t N, const int64_t C, const int64_t ignore_index,
    const TargetT* __restrict__ target, T* __restrict__ dx, T* __restrict__ mask) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kLossWaves + threadIdx.x / kWaveSize;
       row < N; row += static_cast<int64_t>(gridDim.x) * kLossWaves) {
    const TargetT tgt = target[row];
    if (target_valid(tgt, ignore_index, C)) {
      if (lane == 0) {
        dx[row * C + static_cast<int64_t>(tgt)] -= T(1);
        mask[row] = T(1);
      }
    } else {
      for (int64_t k = lane; k < C; k += kWaveSize) dx[row * C + k] = T(0);
      if (lane == 0) mask[row] = T(0);
    }
  }
}

// ------------------------------------------------------------------ loss reductions

template <typename T, int kWaves = kLossWaves>
__device__ __forceinline__ T block_sum(T v, T* lds /*kWaves*/) {
  v = wave_allreduce(v, SumOp());
  if ((threadIdx.x & (kWaveSize - 1)) == 0) lds[threadIdx.x / kWaveSize] = v;
  __syncthreads();
  T r = lds[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) r += lds[i];
  __syncthreads();
  return r;
}

// Stage one: workgroup b adds its slice of x[0, n_x) and of mask[0, n_mask)
// and writes partial[2b], partial[2b+1]. Either array may be absent (n == 0).
template <typename T>
__global__ __launch_bounds__(kLossThreads) void loss_partial_sums(
    const int64_t n_x, const T* __restrict__ x, const int64_t n_mask, const T* __restrict__ mask,
    T* __restrict__ partial) {
  __shared__ T lds[kLossWaves];
  T a = T(0), b = T(0);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kLossThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < n_x;
       i += stride)
    a += x[i];
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < n_mask;
       i += stride)
    b += mask[i];
  a = block_sum(a, lds);
  b = block_sum(b, lds);
  if (threadIdx.x == 0) {
    partial[2 * blockIdx.x] = a;
    partial[2 * blockIdx.x + 1] = b;
  }
}

// Stage one of counting valid targets: partial[2b] = 0, partial[2b+1] = count.
template <typename T, typename TargetT>
__global__ __launch_bounds__(kLossThreads) void valid_target_partial_counts(
    const int64_t NxS, const int64_t C, const int64_t ignore_index,
    const TargetT* __restrict__ target, T* __restrict__ partial) {
  __shared__ T lds[kLossWaves];
  T b = T(0);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < NxS;
       i += static_cast<int64_t>(gridDim.x) * kLossThreads)
    b += target_valid(target[i], ignore_index, C) ? T(1) : T(0);
  b = block_sum(b, lds);
  if (threadIdx.x == 0) {
    partial[2 * blockIdx.x] = T(0);
    partial[2 * blockIdx.x + 1] = b;
  }
}

// Stage two (one workgroup): totals of the partial pairs in index order, then
//   kReduce   y[0] = sum_x * (1 / max(inv_scale, 1))              (ReduceLoss)
//   kGradScale  y[0] = dl[0] / max(inv_scale, 0.5)                (ReduceLossGrad)
// with inv_scale = sum_mask when `by_mask`, else `normalizer`.
enum LossFinal { kReduce = 0, kGradScale = 1 };
template <typename T, int kMode>
__global__ __launch_bounds__(kLossThreads) void loss_finalize(
    const int nparts, const T* __restrict__ partial, const bool by_mask, const float normalizer,
    const T* __restrict__ dl, T* __restrict__ y) {
  __shared__ T lds[kLossWaves];
  T a = T(0), b = T(0);
  for (int i = threadIdx.x; i < nparts; i += kLossThreads) {
    a += partial[2 * i];
    b += partial[2 * i + 1];
  }
  a = block_sum(a, lds);
  b = block_sum(b, lds);
  if (threadIdx.x == 0) {
    const float inv_scale = by_mask ? static_cast<float>(b) : normalizer;
    if (kMode == kReduce) {
      const float scale = 1.f / (inv_scale > 1.f ? inv_scale : 1.f);
      y[0] = a * static_cast<T>(scale);
    } else {
      y[0] = static_cast<T>(static_cast<float>(dl[0]) / (inv_scale > 0.5f ? inv_scale : 0.5f));
    }
  }
}

// Both stages in one workgroup, for reductions short enough that a second
// launch would cost more than the loop: sums x[0, n_x) and mask[0, n_mask)
// (or, with kCountTargets, counts the valid targets) and applies the epilogue
// of loss_finalize.
constexpr int kDirectThreads = 1024;
constexpr int64_t kDirectReduceMax = 16 * 1024;
template <typename T, typename TargetT, int kMode, bool kCountTargets>
__global__ __launch_bounds__(kDirectThreads) void loss_reduce_direct(
    const int64_t n_x, const T* __restrict__ x, const int64_t n_mask, const T* __restrict__ mask,
    const TargetT* __restrict__ target, const int64_t C, const int64_t ignore_index,
    const bool by_mask, const float normalizer, const T* __restrict__ dl, T* __restrict__ y) {
  constexpr int kWaves = kDirectThreads / kWaveSize;
  constexpr int kSteps = static_cast<int>(kDirectReduceMax / kDirectThreads);
  __shared__ T lds[kWaves];
  T a = T(0), b = T(0);
  // fixed trip count with guarded, independent loads: all of them are in flight at once
#pragma unroll
  for (int k = 0; k < kSteps; ++k) {
    const int64_t i = static_cast<int64_t>(k) * kDirectThreads + threadIdx.x;
    if (i < n_x) a += x[i];
    if (i < n_mask) {
      if constexpr (kCountTargets) {
        b += target_valid(target[i], ignore_index, C) ? T(1) : T(0);
      } else {
        b += mask[i];
      }
    }
  }
  a = block_sum<T, kWaves>(a, lds);
  b = block_sum<T, kWaves>(b, lds);
  if (threadIdx.x == 0) {
    const float inv_scale = by_mask ? static_cast<float>(b) : normalizer;
    if (kMode == kReduce) {
      const float scale = 1.f / (inv_scale > 1.f ? inv_scale : 1.f);
      y[0] = a * static_cast<T>(scale);
    } else {
      y[0] = static_cast<T>(static_cast<float>(dl[0]) / (inv_scale > 0.5f ? inv_scale : 0.5f));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kLossThreads) void scale_by_device_scalar(
    const int64_t N, const T* __restrict__ scale, T* __restrict__ dx) {
  const T alpha = scale[0];
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < N;
       i += static_cast<int64_t>(gridDim.x) * kLossThreads)
    dx[i] *= alpha;
}

template <typename T>
__global__ __launch_bounds__(kLossThreads) void broadcast_loss_grad(
    const int64_t NxCxS, const int64_t CxS, const int64_t S, const T* __restrict__ dl,
    T* __restrict__ dx) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; i < NxCxS;
       i += static_cast<int64_t>(gridDim.x) * kLossThreads)
    dx[i] *= dl[i / CxS * S + i % S];
}

// ------------------------------------------------------------------ fused forward (S == 1)

// softmax_rows with the loss gather folded in: the thread whose tile slot holds
// column `target[row]` writes -log(max(p, FLT_MIN)).
template <typename T, typename TargetT, int kTPR, int kVPT, bool kRagged>
__global__ __launch_bounds__(row_threads(kTPR)) void softmax_ce_rows(
    const int64_t N, const int C, const int64_t ignore_index, const T* __restrict__ x,
    const TargetT* __restrict__ target, T* __restrict__ prob, T* __restrict__ loss,
    T* __restrict__ mask) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = Tile::extent_of(C);

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < N; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile t;
    t.load(x + row * C, npackets, acc_neg_inf<A>());
    const TargetT tgt = target[row];
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) m = MaxOp()(m, t.v[i][e]);
    m = Tile::reduce(m, MaxOp(), slots[0]);
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = acc_exp(t.v[i][e] - m);
        s += t.v[i][e];
      }
    s = Tile::reduce(s, SumOp(), slots[1]);
    const bool valid = target_valid(tgt, ignore_index, C);
    const int col = valid ? static_cast<int>(tgt) : -1;
    const A inv = A(1) / s;  // fp32 multiplies by the reciprocal, as the softmax kernels do
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = sizeof(A) == 4 ? t.v[i][e] * inv : t.v[i][e] / s;
        if ((i * kTPR + Tile::lane()) * kVec + e == col) {
          loss[row] = neg_log_clamped(t.v[i][e]);
          mask[row] = T(1);
        }
      }
    if (!valid && Tile::lane() == 0) loss[row] = mask[row] = T(0);
    t.store(prob + row * C, npackets);
    if (kTPR != kWaveSize) __syncthreads();
  }
}

// The same for short rows (a handful to a few hundred classes): a policy of the
// LDS-staged kernel (short_rows.h), several rows per wavefront. The row's target
// travels as the per-row scalar: its column, or -1 when ignored.
template <typename T, typename TargetT, int kE>
struct SoftmaxCeShortOp {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 1;
  int64_t ignore_index;
  int classes;
  const TargetT* target;
  T* loss;
  T* mask;
  __device__ __forceinline__ A fill0() const { return acc_neg_inf<A>(); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[1]) const {
    const TargetT tgt = target[row];
    w[0] = target_valid(tgt, ignore_index, classes) ? static_cast<A>(tgt) : A(-1);  // < 1024: exact
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A* side, int l, int, A (&v)[kE],
                                      const A (&)[kE]) const {
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int j = 0; j < kE; ++j) m = MaxOp()(m, v[j]);
    m = group_allreduce<kL>(m, MaxOp());
    A s = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      v[j] = acc_exp(v[j] - m);  // lanes past the row: exp(-inf) = 0
      s += v[j];
    }
    s = group_allreduce<kL>(s, SumOp());
    const int col = static_cast<int>(side[0]);
    const A inv = A(1) / s;
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      v[j] = sizeof(A) == 4 ? v[j] * inv : v[j] / s;
      if (l + j * kL == col) {
        loss[r] = neg_log_clamped(v[j]);
        mask[r] = T(1);
      }
    }
    if (col < 0 && l == 0) loss[r] = mask[r] = T(0);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename T, int kE>
using SoftmaxCeShortI32 = SoftmaxCeShortOp<T, int32_t, kE>;
template <typename T, int kE>
using SoftmaxCeShortI64 = SoftmaxCeShortOp<T, int64_t, kE>;

// The same for rows that take a whole 1024-thread workgroup: persistent
// workgroups that request the next row's packets before reducing the current
// one (see softmax_wide_rows).
template <typename T, typename TargetT, int kVPT>
__global__ __launch_bounds__(1024) void softmax_ce_wide_rows(
    const int64_t N, const int C, const int64_t ignore_index, const T* __restrict__ x,
    const TargetT* __restrict__ target, T* __restrict__ prob, T* __restrict__ loss,
    T* __restrict__ mask) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = C / kVec;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  Raw cur;
  cur.load(x + (row < N ? row : 0) * C, npackets, row < N);
  for (; row < N; row += stride) {
    Raw nxt;
    const bool more = row + stride < N;
    nxt.load(x + (more ? row + stride : 0) * C, npackets, more);
    const TargetT tgt = target[row];
    Tile t;
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      cur.unpack(i, t.v[i]);
      const bool on = Tile::active(i, npackets);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = on ? t.v[i][e] : acc_neg_inf<A>();  // raw padding is zero bits
        m = MaxOp()(m, t.v[i][e]);
      }
    }
    m = Tile::reduce(m, MaxOp(), slots[0]);
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = acc_exp(t.v[i][e] - m);
        s += t.v[i][e];
      }
    s = Tile::reduce(s, SumOp(), slots[1]);
    const bool valid = target_valid(tgt, ignore_index, C);
    const int col = valid ? static_cast<int>(tgt) : -1;
    const A inv = A(1) / s;
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = sizeof(A) == 4 ? t.v[i][e] * inv : t.v[i][e] / s;
        if ((i * kTPR + static_cast<int>(threadIdx.x)) * kVec + e == col) {
          loss[row] = neg_log_clamped(t.v[i][e]);
          mask[row] = T(1);
        }
      }
    if (!valid && threadIdx.x == 0) loss[row] = mask[row] = T(0);
    nxt.wait_ready();
    cur = nxt;
    t.store(prob + row * C, npackets);
    __syncthreads();  // slots are reused by the next row
  }
}

// softmax_ce_wide_rows for rows that are not whole aligned packets, through the
// aligned packets that cover a row (RowWindow; x and prob congruent modulo 16
// bytes; the caller picks kVPT for C / kVec + 2 packets). What the window's
// first and last packet hold of the neighbouring rows is set to -inf in the two
// lanes concerned before the row is reduced; those two packets of the output go
// through LDS and are stored element by element. The target's column moves by
// the window's lead.
template <typename T, typename TargetT, int kVPT>
__global__ __launch_bounds__(1024) void softmax_ce_wide_windows(
    const int64_t N, const int C, const int64_t ignore_index, const T* __restrict__ x,
    const TargetT* __restrict__ target, T* __restrict__ prob, T* __restrict__ loss,
    T* __restrict__ mask) {
  constexpr int kTPR = 1024;
  using Tile = RowTile<T, kTPR, kVPT>;
  using Raw = RawRowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  __shared__ u32x4 edge[2];
  const int lane = threadIdx.x;
  const int64_t stride = gridDim.x;
  int64_t row = blockIdx.x;
  auto request = [&](Raw& t, const int64_t at, const bool valid) {
    const int64_t from = valid ? at : 0;
    const RowWindow<T> w(x + from * C, C);
    t.load(x + from * C - w.lead, w.packets, valid);
  };
  Raw cur;
  request(cur, row, row < N);
  for (; row < N; row += stride) {
    Raw nxt;
    request(nxt, row + stride, row + stride < N);
    const RowWindow<T> w(x + row * C, C);
    const int tail_slot = (w.packets - 1) / kTPR, tail_lane = (w.packets - 1) % kTPR;
    const bool head_partial = w.lead > 0 || (w.packets == 1 && w.tail_valid < kVec);
    const bool tail_partial = w.packets > 1 && w.tail_valid < kVec;
    auto keep = [&](u32x4& packet, const int first, const int last) {
      A v[kVec];
      IO<T>::unpack(packet, v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        if (e < first || e >= last) v[e] = acc_neg_inf<A>();
      }
      packet = IO<T>::pack(v);
    };
    if (head_partial && lane == 0) keep(cur.p[0], w.lead, w.packets == 1 ? w.tail_valid : kVec);
    if (tail_partial && lane == tail_lane) {
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (i == tail_slot) keep(cur.p[i], 0, w.tail_valid);
      }
    }
    const TargetT tgt = target[row];
    Tile t;
    A m = acc_neg_inf<A>();
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      cur.unpack(i, t.v[i]);
      const bool on = Tile::active(i, w.packets);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = on ? t.v[i][e] : acc_neg_inf<A>();  // raw padding is zero bits
        m = MaxOp()(m, t.v[i][e]);
      }
    }
    m = Tile::reduce(m, MaxOp(), slots[0]);
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = acc_exp(t.v[i][e] - m);
        s += t.v[i][e];
      }
    s = Tile::reduce(s, SumOp(), slots[1]);
    const bool valid = target_valid(tgt, ignore_index, C);
    const int col = valid ? static_cast<int>(tgt) + w.lead : -1;  // from the window's start
    const A inv = A(1) / s;
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        t.v[i][e] = sizeof(A) == 4 ? t.v[i][e] * inv : t.v[i][e] / s;
        if ((i * kTPR + lane) * kVec + e == col) {
          loss[row] = neg_log_clamped(t.v[i][e]);
          mask[row] = T(1);
        }
      }
    if (!valid && lane == 0) loss[row] = mask[row] = T(0);
    nxt.wait_ready();
    cur = nxt;
    T* base = prob + row * C - w.lead;
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      const int idx = i * kTPR + lane;
      if (idx < w.packets) {
        const u32x4 packet = IO<T>::pack(t.v[i]);
        if (idx == 0 && head_partial) {
          edge[0] = packet;
        } else if (idx == w.packets - 1 && tail_partial) {
          edge[1] = packet;
        } else {
          store_packet(base + static_cast<int64_t>(idx) * kVec, packet);
        }
      }
    }
    __syncthreads();  // slots are reused by the next row; the edge packets are in LDS
    if (lane < 2 * kVec) {
      const int which = lane / kVec, e = lane % kVec;
      const T* from = reinterpret_cast<const T*>(&edge[which]);
      if (which == 0 && head_partial) {
        const int last = w.packets == 1 ? w.tail_valid : kVec;
        if (e >= w.lead && e < last) base[e] = from[e];
      } else if (which == 1 && tail_partial) {
        if (e < w.tail_valid) base[static_cast<int64_t>(w.packets - 1) * kVec + e] = from[e];
      }
    }
  }
}

// ------------------------------------------------------------------ fused backward

// dx = (p - [k == target]) * w over [N, C, S], with w = 0 where the target is
// ignored, else dl[n * S + s] (kPerPosition) or the scalar scale[0]. kAlongC:
// the packet runs along C (S == 1), else along S.
template <typename T, typename TargetT, int kVec, bool kAlongC, bool kPerPosition>
__global__ __launch_bounds__(kLossThreads) void softmax_ce_backward(
    const int64_t npackets, const int64_t S, const int64_t C, const int64_t ignore_index,
    const T* __restrict__ prob, const TargetT* __restrict__ target, const T* __restrict__ dl,
    const T* __restrict__ scale, T* __restrict__ dx) {
  using A = typename IO<T>::Acc;
  const A alpha = kPerPosition ? A(0) : static_cast<A>(scale[0]);
  for (int64_t ip = static_cast<int64_t>(blockIdx.x) * kLossThreads + threadIdx.x; ip < npackets;
       ip += static_cast<int64_t>(gridDim.x) * kLossThreads) {
    const int64_t i = ip * kVec;
    A v[kVec];
    if constexpr (kVec == 1) {
      v[0] = IO<T>::load1(prob + i);
    } else {
      load_unpack<T>(prob + i, v);
    }
    if constexpr (kAlongC) {
      const int64_t n = i / C, k0 = i - n * C;
      if (k0 + kVec <= C) {  // the packet lies within one row
        const TargetT tgt = target[n];
        const bool valid = target_valid(tgt, ignore_index, C);
        const A w = valid ? (kPerPosition ? static_cast<A>(dl[n]) : alpha) : A(0);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A hot = (valid && k0 + e == static_cast<int64_t>(tgt)) ? A(1) : A(0);
          v[e] = (v[e] - hot) * w;
        }
      } else {  // C is not a multiple of the packet: this one straddles rows
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const int64_t ne = (i + e) / C, ke = (i + e) - ne * C;
          const TargetT tgt = target[ne];
          const bool valid = target_valid(tgt, ignore_index, C);
          const A w = valid ? (kPerPosition ? static_cast<A>(dl[ne]) : alpha) : A(0);
          const A hot = (valid && ke == static_cast<int64_t>(tgt)) ? A(1) : A(0);
          v[e] = (v[e] - hot) * w;
        }
      }
    } else {
      const int64_t n = i / (C * S);
      const int64_t rem = i - n * C * S;
      const int64_t k = rem / S, s0 = rem - k * S;
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const int64_t pos = n * S + s0 + e;
        const TargetT tgt = target[pos];
        const bool valid = target_valid(tgt, ignore_index, C);
        const A w = valid ? (kPerPosition ? static_cast<A>(dl[pos]) : alpha) : A(0);
        const A hot = (valid && k == static_cast<int64_t>(tgt)) ? A(1) : A(0);
        v[e] = (v[e] - hot) * w;
      }
    }
    if constexpr (kVec == 1) {
      IO<T>::store1(dx + i, v[0]);
    } else {
      pack_store<T>(dx + i, v);
    }
  }
}

// The same for S == 1 in whole packets: a workgroup takes chunks of kLossThreads * 4
// consecutive packets (16 KB) and requests a thread's four packets, and their rows'
// targets, before it uses the first; the row of a packet comes from one division per chunk
// and a 32-bit one per packet.
template <typename T, typename TargetT, bool kPerPosition>
__global__ __launch_bounds__(kLossThreads) void softmax_ce_backward_chunks(
    const int64_t npackets, const int64_t C, const int64_t ignore_index,
    const T* __restrict__ prob, const TargetT* __restrict__ target, const T* __restrict__ dl,
    const T* __restrict__ scale, T* __restrict__ dx) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kBatch = 4;
  constexpr int64_t kChunk = static_cast<int64_t>(kLossThreads) * kBatch;
  const A alpha = kPerPosition ? A(0) : static_cast<A>(scale[0]);
  for (int64_t c0 = static_cast<int64_t>(blockIdx.x) * kChunk; c0 < npackets;
       c0 += static_cast<int64_t>(gridDim.x) * kChunk) {
    const int64_t n0 = c0 * kVec / C;                       // uniform over the workgroup
    const uint32_t k_start = static_cast<uint32_t>(c0 * kVec - n0 * C);
    u32x4 raw[kBatch];
    int64_t rn[kBatch];
    uint32_t rk[kBatch];
    TargetT tg[kBatch];
    A wl[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int64_t p = c0 + j * kLossThreads + threadIdx.x;
      const bool on = p < npackets;
      raw[j] = load_packet(prob + (on ? p : c0) * kVec);
      const uint32_t k = k_start + static_cast<uint32_t>(on ? j * kLossThreads + threadIdx.x : 0) * kVec;
      const uint32_t dn = k / static_cast<uint32_t>(C);
      rn[j] = n0 + dn;
      rk[j] = k - dn * static_cast<uint32_t>(C);
      tg[j] = target[rn[j]];
      wl[j] = kPerPosition ? static_cast<A>(dl[rn[j]]) : alpha;
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int64_t p = c0 + j * kLossThreads + threadIdx.x;
      if (p >= npackets) continue;
      A v[kVec];
      IO<T>::unpack(raw[j], v);
      if (rk[j] + kVec <= C) {  // the packet lies within one row
        const bool valid = target_valid(tg[j], ignore_index, C);
        const A w = valid ? wl[j] : A(0);
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A hot = (valid && static_cast<int64_t>(rk[j]) + e == static_cast<int64_t>(tg[j])) ? A(1) : A(0);
          v[e] = (v[e] - hot) * w;
        }
      } else {  // C is not a multiple of the packet: this one straddles two rows
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const bool next = rk[j] + e >= C;
          const int64_t ne = rn[j] + (next ? 1 : 0);
          const int64_t ke = static_cast<int64_t>(rk[j]) + e - (next ? C : 0);
          const TargetT tgt = target[ne];
          const bool valid = target_valid(tgt, ignore_index, C);
          const A w = valid ? (kPerPosition ? static_cast<A>(dl[ne]) : alpha) : A(0);
          const A hot = (valid && ke == static_cast<int64_t>(tgt)) ? A(1) : A(0);
          v[e] = (v[e] - hot) * w;
        }
      }
      pack_store<T>(dx + p * kVec, v);
    }
  }
}

// The same for a class axis in the middle (S > 1, a multiple of the packet): the packet runs
// along S, so its elements share a class and belong to kVec consecutive positions.
template <typename T, typename TargetT, bool kPerPosition>
__global__ __launch_bounds__(kLossThreads) void softmax_ce_backward_chunks_strided(
    const int64_t npackets, const uint32_t S, const uint32_t C, const int64_t ignore_index,
    const T* __restrict__ prob, const TargetT* __restrict__ target, const T* __restrict__ dl,
    const T* __restrict__ scale, T* __restrict__ dx) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  constexpr int kBatch = 4;
  constexpr int64_t kChunk = static_cast<int64_t>(kLossThreads) * kBatch;
  const A alpha = kPerPosition ? A(0) : static_cast<A>(scale[0]);
  const uint32_t CS = C * S;  // the caller keeps it below 2^30
  for (int64_t c0 = static_cast<int64_t>(blockIdx.x) * kChunk; c0 < npackets;
       c0 += static_cast<int64_t>(gridDim.x) * kChunk) {
    const int64_t n0 = c0 * kVec / CS;  // uniform over the workgroup
    const uint32_t rem0 = static_cast<uint32_t>(c0 * kVec - n0 * CS);
    u32x4 raw[kBatch];
    uint32_t rk[kBatch];
    int64_t pos[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int64_t p = c0 + j * kLossThreads + threadIdx.x;
      const bool on = p < npackets;
      raw[j] = load_packet(prob + (on ? p : c0) * kVec);
      uint32_t r = rem0 + static_cast<uint32_t>(on ? j * kLossThreads + threadIdx.x : 0) * kVec;
      const uint32_t dn = r / CS;
      r -= dn * CS;
      rk[j] = r / S;
      pos[j] = (n0 + dn) * S + (r - rk[j] * S);
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      const int64_t p = c0 + j * kLossThreads + threadIdx.x;
      if (p >= npackets) continue;
      A v[kVec];
      IO<T>::unpack(raw[j], v);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const TargetT tgt = target[pos[j] + e];
        const bool valid = target_valid(tgt, ignore_index, C);
        const A w = valid ? (kPerPosition ? static_cast<A>(dl[pos[j] + e]) : alpha) : A(0);
        const A hot = (valid && static_cast<int64_t>(rk[j]) == static_cast<int64_t>(tgt)) ? A(1) : A(0);
        v[e] = (v[e] - hot) * w;
      }
      pack_store<T>(dx + p * kVec, v);
    }
  }
}

// ------------------------------------------------------------------ launchers

inline unsigned loss_grid(int64_t work_items) {
  const int64_t want = ceil_div(work_items, kLossThreads);
  const int64_t cap = static_cast<int64_t>(num_cus()) * 32;
  return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

// Stage-one workgroups of a reduction over n elements (at most kMaxPartials).
inline int partial_blocks(int64_t n) {
  const int64_t want = ceil_div(n, static_cast<int64_t>(kLossThreads) * 8);
  return static_cast<int>(want < 1 ? 1 : (want > kMaxPartials ? kMaxPartials : want));
}

// Scratch of a loss reduction: the partial pairs plus one scalar.
inline size_t reduce_loss_scratch(size_t elem) { return (2 * kMaxPartials + 1) * elem; }
// Scratch of the fused loss forward: loss[NxS], mask[NxS], the reduction's
// partial pairs and scalar, rounded up to 16 bytes; what the softmax of rows
// beyond the fused row tiles asks for follows.
inline size_t fused_loss_head_bytes(size_t elem, int64_t N, int64_t S) {
  const size_t head = static_cast<size_t>(2 * N * S) * elem + reduce_loss_scratch(elem);
  return (head + 15) / 16 * 16;
}

template <typename T>
int launch_cross_entropy(int64_t N, const void* input, const void* target, void* loss,
                         hipStream_t stream) {
  hipLaunchKernelGGL((cross_entropy_dense<T>), dim3(loss_grid(N)), dim3(kLossThreads), 0, stream,
                     N, static_cast<const T*>(input), static_cast<const T*>(target),
                     static_cast<T*>(loss));
  return status_of_launch();
}

template <typename T, typename TargetT>
int launch_sparse_cross_entropy(int64_t N, int64_t S, int64_t C, int64_t ignore_index,
                                const void* input, const void* target, void* loss, void* mask,
                                hipStream_t stream) {
  hipLaunchKernelGGL((cross_entropy_sparse<T, TargetT>), dim3(loss_grid(N * S)),
                     dim3(kLossThreads), 0, stream, N * S, S, C, ignore_index,
                     static_cast<const T*>(input), static_cast<const TargetT*>(target),
                     static_cast<T*>(loss), static_cast<T*>(mask));
  return status_of_launch();
}

template <typename T, typename TargetT>
int launch_softmax_ce_grad(int64_t N, int64_t S, int64_t C, int64_t ignore_index,
                           const void* target, void* dx, void* mask, hipStream_t stream) {
  const TargetT* tp = static_cast<const TargetT*>(target);
  if (S == 1) {
    hipLaunchKernelGGL((softmax_ce_grad_rows<T, TargetT>), dim3(loss_grid(N * kWaveSize)),
                       dim3(kLossThreads), 0, stream, N, C, ignore_index, tp, static_cast<T*>(dx),
                       static_cast<T*>(mask));
  } else {
    hipLaunchKernelGGL((softmax_ce_grad_positions<T, TargetT>), dim3(loss_grid(N * S)),
                       dim3(kLossThreads), 0, stream, N * S, S, C, ignore_index, tp,
                       static_cast<T*>(dx), static_cast<T*>(mask));
  }
  return status_of_launch();
}

template <typename T>
int launch_reduce_loss(int64_t N, int64_t num_masks, float normalizer, const void* x,
                       const void* mask, void* y, void* scratch, hipStream_t stream) {
  const bool by_mask = num_masks > 0 && normalizer < 0.f;
  T* part = static_cast<T*>(scratch);
  const int64_t n_mask = by_mask ? num_masks : 0;
  if (N <= kDirectReduceMax && n_mask <= kDirectReduceMax) {
    hipLaunchKernelGGL((loss_reduce_direct<T, int32_t, kReduce, false>), dim3(1),
                       dim3(kDirectThreads), 0, stream, N, static_cast<const T*>(x), n_mask,
                       static_cast<const T*>(mask), static_cast<const int32_t*>(nullptr),
                       static_cast<int64_t>(0), static_cast<int64_t>(0), by_mask, normalizer,
                       static_cast<const T*>(nullptr), static_cast<T*>(y));
    return status_of_launch();
  }
  const int nparts = partial_blocks(N > n_mask ? N : n_mask);
  hipLaunchKernelGGL((loss_partial_sums<T>), dim3(nparts), dim3(kLossThreads), 0, stream, N,
                     static_cast<const T*>(x), n_mask, static_cast<const T*>(mask), part);
  hipLaunchKernelGGL((loss_finalize<T, kReduce>), dim3(1), dim3(kLossThreads), 0, stream, nparts,
                     part, by_mask, normalizer, static_cast<const T*>(nullptr),
                     static_cast<T*>(y));
  return status_of_launch();
}

template <typename T>
int launch_reduce_loss_grad(int64_t N, int64_t num_masks, float normalizer, const void* dl,
                            const void* mask, void* dx, void* scratch, hipStream_t stream) {
  const bool by_mask = num_masks > 0 && normalizer < 0.f;
  T* part = static_cast<T*>(scratch);
  T* scalar = part + 2 * kMaxPartials;
  if (!by_mask || num_masks <= kDirectReduceMax) {
    hipLaunchKernelGGL((loss_reduce_direct<T, int32_t, kGradScale, false>), dim3(1),
                       dim3(kDirectThreads), 0, stream, static_cast<int64_t>(0),
                       static_cast<const T*>(nullptr), by_mask ? num_masks : static_cast<int64_t>(0),
                       static_cast<const T*>(mask), static_cast<const int32_t*>(nullptr),
                       static_cast<int64_t>(0), static_cast<int64_t>(0), by_mask, normalizer,
                       static_cast<const T*>(dl), scalar);
  } else {
    const int nparts = partial_blocks(num_masks);
    hipLaunchKernelGGL((loss_partial_sums<T>), dim3(nparts), dim3(kLossThreads), 0, stream,
                       static_cast<int64_t>(0), static_cast<const T*>(nullptr), num_masks,
                       static_cast<const T*>(mask), part);
    hipLaunchKernelGGL((loss_finalize<T, kGradScale>), dim3(1), dim3(kLossThreads), 0, stream,
                       nparts, part, by_mask, normalizer, static_cast<const T*>(dl), scalar);
  }
  hipLaunchKernelGGL((scale_by_device_scalar<T>), dim3(loss_grid(N)), dim3(kLossThreads), 0,
                     stream, N, scalar, static_cast<T*>(dx));
  return status_of_launch();
}

template <typename T>
int launch_broadcast_loss_grad(int64_t N, int64_t S, int64_t C, const void* dl, void* dx,
                               hipStream_t stream) {
  hipLaunchKernelGGL((broadcast_loss_grad<T>), dim3(loss_grid(N * C * S)), dim3(kLossThreads), 0,
                     stream, N * C * S, C * S, S, static_cast<const T*>(dl), static_cast<T*>(dx));
  return status_of_launch();
}

enum Reduction { kNone = 0, kSum = 1, kMean = 2, kBatchMean = 3, kValid = 4 };

// The normalizer the operator bodies derive from the reduction
// (cross_entropy_softmax_loss_op.cc:69-78); -1 selects the mask count.
inline float loss_normalizer(int reduction, int64_t N, int64_t S, bool has_mask) {
  switch (reduction) {
    case kValid: return has_mask ? -1.f : static_cast<float>(N * S);
    case kBatchMean: return static_cast<float>(N);
    case kMean: return static_cast<float>(N * S);
    default: return 1.f;
  }
}

template <typename T, typename TargetT>
int launch_fused_forward(int64_t N, int64_t S, int64_t C, int64_t ignore_index, int reduction,
                         const void* x, const void* target, void* prob, void* out, void* scratch,
                         hipStream_t stream) {
  constexpr int kVec = IO<T>::kVec;
  const T* xp = static_cast<const T*>(x);
  const TargetT* tp = static_cast<const TargetT*>(target);
  T* pp = static_cast<T*>(prob);
  const int64_t NxS = N * S;
  // reduction == NONE writes the per-position loss straight to the output
  T* loss = reduction == kNone ? static_cast<T*>(out) : static_cast<T*>(scratch);
  T* mask = static_cast<T*>(scratch) + NxS;
  T* part = mask + NxS;
  ShortPlan sp;
  // rows of up to 512 bytes, and longer rows that are not whole aligned packets
  if (S == 1 && C <= 1024 && congruent16(x, prob) &&
      (C * sizeof(T) <= 512 || (C * sizeof(T)) % 16 != 0 || !aligned16(x)) &&
      plan_short_rows(C, sizeof(T), 4, aligned16(x), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16 + sp.rows_per_chunk * sizeof(T);
    const unsigned grid = short_grid(N, sp.rows_per_chunk);
    if constexpr (sizeof(TargetT) == 4) {
      DRAGON_HIP_SHORT_LAUNCH(T, SoftmaxCeShortI32, sp, lds, grid, stream, N, static_cast<int>(C),
                              xp, xp, pp, ignore_index, static_cast<int>(C),
                              reinterpret_cast<const int32_t*>(tp), loss, mask);
    } else {
      DRAGON_HIP_SHORT_LAUNCH(T, SoftmaxCeShortI64, sp, lds, grid, stream, N, static_cast<int>(C),
                              xp, xp, pp, ignore_index, static_cast<int>(C),
                              reinterpret_cast<const int64_t*>(tp), loss, mask);
    }
  } else
  if (RowConfig cfg; S == 1 && pick_row_config(ceil_div(C, kVec), 8, &cfg)) {
    const bool regular = C % kVec == 0 && aligned16(x) && aligned16(prob);  // else ragged tiles
    if (regular && cfg.tpr == 1024) {
#define LAUNCH_WIDE(VPT)                                                                        \
  {                                                                                             \
    note_flavour("softmax_ce_wide_rows<" #VPT ">");                                            \
    auto kernel = softmax_ce_wide_rows<T, TargetT, VPT>;                                        \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                   \
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C),       \
                       ignore_index, xp, tp, pp, loss, mask);                                   \
  }
      if (cfg.vpt == 2) LAUNCH_WIDE(2) else if (cfg.vpt == 4) LAUNCH_WIDE(4) else LAUNCH_WIDE(8)
#undef LAUNCH_WIDE
    } else if (RowConfig wcfg; !regular && congruent16(x, prob) &&
               pick_row_config(C / kVec + 2, 8, &wcfg) && wcfg.tpr == 1024) {
      // rows of 1024-thread size that are not whole aligned packets: through their windows
#define LAUNCH_WINDOWS(VPT)                                                                     \
  {                                                                                             \
    note_flavour("softmax_ce_wide_windows<" #VPT ">");                                         \
    auto kernel = softmax_ce_wide_windows<T, TargetT, VPT>;                                     \
    const unsigned resident = resident_grid(kernel, 1024, 0);                                   \
    const unsigned grid = N < static_cast<int64_t>(resident) ? static_cast<unsigned>(N) : resident; \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(1024), 0, stream, N, static_cast<int>(C),       \
                       ignore_index, xp, tp, pp, loss, mask);                                   \
  }
      if (wcfg.vpt == 2) LAUNCH_WINDOWS(2) else if (wcfg.vpt == 4) LAUNCH_WINDOWS(4)
      else LAUNCH_WINDOWS(8)
#undef LAUNCH_WINDOWS
    } else {
#define LAUNCH(TPR, VPT)                                                                        \
  {                                                                                             \
    using Tile = RowTile<T, TPR, VPT>;                                                          \
    const dim3 grid(row_grid(N, Tile::kRowsPerBlock)), block(Tile::kThreads);                   \
    if (regular) {                                                                              \
      hipLaunchKernelGGL((softmax_ce_rows<T, TargetT, TPR, VPT, false>), grid, block, 0, stream, \
                         N, static_cast<int>(C), ignore_index, xp, tp, pp, loss, mask);         \
    } else {                                                                                    \
      hipLaunchKernelGGL((softmax_ce_rows<T, TargetT, TPR, VPT, true>), grid, block, 0, stream, \
                         N, static_cast<int>(C), ignore_index, xp, tp, pp, loss, mask);         \
    }                                                                                           \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
    }
  } else if (S > 1 && launch_softmax_cols_with_loss<T, TargetT>(N, S, C, ignore_index, xp, tp, pp,
                                                                loss, mask, stream) ==
                          DRAGON_HIP_OK) {
    // class axis in the middle (segmentation logits): the column-tile softmax
    // writes the per-position loss itself
  } else {
    // rows beyond the fused row tiles: Softmax (several workgroups per row where
    // that pays), then the per-position loss
    const int tag = sizeof(T) == 8 ? DRAGON_HIP_F64 : DRAGON_HIP_F32;
    const int st = dragon_hip_softmax(tag, N, S, C, x, prob,
                                      static_cast<char*>(scratch) + fused_loss_head_bytes(sizeof(T), N, S),
                                      dragon_hip_softmax_scratch_bytes(tag, N, S, C), stream);
    if (st != DRAGON_HIP_OK) return st;
    hipLaunchKernelGGL((cross_entropy_sparse<T, TargetT>), dim3(loss_grid(NxS)),
                       dim3(kLossThreads), 0, stream, NxS, S, C, ignore_index, pp, tp, loss, mask);
  }
  if (reduction != kNone) {
    const float normalizer = loss_normalizer(reduction, N, S, true);
    const bool by_mask = normalizer < 0.f;
    const int64_t n_mask = by_mask ? NxS : static_cast<int64_t>(0);
    if (NxS <= kDirectReduceMax) {
      hipLaunchKernelGGL((loss_reduce_direct<T, TargetT, kReduce, false>), dim3(1),
                         dim3(kDirectThreads), 0, stream, NxS, loss, n_mask, mask,
                         static_cast<const TargetT*>(nullptr), static_cast<int64_t>(0),
                         static_cast<int64_t>(0), by_mask, normalizer,
                         static_cast<const T*>(nullptr), static_cast<T*>(out));
    } else {
      const int nparts = partial_blocks(NxS);
      hipLaunchKernelGGL((loss_partial_sums<T>), dim3(nparts), dim3(kLossThreads), 0, stream, NxS,
                         loss, n_mask, mask, part);
      hipLaunchKernelGGL((loss_finalize<T, kReduce>), dim3(1), dim3(kLossThreads), 0, stream,
                         nparts, part, by_mask, normalizer, static_cast<const T*>(nullptr),
                         static_cast<T*>(out));
    }
  }
  return status_of_launch();
}

template <typename T, typename TargetT>
int launch_fused_backward(int64_t N, int64_t S, int64_t C, int64_t ignore_index, int reduction,
                          const void* prob, const void* target, const void* dl, void* dx,
                          void* scratch, hipStream_t stream) {
  constexpr int kVec = IO<T>::kVec;
  const T* pp = static_cast<const T*>(prob);
  const TargetT* tp = static_cast<const TargetT*>(target);
  const T* dlp = static_cast<const T*>(dl);
  T* dp = static_cast<T*>(dx);
  T* part = static_cast<T*>(scratch);
  T* scalar = part + 2 * kMaxPartials;
  const int64_t NxS = N * S, total = N * C * S;
  if (reduction != kNone) {
    const float normalizer = loss_normalizer(reduction, N, S, true);
    const bool by_mask = normalizer < 0.f;
    if (!by_mask || NxS <= kDirectReduceMax) {
      hipLaunchKernelGGL((loss_reduce_direct<T, TargetT, kGradScale, true>), dim3(1),
                         dim3(kDirectThreads), 0, stream, static_cast<int64_t>(0),
                         static_cast<const T*>(nullptr), by_mask ? NxS : static_cast<int64_t>(0),
                         static_cast<const T*>(nullptr), tp, C, ignore_index, by_mask, normalizer,
                         dlp, scalar);
    } else {
      const int nparts = partial_blocks(NxS);
      hipLaunchKernelGGL((valid_target_partial_counts<T, TargetT>), dim3(nparts),
                         dim3(kLossThreads), 0, stream, NxS, C, ignore_index, tp, part);
      hipLaunchKernelGGL((loss_finalize<T, kGradScale>), dim3(1), dim3(kLossThreads), 0, stream,
                         nparts, part, by_mask, normalizer, dlp, scalar);
    }
  }
  const bool aligned = aligned16(prob) && aligned16(dx);
#define LAUNCH(VEC, ALONG_C, PER_POS)                                                          \
  hipLaunchKernelGGL((softmax_ce_backward<T, TargetT, VEC, ALONG_C, PER_POS>),                 \
                     dim3(loss_grid(total / VEC)), dim3(kLossThreads), 0, stream, total / VEC, \
                     S, C, ignore_index, pp, tp, dlp, scalar, dp)
  if (S == 1 && total % kVec == 0 && aligned && C >= kVec && C < (int64_t(1) << 30)) {
    // a packet touches two rows at most, and a chunk's offsets fit 32 bits
    const int64_t npackets = total / kVec;
    const int64_t chunks = ceil_div(npackets, static_cast<int64_t>(kLossThreads) * 4);
    const int64_t cap = static_cast<int64_t>(num_cus()) * 64;
    const dim3 grid(static_cast<unsigned>(chunks < cap ? chunks : cap));
    if (reduction == kNone) {
      hipLaunchKernelGGL((softmax_ce_backward_chunks<T, TargetT, true>), grid, dim3(kLossThreads), 0,
                         stream, npackets, C, ignore_index, pp, tp, dlp, scalar, dp);
    } else {
      hipLaunchKernelGGL((softmax_ce_backward_chunks<T, TargetT, false>), grid, dim3(kLossThreads),
                         0, stream, npackets, C, ignore_index, pp, tp, dlp, scalar, dp);
    }
  } else if (S == 1 && total % kVec == 0 && aligned) {
    if (reduction == kNone) LAUNCH(kVec, true, true); else LAUNCH(kVec, true, false);
  } else if (S > 1 && S % kVec == 0 && aligned && C * S < (int64_t(1) << 30)) {
    const int64_t npackets = total / kVec;
    const int64_t chunks = ceil_div(npackets, static_cast<int64_t>(kLossThreads) * 4);
    const int64_t cap = static_cast<int64_t>(num_cus()) * 64;
    const dim3 grid(static_cast<unsigned>(chunks < cap ? chunks : cap));
    if (reduction == kNone) {
      hipLaunchKernelGGL((softmax_ce_backward_chunks_strided<T, TargetT, true>), grid,
                         dim3(kLossThreads), 0, stream, npackets, static_cast<uint32_t>(S),
                         static_cast<uint32_t>(C), ignore_index, pp, tp, dlp, scalar, dp);
    } else {
      hipLaunchKernelGGL((softmax_ce_backward_chunks_strided<T, TargetT, false>), grid,
                         dim3(kLossThreads), 0, stream, npackets, static_cast<uint32_t>(S),
                         static_cast<uint32_t>(C), ignore_index, pp, tp, dlp, scalar, dp);
    }
  } else if (S > 1 && S % kVec == 0 && aligned) {
    if (reduction == kNone) LAUNCH(kVec, false, true); else LAUNCH(kVec, false, false);
  } else {
    if (reduction == kNone) LAUNCH(1, false, true); else LAUNCH(1, false, false);
  }
#undef LAUNCH
  return status_of_launch();
}

inline bool loss_dtype_ok(int dtype) { return dtype == DRAGON_HIP_F32 || dtype == DRAGON_HIP_F64; }
inline bool target_dtype_ok(int t) { return t == DRAGON_HIP_I32 || t == DRAGON_HIP_I64; }
inline size_t loss_elem(int dtype) { return dtype == DRAGON_HIP_F64 ? 8 : 4; }

// Calls FN<T, TargetT>(args...) for T in {float, double}, TargetT in {int32, int64}.
#define DRAGON_HIP_DISPATCH_LOSS(dtype, target_dtype, FN, ...)                      \
  if (dtype == DRAGON_HIP_F32) {                                                    \
    return target_dtype == DRAGON_HIP_I32 ? FN<float, int32_t>(__VA_ARGS__)         \
                                          : FN<float, int64_t>(__VA_ARGS__);        \
  }                                                                                 \
  return target_dtype == DRAGON_HIP_I32 ? FN<double, int32_t>(__VA_ARGS__)          \
                                        : FN<double, int64_t>(__VA_ARGS__)

#define DRAGON_HIP_DISPATCH_LOSS_T(dtype, FN, ...)         \
  if (dtype == DRAGON_HIP_F32) return FN<float>(__VA_ARGS__); \
  return FN<double>(__VA_ARGS__)

} // namespace
} // namespace dragon_hip

extern "C" {

using namespace dragon_hip;

int dragon_hip_cross_entropy(int dtype, int64_t N, const void* input, const void* target,
                             void* loss, void* stream) {
  if (!loss_dtype_ok(dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0) return DRAGON_HIP_EINVAL;
  if (N == 0) return DRAGON_HIP_OK;
  if (!input || !target || !loss) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS_T(dtype, launch_cross_entropy, N, input, target, loss, s);
}

int dragon_hip_sparse_cross_entropy(int dtype, int target_dtype, int64_t N, int64_t S, int64_t C,
                                    int64_t ignore_index, const void* input, const void* target,
                                    void* loss, void* mask, void* stream) {
  if (!loss_dtype_ok(dtype) || !target_dtype_ok(target_dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || S < 0 || C <= 0) return DRAGON_HIP_EINVAL;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!input || !target || !loss || !mask) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS(dtype, target_dtype, launch_sparse_cross_entropy, N, S, C, ignore_index,
                           input, target, loss, mask, s);
}

int dragon_hip_softmax_cross_entropy_grad(int dtype, int target_dtype, int64_t N, int64_t S,
                                          int64_t C, int64_t ignore_index, const void* input,
                                          const void* target, void* dx, void* mask, void* stream) {
  (void)input;  // the probabilities are already in dx (cross_entropy_kernel.cc:80-108)
  if (!loss_dtype_ok(dtype) || !target_dtype_ok(target_dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || S < 0 || C <= 0) return DRAGON_HIP_EINVAL;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!target || !dx || !mask) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS(dtype, target_dtype, launch_softmax_ce_grad, N, S, C, ignore_index,
                           target, dx, mask, s);
}

size_t dragon_hip_reduce_loss_scratch_bytes(int dtype) {
  return loss_dtype_ok(dtype) ? reduce_loss_scratch(loss_elem(dtype)) : 0;
}

int dragon_hip_reduce_loss(int dtype, int64_t N, int64_t num_masks, float normalizer,
                           const void* x, const void* mask, void* y, void* scratch,
                           size_t scratch_bytes, void* stream) {
  if (!loss_dtype_ok(dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || num_masks < 0 || !y || (N > 0 && !x)) return DRAGON_HIP_EINVAL;
  if (num_masks > 0 && normalizer < 0.f && !mask) return DRAGON_HIP_EINVAL;
  if (!scratch || scratch_bytes < reduce_loss_scratch(loss_elem(dtype))) return DRAGON_HIP_ESCRATCH;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS_T(dtype, launch_reduce_loss, N, num_masks, normalizer, x, mask, y,
                             scratch, s);
}

int dragon_hip_reduce_loss_grad(int dtype, int64_t N, int64_t num_masks, float normalizer,
                                const void* dl, const void* mask, void* dx, void* scratch,
                                size_t scratch_bytes, void* stream) {
  if (!loss_dtype_ok(dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || num_masks < 0 || !dl) return DRAGON_HIP_EINVAL;
  if (N == 0) return DRAGON_HIP_OK;
  if (!dx || (num_masks > 0 && normalizer < 0.f && !mask)) return DRAGON_HIP_EINVAL;
  if (!scratch || scratch_bytes < reduce_loss_scratch(loss_elem(dtype))) return DRAGON_HIP_ESCRATCH;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS_T(dtype, launch_reduce_loss_grad, N, num_masks, normalizer, dl, mask, dx,
                             scratch, s);
}

int dragon_hip_broadcast_loss_grad(int dtype, int64_t N, int64_t S, int64_t C, const void* dl,
                                   void* dx, void* stream) {
  if (!loss_dtype_ok(dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || S < 0 || C < 0) return DRAGON_HIP_EINVAL;
  if (N * S * C == 0) return DRAGON_HIP_OK;
  if (!dl || !dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS_T(dtype, launch_broadcast_loss_grad, N, S, C, dl, dx, s);
}

size_t dragon_hip_softmax_cross_entropy_loss_scratch_bytes(int dtype, int64_t N, int64_t S,
                                                           int64_t C) {
  if (!loss_dtype_ok(dtype) || N < 0 || S < 0 || C <= 0) return 0;
  return dragon_hip::fused_loss_head_bytes(loss_elem(dtype), N, S) +
      dragon_hip_softmax_scratch_bytes(dtype, N, S, C);
}

int dragon_hip_softmax_cross_entropy_loss_forward(int dtype, int target_dtype, int64_t N, int64_t S,
                                                  int64_t C, int64_t ignore_index, int reduction,
                                                  const void* x, const void* target, void* prob,
                                                  void* loss, void* scratch, size_t scratch_bytes,
                                                  void* stream) {
  if (!loss_dtype_ok(dtype) || !target_dtype_ok(target_dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || S < 0 || C <= 0 || reduction < kNone || reduction > kValid) return DRAGON_HIP_EINVAL;
  if (!loss) return DRAGON_HIP_EINVAL;
  if (N * S > 0 && (!x || !target || !prob)) return DRAGON_HIP_EINVAL;
  if (N * S == 0 && reduction == kNone) return DRAGON_HIP_OK;
  if (!scratch ||
      scratch_bytes < dragon_hip_softmax_cross_entropy_loss_scratch_bytes(dtype, N, S, C)) {
    return DRAGON_HIP_ESCRATCH;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS(dtype, target_dtype, launch_fused_forward, N, S, C, ignore_index,
                           reduction, x, target, prob, loss, scratch, s);
}

int dragon_hip_softmax_cross_entropy_loss_backward(int dtype, int target_dtype, int64_t N,
                                                   int64_t S, int64_t C, int64_t ignore_index,
                                                   int reduction, const void* prob,
                                                   const void* target, const void* dl, void* dx,
                                                   void* scratch, size_t scratch_bytes,
                                                   void* stream) {
  if (!loss_dtype_ok(dtype) || !target_dtype_ok(target_dtype)) return DRAGON_HIP_EDTYPE;
  if (N < 0 || S < 0 || C <= 0 || reduction < kNone || reduction > kValid) return DRAGON_HIP_EINVAL;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!prob || !target || !dl || !dx) return DRAGON_HIP_EINVAL;
  if (!scratch || scratch_bytes < reduce_loss_scratch(loss_elem(dtype))) return DRAGON_HIP_ESCRATCH;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_LOSS(dtype, target_dtype, launch_fused_backward, N, S, C, ignore_index,
                           reduction, prob, target, dl, dx, scratch, s);
}

} // extern "C"
