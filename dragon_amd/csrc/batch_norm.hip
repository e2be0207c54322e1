// BatchNorm kernels for gfx950.
//
// Replaces (dragon/kernels/normalization/op_kernels.h:36-109; CPU
// dragon/kernels/normalization/cpu/batch_norm_kernel.cc)
//   kernels::BatchNormExpectation   ex = sum(x)/normalizer, ex2 = sum(x^2)/normalizer
//   kernels::BatchNorm              scale = gamma*rsig, bias = beta - scale*mu,
//                                   y = x*scale[c] + bias[c]
//   kernels::BatchNormWGrad         dgamma = sum dy*(x-mu)*rsig, dbeta = sum dy
//   kernels::BatchNormTrainingGrad  dx = gamma*rsig*(dy - ((x-mu)*rsig*dgamma + dbeta)/normalizer)
//   kernels::BatchNormInferenceGrad dx = gamma*rsig*dy (+ WGrad)
// and fuses the training-forward operator body
// (dragon/operators/normalization/batch_norm_op.cc:49-82: Moments, two Axpby
// running-statistics updates, InvStd, BatchNorm) into two passes over x.
//
// x is [N, C, S] (NCHW) or [N, S, C] (NHWC). A channel's N*S values do not
// fit one compute unit (800 KB per channel at 64x56x56 fp32), so per-channel
// reductions are split over many workgroups (C alone cannot fill 256 compute
// units either). Two structures:
//   * split path (any layout and alignment): statistics and normalisation are
//     separate passes over x; the partial sums are finished by a [C]-sized
//     kernel that also carries every [C]-sized epilogue, so no separate
//     InvStd / Axpby / fused-params launches remain;
//   * single-read path (NCHW, whole packets; training forward and backward):
//     the slices of a channel stay in the registers of several workgroups,
//     which exchange their partial sums through HBM inside one kernel, so x
//     (and dy) is read once: 2 tensor passes forward and 3 backward instead of
//     3 and 5.
#include "long_rows.h"
#include "reduce.h"
#include "short_rows.h"
#include "slices.h"

// Scratch of dragon_hip_batch_norm_training_forward_noalloc: device memory that
// exists from the moment the library is loaded, so the entry point never
// allocates. Every device that runs the library holds its own copy at its own
// address; in host code the name below is a stand-in for the symbol, not a
// device address, and only static_scratch_on_current_device() may mention it.
static __device__ __align__(256) unsigned char scratch[DRAGON_HIP_STATIC_SCRATCH_BYTES];

namespace dragon_hip {
namespace {

struct ChannelShape {
  uint32_t N, C, S;
  bool nchw;
};

inline SegmentedReduce channel_segments(const ChannelShape& sh) {
  SegmentedReduce s{sh.C, sh.C, 0, sh.S, sh.N, sh.S, sh.C * sh.S, 1};
  s.split = pick_split(sh.C, static_cast<int64_t>(sh.N) * sh.S);
  return s;
}
inline size_t channel_scratch_bytes(const ChannelShape& sh, size_t acc_bytes) {
  const uint32_t split = sh.nchw ? channel_segments(sh).split
                                 : column_split_bound(static_cast<int64_t>(sh.N) * sh.S, sh.C);
  size_t pairs = static_cast<size_t>(sh.C) * split;
  // one pair per (n, c) row where the rows may take the short- or long-row kernels
  if (sh.nchw && pairs < static_cast<size_t>(sh.N) * sh.C) {
    pairs = static_cast<size_t>(sh.N) * sh.C;
  }
  return pairs * 2 * acc_bytes;
}

// NCHW tensors whose (n, c) rows of S elements are not whole aligned packets
// (14x14 and 7x7 feature maps in 16-bit types): the rows go through the
// LDS-staged short-row kernel (short_rows.h), which reads and writes aligned
// packets whatever S is. A reduction leaves one pair per (n, c) row, summed
// over n by the column finalize; a map fetches its channel's parameters once
// per row.
inline bool ragged_channel_rows(const ChannelShape& sh, size_t elem_bytes, const void* a,
                                const void* b, const void* c) {
  const int vec = static_cast<int>(16 / elem_bytes);
  const bool packets = sh.S % vec == 0 && aligned16(a) && aligned16(b) && aligned16(c);
  return sh.nchw && !packets && congruent16(a, b) && congruent16(a, c);
}
inline bool short_channel_rows(const ChannelShape& sh, size_t elem_bytes, const void* a,
                               const void* b, const void* c) {
  return sh.S <= 1024 && ragged_channel_rows(sh, elem_bytes, a, b, c);
}
// Longer rows of that kind (35x35, 71x71 maps): one wavefront per row (long_rows.h).
inline bool long_channel_rows(const ChannelShape& sh, size_t elem_bytes, const void* a,
                              const void* b, const void* c) {
  return sh.S > 1024 && ragged_channel_rows(sh, elem_bytes, a, b, c);
}

template <typename T, int kE, typename F, int kInputs>
struct ChannelRowSumsOp {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = kInputs;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 1;
  static constexpr bool kReadOnly = true;
  F f;
  uint32_t C, S;
  A* partial;  // [N][C] pairs
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[1]) const {
    const uint32_t c = static_cast<uint32_t>(row % C);
    F g = f;
    g.begin(c, c * S);
    w[0] = g.state();
  }
  // the same for the one-wavefront-per-row kernel (long_rows.h)
  static constexpr int kParams = 1;
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[1]) const { fetch_side(row, w); }
  __device__ __forceinline__ void add(const A* w, A x0, A x1, A& a, A& b) const {
    F g = f;
    g.set_state(w[0]);
    g.add(0u, 0u, 0u, x0, x1, a, b);
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A* side, int l, int width, A (&v0)[kE],
                                      const A (&v1)[kE]) const {
    F g = f;
    g.set_state(side[0]);
    A a = A(0), b = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      if (l + j * kL < width) g.add(0u, 0u, 0u, v0[j], v1[j], a, b);
    }
    a = group_allreduce<kL>(a, SumOp());
    b = group_allreduce<kL>(b, SumOp());
    if (l == 0) {
      partial[2 * r] = a;
      partial[2 * r + 1] = b;
    }
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename F, int kInputs>
struct RowSumsOf {
  template <typename T, int kE>
  using Op = ChannelRowSumsOp<T, kE, F, kInputs>;
};

template <typename T, int kE, typename F, int kInputs>
struct ChannelRowMapOp {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = kInputs;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = F::kParams;
  F f;
  uint32_t C;
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  __device__ __forceinline__ void fetch_side(int64_t row, A (&w)[F::kParams]) const {
    f.params(static_cast<uint32_t>(row % C), w);
  }
  static constexpr int kParams = F::kParams;
  __device__ __forceinline__ void row_params(int64_t row, A (&w)[F::kParams]) const {
    fetch_side(row, w);
  }
  __device__ __forceinline__ A apply(const A* w, A x0, A x1) const { return f.apply(w, x0, x1); }
  template <int kL>
  __device__ __forceinline__ void row(int64_t, const A* side, int, int, A (&v0)[kE],
                                      const A (&v1)[kE]) const {
#pragma unroll
    for (int j = 0; j < kE; ++j) v0[j] = f.apply(side, v0[j], v1[j]);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename F, int kInputs>
struct RowMapOf {
  template <typename T, int kE>
  using Op = ChannelRowMapOp<T, kE, F, kInputs>;
};

// Runs the split reduction of accumulator F (one or two inputs) over every
// channel and hands the per-channel totals to epilogue E.
template <typename T, int kIn, typename F, typename E>
void reduce_channels(const ChannelShape& sh, const T* in0, const T* in1, F f, E e,
                     typename IO<T>::Acc* part, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const unsigned fin_grid = static_cast<unsigned>(ceil_div(sh.C, kReduceThreads));
  ShortPlan sp;
  auto lds_of = [](const ShortPlan& q) {
    return static_cast<size_t>(q.stage_packets) * 16 * kIn + q.rows_per_chunk * sizeof(A);
  };
  if (short_channel_rows(sh, sizeof(T), in0, in1, in0) &&
      plan_short_rows_within(sh.S, sizeof(T), kIn == 1 ? 4 : 3, false, lds_of, &sp)) {
    using Holder = RowSumsOf<F, kIn>;
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    const size_t lds = lds_of(sp);
    T* none = nullptr;
    DRAGON_HIP_SHORT_LAUNCH(T, typename Holder::template Op, sp, lds,
                            short_grid(rows, sp.rows_per_chunk), stream, rows,
                            static_cast<int>(sh.S), in0, in1, none, f, sh.C, sh.S, part);
    launch_reduce2_finalize<A, E>(sh.C, sh.N, false, part, e, stream);
    return;
  }
  // (Fewer than 2048 such rows are too few wavefronts: they go to the split
  // segment reduction below, through their packet windows. [16,32,225,225] bf16,
  // 512 rows: 104 us a wavefront per row, 30 us split.)
  if (long_channel_rows(sh, sizeof(T), in0, in1, in0) &&
      !(sizeof(T) <= 4 && static_cast<int64_t>(sh.N) * sh.C < 2048)) {
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    const ChannelRowSumsOp<T, 8, F, kIn> op{f, sh.C, sh.S, part};
    hipLaunchKernelGGL((long_rows_sums<T, kIn, ChannelRowSumsOp<T, 8, F, kIn>>),
                       dim3(long_rows_grid(rows)), dim3(kLongThreads), 0, stream, rows,
                       static_cast<int>(sh.S), in0, in1, op, part);
    launch_reduce2_finalize<A, E>(sh.C, sh.N, false, part, e, stream);
    return;
  }
  if (sh.nchw) {
    const SegmentedReduce s = channel_segments(sh);
    const dim3 grid(s.n_out * s.split);
    const bool vec_ok = aligned16(in0) && aligned16(in1) && sh.S % kVec == 0;
    if (vec_ok) {
      hipLaunchKernelGGL((reduce2_segments<T, kIn, kVec, F>), grid, dim3(kReduceThreads), 0, stream,
                         s, in0, in1, f, part);
    } else if (sizeof(T) <= 4 && sh.S >= 4u * kVec && congruent16(in0, in1)) {
      hipLaunchKernelGGL((reduce2_segments_windows<T, kIn, F>), grid, dim3(kReduceThreads), 0,
                         stream, s, in0, in1, f, part);
    } else {
      hipLaunchKernelGGL((reduce2_segments<T, kIn, 1, F>), grid, dim3(kReduceThreads), 0, stream, s,
                         in0, in1, f, part);
    }
    hipLaunchKernelGGL((reduce2_finalize<A, E>), dim3(fin_grid), dim3(kReduceThreads), 0, stream,
                       sh.C, s.split, true, part, e);
  } else {
    const uint32_t split = launch_reduce2_columns<T, kIn, F>(sh.N * sh.S, sh.C, in0, in1, f, part,
                                                             stream);
    launch_reduce2_finalize<A, E>(sh.C, split, false, part, e, stream);
  }
}

// ---------------------------------------------------------------- accumulators

template <typename T>
struct SumSqAccum {  // a = sum x, b = sum x^2
  using A = typename IO<T>::Acc;
  __device__ __forceinline__ void begin(uint32_t, uint32_t) {}
  // the per-output scalar that begin() fetched (none here)
  __device__ __forceinline__ A state() const { return A(0); }
  __device__ __forceinline__ void set_state(A) {}
  template <int V>
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, uint32_t, const A (&x)[V],
                                      const A (&)[V], A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      a += x[e];
      b += x[e] * x[e];
    }
  }
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, A x, A, A& a, A& b) const {
    a += x;
    b += x * x;
  }
};

template <typename T>
struct ShiftedSumSqAccum {  // a = sum (x-s), b = sum (x-s)^2, s = first value of the channel
  using A = typename IO<T>::Acc;
  const T* x;
  A shift;
  __device__ __forceinline__ void begin(uint32_t, uint32_t first_off) {
    shift = load_shift(x + first_off);
  }
  __device__ __forceinline__ A state() const { return shift; }
  __device__ __forceinline__ void set_state(A v) { shift = v; }
  template <int V>
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, uint32_t, const A (&v)[V],
                                      const A (&)[V], A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const A d = v[e] - shift;
      a += d;
      b += d * d;
    }
  }
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, A v, A, A& a, A& b) const {
    const A d = v - shift;
    a += d;
    b += d * d;
  }
};

template <typename T>
struct WGradAccum {  // a = sum dy*(x-mu[c]), b = sum dy
  using A = typename IO<T>::Acc;
  const A* mu;
  A m;
  __device__ __forceinline__ void begin(uint32_t c, uint32_t) { m = mu[c]; }
  __device__ __forceinline__ A state() const { return m; }
  __device__ __forceinline__ void set_state(A v) { m = v; }
  template <int V>
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, uint32_t, const A (&x)[V],
                                      const A (&dy)[V], A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      a += dy[e] * (x[e] - m);
      b += dy[e];
    }
  }
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, A x, A dy, A& a, A& b) const {
    a += dy * (x - m);
    b += dy;
  }
};

// ---------------------------------------------------------------- epilogues

template <typename A>
struct ExpectationEpilogue {
  A normalizer;
  A* ex;
  A* ex2;
  __device__ __forceinline__ void operator()(uint32_t c, A a, A b) const {
    ex[c] = a / normalizer;
    ex2[c] = b / normalizer;
  }
};

template <typename A>
struct WGradEpilogue {
  const A* rsig;
  A* dgamma;
  A* dbeta;
  __device__ __forceinline__ void operator()(uint32_t c, A a, A b) const {
    dgamma[c] = a * rsig[c];
    dbeta[c] = b;
  }
};

// round(round(y*beta) + round(x*alpha)) as math::Axpby's Scale-then-Axpy pair.
template <typename A>
__device__ __forceinline__ A scale_then_axpy(A y, A beta, A x, A alpha) {
#pragma clang fp contract(off)
  const A scaled = y * beta;
  const A prod = x * alpha;
  return scaled + prod;
}

// scale = gamma*rsig; bias = beta - round(scale*mu) as the reference's array expression.
template <typename A>
__device__ __forceinline__ void fused_params(A mu, A rsig, A gamma, A beta, A* scale, A* bias) {
#pragma clang fp contract(off)
  const A s = gamma * rsig;
  const A p = s * mu;
  *scale = s;
  *bias = beta - p;
}

// Everything [C]-sized of the training forward in one epilogue: mean/var from
// the shifted sums, running statistics, rsig, scale and bias.
template <typename T>
struct TrainingStatsEpilogue {
  using A = typename IO<T>::Acc;
  const T* x;
  uint32_t chan_stride;  // S for NCHW, 1 for NHWC
  A inv_n, momentum, one_minus_momentum, eps;
  const A* gamma;
  const A* beta;
  A* running_mean;
  A* running_var;
  A* mu;
  A* rsig;
  A* scale;
  A* bias;
  __device__ __forceinline__ void operator()(uint32_t c, A a, A b) const {
    const A shift = load_shift(x + c * chan_stride);
    const A d = a * inv_n;
    const A mean = shift + d;
    const A var = b * inv_n - d * d;
    running_mean[c] = scale_then_axpy(running_mean[c], momentum, mean, one_minus_momentum);
    running_var[c] = scale_then_axpy(running_var[c], momentum, var, one_minus_momentum);
    const A rs = acc_rsqrt_exact(var + eps);
    mu[c] = mean;
    rsig[c] = rs;
    fused_params(mean, rs, gamma[c], beta[c], scale + c, bias + c);
  }
};

template <typename A>
__global__ __launch_bounds__(256) void fused_params_kernel(const uint32_t C, const A* mu,
                                                           const A* rsig, const A* gamma,
                                                           const A* beta, A* scale, A* bias) {
  const uint32_t c = blockIdx.x * 256 + threadIdx.x;
  if (c < C) fused_params(mu[c], rsig[c], gamma[c], beta[c], scale + c, bias + c);
}

// ---------------------------------------------------------------- maps

// Channel of the first element of a packet, and whether the packet spans kVec
// consecutive channels (NHWC) or one channel (NCHW).
struct ChannelIndex {
  ChannelShape sh;
  __device__ __forceinline__ uint32_t operator()(uint32_t i) const {
    return sh.nchw ? (i / sh.S) % sh.C : i % sh.C;
  }
};

// kVec consecutive per-channel parameters starting at channel c (NHWC packets).
template <int kVec, typename A>
__device__ __forceinline__ void load_channel_params(const A* p, uint32_t c, A (&v)[kVec]) {
  if constexpr (kVec == 1) {
    v[0] = p[c];
  } else {
    load_params_ragged<kVec>(p + c, kVec, v);
  }
}

template <typename T, int kVec>
struct AffineApply {  // y = x*scale[c] + bias[c]
  using A = typename IO<T>::Acc;
  ChannelIndex idx;
  const A* scale;
  const A* bias;
  // The same map with the channel's parameters fetched once per row (NCHW).
  static constexpr int kParams = 2;
  __device__ __forceinline__ void params(uint32_t c, A (&w)[kParams]) const {
    w[0] = scale[c], w[1] = bias[c];
  }
  __device__ __forceinline__ A apply(const A* w, A x, A) const { return x * w[0] + w[1]; }
  __device__ __forceinline__ void operator()(uint32_t i, A (&v)[kVec], const A (&)[kVec]) const {
    const uint32_t c = idx(i);
    if (idx.sh.nchw) {
      const A s = scale[c], b = bias[c];
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = v[e] * s + b;
    } else {
      A s[kVec], b[kVec];
      load_channel_params<kVec>(scale, c, s);
      load_channel_params<kVec>(bias, c, b);
#pragma unroll
      for (int e = 0; e < kVec; ++e) v[e] = v[e] * s[e] + b[e];
    }
  }
};

template <typename T, int kVec>
struct TrainingGradApply {
  using A = typename IO<T>::Acc;
  ChannelIndex idx;
  const A* mu;
  const A* rsig;
  const A* gamma;
  const A* dgamma;
  const A* dbeta;
  A normalizer;
  static constexpr int kParams = 5;
  __device__ __forceinline__ void params(uint32_t c, A (&w)[kParams]) const {
    w[0] = rsig[c], w[1] = mu[c], w[2] = gamma[c] * w[0], w[3] = dgamma[c], w[4] = dbeta[c];
  }
  __device__ __forceinline__ A apply(const A* w, A x, A dy) const {
    return w[2] * (dy - ((x - w[1]) * w[0] * w[3] + w[4]) / normalizer);
  }
  __device__ __forceinline__ void operator()(uint32_t i, A (&x)[kVec], const A (&dy)[kVec]) const {
    const uint32_t c = idx(i);
    if (idx.sh.nchw) {
      const A r = rsig[c], m = mu[c], g = gamma[c] * r, dg = dgamma[c], db = dbeta[c];
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        x[e] = g * (dy[e] - ((x[e] - m) * r * dg + db) / normalizer);
      }
    } else {
      A r[kVec], m[kVec], g[kVec], dg[kVec], db[kVec];
      load_channel_params<kVec>(rsig, c, r);
      load_channel_params<kVec>(mu, c, m);
      load_channel_params<kVec>(gamma, c, g);
      load_channel_params<kVec>(dgamma, c, dg);
      load_channel_params<kVec>(dbeta, c, db);
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const A x_norm = (x[e] - m[e]) * r[e];
        x[e] = g[e] * r[e] * (dy[e] - (x_norm * dg[e] + db[e]) / normalizer);
      }
    }
  }
};

template <typename T, int kVec>
struct InferenceGradApply {  // dx = dy * gamma[c] * rsig[c]
  using A = typename IO<T>::Acc;
  ChannelIndex idx;
  const A* rsig;
  const A* gamma;
  static constexpr int kParams = 1;
  __device__ __forceinline__ void params(uint32_t c, A (&w)[kParams]) const {
    w[0] = gamma[c] * rsig[c];
  }
  __device__ __forceinline__ A apply(const A* w, A dy, A) const { return dy * w[0]; }
  __device__ __forceinline__ void operator()(uint32_t i, A (&dy)[kVec], const A (&)[kVec]) const {
    const uint32_t c = idx(i);
    if (idx.sh.nchw) {
      const A g = gamma[c] * rsig[c];
#pragma unroll
      for (int e = 0; e < kVec; ++e) dy[e] = dy[e] * g;
    } else {
      A g[kVec], r[kVec];
      load_channel_params<kVec>(gamma, c, g);
      load_channel_params<kVec>(rsig, c, r);
#pragma unroll
      for (int e = 0; e < kVec; ++e) dy[e] = dy[e] * (g[e] * r[e]);
    }
  }
};

template <typename T, int kIn, template <typename, int> class F, typename... Args>
void map_channels(const ChannelShape& sh, const T* in0, const T* in1, T* out, hipStream_t stream,
                  Args... args) {
  constexpr int kVec = IO<T>::kVec;
  using A = typename IO<T>::Acc;
  const uint32_t total = sh.N * sh.C * sh.S;
  const bool vec_ok = aligned16(in0) && aligned16(in1) && aligned16(out) &&
      (sh.nchw ? sh.S % kVec == 0 : sh.C % kVec == 0);
  ShortPlan sp;
  auto lds_of = [](const ShortPlan& q) {
    return static_cast<size_t>(q.stage_packets) * 16 * kIn +
        static_cast<size_t>(q.rows_per_chunk) * F<T, 1>::kParams * sizeof(A);
  };
  // Maps of 48 packets or more that are not whole aligned packets: the aligned
  // packets that cover the tensor, the channel found once per packet. Shorter
  // ones have a packet across two maps in every wavefront and do better staged
  // through LDS (bf16 7x7 with two inputs: 43 us against 32; fp32 15x15: 62
  // against 67 the other way).
  if (sizeof(T) <= 4 && sh.S / kVec >= 48 && ragged_channel_rows(sh, sizeof(T), in0, in1, out)) {
    using Fn = F<T, 1>;
    const ChannelRowMapOp<T, 8, Fn, kIn> op{Fn{ChannelIndex{sh}, args...}, sh.C};
    hipLaunchKernelGGL((map_flat_windows<T, kIn, ChannelRowMapOp<T, 8, Fn, kIn>>),
                       dim3(map_grid(total / kVec + 2)), dim3(256), 0, stream, total, sh.S, in0, in1,
                       out, op);
    return;
  }
  if (short_channel_rows(sh, sizeof(T), in0, in1, out) &&
      plan_short_rows_within(sh.S, sizeof(T), kIn == 1 ? 4 : 3, false, lds_of, &sp)) {
    using Fn = F<T, 1>;
    using Holder = RowMapOf<Fn, kIn>;
    const Fn fn{ChannelIndex{sh}, args...};
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    const size_t lds = lds_of(sp);
    DRAGON_HIP_SHORT_LAUNCH(T, typename Holder::template Op, sp, lds,
                            short_grid(rows, sp.rows_per_chunk), stream, rows,
                            static_cast<int>(sh.S), in0, in1, out, fn, sh.C);
    return;
  }
  if (long_channel_rows(sh, sizeof(T), in0, in1, out)) {  // (fp64 only: see above)
    using Fn = F<T, 1>;
    const int64_t rows = static_cast<int64_t>(sh.N) * sh.C;
    const ChannelRowMapOp<T, 8, Fn, kIn> op{Fn{ChannelIndex{sh}, args...}, sh.C};
    hipLaunchKernelGGL((long_rows_map<T, kIn, ChannelRowMapOp<T, 8, Fn, kIn>>),
                       dim3(long_rows_grid(rows)), dim3(kLongThreads), 0, stream, rows,
                       static_cast<int>(sh.S), in0, in1, out, op);
    return;
  }
  if (vec_ok) {
    F<T, kVec> f{ChannelIndex{sh}, args...};
    hipLaunchKernelGGL((map_flat<T, kIn, kVec, F<T, kVec>>), dim3(map_grid(total / kVec)), dim3(256),
                       0, stream, total, in0, in1, out, f);
  } else {
    F<T, 1> f{ChannelIndex{sh}, args...};
    hipLaunchKernelGGL((map_flat<T, kIn, 1, F<T, 1>>), dim3(map_grid(total)), dim3(256), 0, stream,
                       total, in0, in1, out, f);
  }
}

// ---------------------------------------------------------------- single-read path
//
// Training forward and backward of NCHW tensors as policies of the slice
// kernel (slices.h): a channel is the reduction unit, N runs of S elements.
inline SliceUnits channel_units(const ChannelShape& sh) {
  return SliceUnits{sh.C, sh.N, sh.S, sh.S, sh.C * sh.S};
}

template <typename T>
struct CoopForward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr bool kBeginReadsInput = true;
  static constexpr bool kWindows = true;
  static constexpr bool kWholeUnits = true;
  using Merge = PairSum;
  A inv_n, momentum, one_minus_momentum, eps;
  const A* gamma;
  const A* beta;
  A* running_mean;
  A* running_var;
  A* mu;
  A* rsig;
  A* scale;
  A* bias;
  A shift, sc, bi;
  __device__ __forceinline__ void begin(uint32_t, uint32_t base, const T* x) {
    shift = load_shift(x + base);  // one sample of the channel
  }
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t, uint32_t, const A (&x)[V], const A (&)[V],
                                             A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const A t = x[e] - shift;
      a += t;
      b += t * t;
    }
  }
  __device__ __forceinline__ void neutral(A& x, A&) const { x = shift; }
  __device__ __forceinline__ void finish(uint32_t c, bool leader, A a, A b) {
    const A dm = a * inv_n;
    const A mean = shift + dm;
    const A var = b * inv_n - dm * dm;
    const A rs = acc_rsqrt_exact(var + eps);
    fused_params(mean, rs, gamma[c], beta[c], &sc, &bi);
    if (leader) {
      running_mean[c] = scale_then_axpy(running_mean[c], momentum, mean, one_minus_momentum);
      running_var[c] = scale_then_axpy(running_var[c], momentum, var, one_minus_momentum);
      mu[c] = mean;
      rsig[c] = rs;
      scale[c] = sc;
      bias[c] = bi;
    }
  }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t, uint32_t, A (&x)[V], const A (&)[V]) const {
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = x[e] * sc + bi;
  }
};

template <typename T>
struct CoopBackward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  static constexpr bool kWindows = true;
  static constexpr bool kWholeUnits = true;
  using Merge = PairSum;
  A normalizer;
  const A* mu;
  const A* rsig;
  const A* gamma;
  A* dgamma;
  A* dbeta;
  A m, r, gr, ca, cb;
  __device__ __forceinline__ void begin(uint32_t c, uint32_t, const T*) { m = mu[c], r = rsig[c]; }
  template <int V>
  __device__ __forceinline__ void accumulate(uint32_t, uint32_t, const A (&x)[V], const A (&dy)[V],
                                             A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      a += dy[e] * (x[e] - m);
      b += dy[e];
    }
  }
  __device__ __forceinline__ void neutral(A& x, A& dy) const { x = m, dy = A(0); }
  // dx = gamma*rsig*(dy - ((x-mu)*rsig*dgamma + dbeta)/normalizer), with everything that is
  // constant over the channel folded into coefficients: dx = gr*dy + (ca*(x-mu) + cb).
  __device__ __forceinline__ void finish(uint32_t c, bool leader, A a, A b) {
    const A dg = a * r, db = b;
    if (leader) {
      dgamma[c] = dg;
      dbeta[c] = db;
    }
    gr = gamma[c] * r;
    const A q = -gr / normalizer;
    ca = q * r * dg;
    cb = q * db;
  }
  template <int V>
  __device__ __forceinline__ void transform(uint32_t, uint32_t, A (&x)[V], const A (&dy)[V]) const {
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = gr * dy[e] + (ca * (x[e] - m) + cb);
  }
};

// ---------------------------------------------------------------- launchers

template <typename T>
int launch_expectation(const ChannelShape& sh, float normalizer, const void* x, void* ex, void* ex2,
                       void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  const T* xp = static_cast<const T*>(x);
  reduce_channels<T, 1>(sh, xp, xp, SumSqAccum<T>{},
                        ExpectationEpilogue<A>{A(normalizer), static_cast<A*>(ex), static_cast<A*>(ex2)},
                        static_cast<A*>(scratch), stream);
  return status_of_launch();
}

template <typename T>
int launch_batch_norm(const ChannelShape& sh, const void* x, const void* mu, const void* rsig,
                      const void* gamma, const void* beta, void* scale, void* bias, void* y,
                      hipStream_t stream) {
  using A = typename IO<T>::Acc;
  A* sp = static_cast<A*>(scale);
  A* bp = static_cast<A*>(bias);
  hipLaunchKernelGGL((fused_params_kernel<A>), dim3(static_cast<unsigned>(ceil_div(sh.C, 256))),
                     dim3(256), 0, stream, sh.C, static_cast<const A*>(mu),
                     static_cast<const A*>(rsig), static_cast<const A*>(gamma),
                     static_cast<const A*>(beta), sp, bp);
  const T* xp = static_cast<const T*>(x);
  map_channels<T, 1, AffineApply>(sh, xp, xp, static_cast<T*>(y), stream,
                                  static_cast<const A*>(sp), static_cast<const A*>(bp));
  return status_of_launch();
}

template <typename T>
int launch_wgrad(const ChannelShape& sh, const void* x, const void* mu, const void* rsig,
                 const void* dy, void* dgamma, void* dbeta, void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  reduce_channels<T, 2>(sh, static_cast<const T*>(x), static_cast<const T*>(dy),
                        WGradAccum<T>{static_cast<const A*>(mu), A(0)},
                        WGradEpilogue<A>{static_cast<const A*>(rsig), static_cast<A*>(dgamma),
                                         static_cast<A*>(dbeta)},
                        static_cast<A*>(scratch), stream);
  return status_of_launch();
}

template <typename T>
int launch_training_grad(const ChannelShape& sh, float normalizer, const void* x, const void* mu,
                         const void* rsig, const void* gamma, const void* dgamma, const void* dbeta,
                         const void* dy, void* dx, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  map_channels<T, 2, TrainingGradApply>(
      sh, static_cast<const T*>(x), static_cast<const T*>(dy), static_cast<T*>(dx), stream,
      static_cast<const A*>(mu), static_cast<const A*>(rsig), static_cast<const A*>(gamma),
      static_cast<const A*>(dgamma), static_cast<const A*>(dbeta), A(normalizer));
  return status_of_launch();
}

template <typename T>
int launch_inference_grad(const ChannelShape& sh, const void* rsig, const void* gamma,
                          const void* dy, void* dx, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  const T* dyp = static_cast<const T*>(dy);
  map_channels<T, 1, InferenceGradApply>(sh, dyp, dyp, static_cast<T*>(dx), stream,
                                         static_cast<const A*>(rsig), static_cast<const A*>(gamma));
  return status_of_launch();
}

template <typename T>
int launch_training_forward(const ChannelShape& sh, float momentum, float eps, const void* x,
                            const void* gamma, const void* beta, void* running_mean,
                            void* running_var, void* mu, void* rsig, void* params, void* y,
                            void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  const T* xp = static_cast<const T*>(x);
  A* pp = static_cast<A*>(params);
  const float one_minus = 1.f - momentum;  // evaluated in float as the operator does
  TrainingStatsEpilogue<T> e{xp,
                             sh.nchw ? sh.S : 1u,
                             A(1) / A(static_cast<int64_t>(sh.N) * sh.S),
                             A(momentum),
                             A(one_minus),
                             A(eps),
                             static_cast<const A*>(gamma),
                             static_cast<const A*>(beta),
                             static_cast<A*>(running_mean),
                             static_cast<A*>(running_var),
                             static_cast<A*>(mu),
                             static_cast<A*>(rsig),
                             pp,
                             pp + sh.C};
  const CoopForward<T> op{e.inv_n, e.momentum, e.one_minus_momentum, e.eps, e.gamma, e.beta,
                          e.running_mean, e.running_var, e.mu, e.rsig, e.scale, e.bias,
                          A(0), A(0), A(0)};
  const int st = !sh.nchw ? kNotApplicable
                          : try_channel_slices<T>(channel_units(sh), op, xp, xp, static_cast<T*>(y),
                                                  static_cast<A*>(scratch), stream);
  if (st != kNotApplicable) return st;
  reduce_channels<T, 1>(sh, xp, xp, ShiftedSumSqAccum<T>{xp, A(0)}, e, static_cast<A*>(scratch),
                        stream);
  map_channels<T, 1, AffineApply>(sh, xp, xp, static_cast<T*>(y), stream,
                                  static_cast<const A*>(pp), static_cast<const A*>(pp + sh.C));
  return status_of_launch();
}

// BatchNormWGrad + BatchNormTrainingGrad.
template <typename T>
int launch_training_backward(const ChannelShape& sh, float normalizer, const void* x, const void* mu,
                             const void* rsig, const void* gamma, const void* dy, void* dgamma,
                             void* dbeta, void* dx, void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  const CoopBackward<T> op{A(normalizer),
                           static_cast<const A*>(mu),
                           static_cast<const A*>(rsig),
                           static_cast<const A*>(gamma),
                           static_cast<A*>(dgamma),
                           static_cast<A*>(dbeta),
                           A(0), A(0), A(0), A(0), A(0)};
  int st = !sh.nchw ? kNotApplicable
                    : try_channel_slices<T>(channel_units(sh), op, static_cast<const T*>(x),
                                            static_cast<const T*>(dy), static_cast<T*>(dx),
                                            static_cast<A*>(scratch), stream);
  if (st != kNotApplicable) return st;
  st = launch_wgrad<T>(sh, x, mu, rsig, dy, dgamma, dbeta, scratch, stream);
  if (st != DRAGON_HIP_OK) return st;
  return launch_training_grad<T>(sh, normalizer, x, mu, rsig, gamma, dgamma, dbeta, dy, dx, stream);
}

int make_shape(int64_t N, int64_t C, int64_t S, int layout, ChannelShape* sh) {
  if (N < 0 || C <= 0 || S < 0) return DRAGON_HIP_EINVAL;
  if (layout != DRAGON_HIP_NCHW && layout != DRAGON_HIP_NHWC) return DRAGON_HIP_EINVAL;
  if (!fits_int32(N * C * S)) return DRAGON_HIP_EINVAL;
  sh->N = static_cast<uint32_t>(N), sh->C = static_cast<uint32_t>(C);
  // [N, C, 1] and [N, 1, C] are the same memory: with S == 1 a channel is a
  // column of the [N, C] matrix, whatever the layout tag says.
  sh->S = static_cast<uint32_t>(S), sh->nchw = layout == DRAGON_HIP_NCHW && S != 1;
  return DRAGON_HIP_OK;
}

inline size_t acc_bytes(int dtype) { return dtype == DRAGON_HIP_F64 ? 8 : 4; }

// The split reduction's partial pairs or the single-read path's, whichever is larger.
template <typename T>
size_t scratch_bytes_of(const ChannelShape& sh, size_t* out) {
  const size_t split = channel_scratch_bytes(sh, sizeof(typename IO<T>::Acc));
  const size_t coop = sh.nchw ? coop_scratch_bytes<T>(channel_units(sh), true) : 0;
  *out = split > coop ? split : coop;
  return *out;
}
inline size_t scratch_bytes_for(int dtype, const ChannelShape& sh) {
  size_t bytes = 0;
  switch (dtype) {
    case DRAGON_HIP_F16: scratch_bytes_of<f16_t>(sh, &bytes); break;
    case DRAGON_HIP_BF16: scratch_bytes_of<bf16_t>(sh, &bytes); break;
    case DRAGON_HIP_F32: scratch_bytes_of<float>(sh, &bytes); break;
    case DRAGON_HIP_F64: scratch_bytes_of<double>(sh, &bytes); break;
    default: break;
  }
  return bytes;
}

inline int check_scratch(const ChannelShape& sh, int dtype, const void* scratch, size_t bytes) {
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  return (scratch && bytes >= scratch_bytes_for(dtype, sh)) ? DRAGON_HIP_OK : DRAGON_HIP_ESCRATCH;
}

template <typename T>
int exchange_plan_of(const SliceUnits& u, int tensors, int* slices, int* slice_packets,
                     int* packets_per_thread, int* grid) {
  const CoopPlan p = plan_coop<T>(u, tensors);
  if (!p.ok) return 0;
  *slices = static_cast<int>(p.K);
  *slice_packets = static_cast<int>(p.slice);
  *packets_per_thread = p.r;
  *grid = static_cast<int>(coop_grid(coop_rmax(tensors), tensors));
  return 1;
}

// The device address of the static array on the current device, resolved on
// the first call on that device and kept per device.
int static_scratch_on_current_device(void** ptr) {
  static std::atomic<void*> resolved[kMaxDevices];
  int device = 0;
  const hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return static_cast<int>(e);
  if (device < 0 || device >= kMaxDevices) return DRAGON_HIP_EINVAL;
  void* p = resolved[device].load(std::memory_order_acquire);
  if (!p) {
    const hipError_t g = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (g != hipSuccess) return static_cast<int>(g);
    resolved[device].store(p, std::memory_order_release);
  }
  *ptr = p;
  return DRAGON_HIP_OK;
}

} // namespace
} // namespace dragon_hip

extern "C" {

using dragon_hip::ChannelShape;

size_t dragon_hip_batch_norm_reduce_scratch_bytes(int dtype, int64_t N, int64_t C, int64_t S,
                                                  int layout) {
  ChannelShape sh;
  if (dragon_hip::make_shape(N, C, S, layout, &sh) != DRAGON_HIP_OK || N * S == 0) return 0;
  return dragon_hip::scratch_bytes_for(dtype, sh);
}

int dragon_hip_batch_norm_expectation(int dtype, int64_t N, int64_t C, int64_t S,
                                      float normalizer, int layout, const void* x, void* ex,
                                      void* ex2, void* scratch, size_t scratch_bytes,
                                      void* stream) {
  ChannelShape sh;
  int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (!ex || !ex2) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (N * S == 0) {
    const int acc_tag = dtype == DRAGON_HIP_F64 ? DRAGON_HIP_F64 : DRAGON_HIP_F32;
    const int e1 = dragon_hip_set(acc_tag, C, 0.f, ex, s);
    return e1 != DRAGON_HIP_OK ? e1 : dragon_hip_set(acc_tag, C, 0.f, ex2, s);
  }
  if (!x) return DRAGON_HIP_EINVAL;
  if ((st = dragon_hip::check_scratch(sh, dtype, scratch, scratch_bytes)) != DRAGON_HIP_OK) return st;
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_expectation, sh, normalizer, x, ex, ex2,
                            scratch, s);
}

int dragon_hip_batch_norm(int dtype, int64_t N, int64_t C, int64_t S, int layout, const void* x,
                          const void* mu, const void* rsig, const void* gamma,
                          const void* beta, void* scale, void* bias, void* y, void* stream) {
  ChannelShape sh;
  const int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (!mu || !rsig || !gamma || !beta || !scale || !bias) return DRAGON_HIP_EINVAL;
  if (N * S > 0 && (!x || !y)) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  // Aliasing conventions of the reference launcher.
  const size_t acc = dragon_hip::acc_bytes(dtype);
  if (scale == rsig) {
    scale = static_cast<char*>(const_cast<void*>(rsig)) + acc * C;
    bias = static_cast<char*>(const_cast<void*>(rsig)) + acc * C * 2;
  } else if (scale == bias) {
    bias = static_cast<char*>(scale) + acc * C;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_batch_norm, sh, x, mu, rsig, gamma, beta,
                            scale, bias, y, s);
}

int dragon_hip_batch_norm_wgrad(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                const void* x, const void* mu, const void* rsig, const void* dy,
                                void* dgamma, void* dbeta, void* scratch, size_t scratch_bytes,
                                void* stream) {
  ChannelShape sh;
  int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (!dgamma || !dbeta) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  const size_t acc = dragon_hip::acc_bytes(dtype);
  if (dgamma == dbeta) dbeta = static_cast<char*>(dgamma) + acc * C;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (N * S == 0) {
    const int acc_tag = dtype == DRAGON_HIP_F64 ? DRAGON_HIP_F64 : DRAGON_HIP_F32;
    const int e1 = dragon_hip_set(acc_tag, C, 0.f, dgamma, s);
    return e1 != DRAGON_HIP_OK ? e1 : dragon_hip_set(acc_tag, C, 0.f, dbeta, s);
  }
  if (!x || !mu || !rsig || !dy) return DRAGON_HIP_EINVAL;
  if ((st = dragon_hip::check_scratch(sh, dtype, scratch, scratch_bytes)) != DRAGON_HIP_OK) return st;
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_wgrad, sh, x, mu, rsig, dy, dgamma, dbeta,
                            scratch, s);
}

int dragon_hip_batch_norm_training_grad(int dtype, int64_t N, int64_t C, int64_t S,
                                        float normalizer, int layout, const void* x,
                                        const void* mu, const void* rsig, const void* gamma,
                                        const void* dgamma, const void* dbeta, const void* dy,
                                        void* dx, void* stream) {
  ChannelShape sh;
  const int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!x || !mu || !rsig || !gamma || !dgamma || !dbeta || !dy || !dx) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  if (dgamma == dbeta) {
    dbeta = static_cast<const char*>(dgamma) + dragon_hip::acc_bytes(dtype) * C;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_training_grad, sh, normalizer, x, mu, rsig,
                            gamma, dgamma, dbeta, dy, dx, s);
}

int dragon_hip_batch_norm_inference_grad(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                         const void* x, const void* mu, const void* rsig,
                                         const void* gamma, const void* dy, void* dgamma,
                                         void* dbeta, void* dx, void* scratch,
                                         size_t scratch_bytes, void* stream) {
  if (dgamma != nullptr) {
    const int st = dragon_hip_batch_norm_wgrad(dtype, N, C, S, layout, x, mu, rsig, dy, dgamma,
                                               dbeta, scratch, scratch_bytes, stream);
    if (st != DRAGON_HIP_OK) return st;
  }
  ChannelShape sh;
  const int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (N * S == 0) return DRAGON_HIP_OK;
  if (!rsig || !gamma || !dy || !dx) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_inference_grad, sh, rsig, gamma, dy, dx, s);
}

int dragon_hip_exchange_plan(int dtype, int64_t units, int64_t nseg, int64_t seglen, int tensors,
                             int* slices, int* slice_packets, int* packets_per_thread, int* grid) {
  if (!slices || !slice_packets || !packets_per_thread || !grid) return 0;
  if (tensors < 1 || tensors > 2 || units <= 0 || nseg <= 0 || seglen <= 0) return 0;
  if (!dragon_hip::fits_int32(units * nseg * seglen)) return 0;
  const dragon_hip::SliceUnits u{static_cast<uint32_t>(units), static_cast<uint32_t>(nseg),
                                 static_cast<uint32_t>(seglen), static_cast<uint32_t>(seglen),
                                 static_cast<uint32_t>(seglen)};
  switch (dtype) {
    case DRAGON_HIP_F16:
      return dragon_hip::exchange_plan_of<dragon_hip::f16_t>(u, tensors, slices, slice_packets,
                                                             packets_per_thread, grid);
    case DRAGON_HIP_BF16:
      return dragon_hip::exchange_plan_of<dragon_hip::bf16_t>(u, tensors, slices, slice_packets,
                                                              packets_per_thread, grid);
    case DRAGON_HIP_F32:
      return dragon_hip::exchange_plan_of<float>(u, tensors, slices, slice_packets,
                                                 packets_per_thread, grid);
    case DRAGON_HIP_F64:
      return dragon_hip::exchange_plan_of<double>(u, tensors, slices, slice_packets,
                                                  packets_per_thread, grid);
    default: return 0;
  }
}

int dragon_hip_batch_norm_training_backward(int dtype, int64_t N, int64_t C, int64_t S,
                                            float normalizer, int layout, const void* x,
                                            const void* mu, const void* rsig, const void* gamma,
                                            const void* dy, void* dgamma, void* dbeta, void* dx,
                                            void* scratch, size_t scratch_bytes, void* stream) {
  ChannelShape sh;
  int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (!dgamma || !dbeta) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  if (dgamma == dbeta) dbeta = static_cast<char*>(dgamma) + dragon_hip::acc_bytes(dtype) * C;
  if (N * S == 0) {
    return dragon_hip_batch_norm_wgrad(dtype, N, C, S, layout, x, mu, rsig, dy, dgamma, dbeta,
                                       scratch, scratch_bytes, stream);
  }
  if (!x || !mu || !rsig || !gamma || !dy || !dx) return DRAGON_HIP_EINVAL;
  if ((st = dragon_hip::check_scratch(sh, dtype, scratch, scratch_bytes)) != DRAGON_HIP_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_training_backward, sh, normalizer, x, mu, rsig,
                            gamma, dy, dgamma, dbeta, dx, scratch, s);
}

int dragon_hip_batch_norm_training_forward(int dtype, int64_t N, int64_t C, int64_t S, int layout,
                                           float momentum, float eps, const void* x,
                                           const void* gamma, const void* beta,
                                           void* running_mean, void* running_var, void* mu,
                                           void* rsig, void* params, void* y, void* scratch,
                                           size_t scratch_bytes, void* stream) {
  ChannelShape sh;
  int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (N * S == 0) return DRAGON_HIP_EINVAL;  // statistics of an empty batch are undefined
  if (!x || !gamma || !beta || !running_mean || !running_var || !mu || !rsig || !params || !y) {
    return DRAGON_HIP_EINVAL;
  }
  if ((st = dragon_hip::check_scratch(sh, dtype, scratch, scratch_bytes)) != DRAGON_HIP_OK) return st;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_training_forward, sh, momentum, eps, x, gamma,
                            beta, running_mean, running_var, mu, rsig, params, y, scratch, s);
}

int dragon_hip_batch_norm_training_forward_noalloc(int dtype, int64_t N, int64_t C, int64_t S,
                                                   int layout, float momentum, float eps,
                                                   const void* x, const void* gamma,
                                                   const void* beta, void* running_mean,
                                                   void* running_var, void* mu, void* rsig,
                                                   void* params, void* y, void* stream) {
  ChannelShape sh;
  const int st = dragon_hip::make_shape(N, C, S, layout, &sh);
  if (st != DRAGON_HIP_OK) return st;
  if (N * S == 0) return DRAGON_HIP_EINVAL;
  if (dtype < DRAGON_HIP_F16 || dtype > DRAGON_HIP_F64) return DRAGON_HIP_EDTYPE;
  if (dragon_hip::scratch_bytes_for(dtype, sh) > DRAGON_HIP_STATIC_SCRATCH_BYTES) {
    return DRAGON_HIP_ELIMIT;
  }
  void* ptr = nullptr;  // the static array's address on this device; never the array's name
  const int got = dragon_hip::static_scratch_on_current_device(&ptr);
  if (got != DRAGON_HIP_OK) return got;
  return dragon_hip_batch_norm_training_forward(dtype, N, C, S, layout, momentum, eps, x, gamma,
                                                beta, running_mean, running_var, mu, rsig, params,
                                                y, ptr, DRAGON_HIP_STATIC_SCRATCH_BYTES, stream);
}

} // extern "C"
