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
#include "reduce.h"
#include "row_tile.h"

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
  return static_cast<size_t>(sh.C) * split * 2 * acc_bytes;
}

// Runs the split reduction of accumulator F (one or two inputs) over every
// channel and hands the per-channel totals to epilogue E.
template <typename T, int kIn, typename F, typename E>
void reduce_channels(const ChannelShape& sh, const T* in0, const T* in1, F f, E e,
                     typename IO<T>::Acc* part, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const unsigned fin_grid = static_cast<unsigned>(ceil_div(sh.C, kReduceThreads));
  if (sh.nchw) {
    const SegmentedReduce s = channel_segments(sh);
    const dim3 grid(s.n_out * s.split);
    const bool vec_ok = aligned16(in0) && aligned16(in1) && sh.S % kVec == 0;
    if (vec_ok) {
      hipLaunchKernelGGL((reduce2_segments<T, kIn, kVec, F>), grid, dim3(kReduceThreads), 0, stream,
                         s, in0, in1, f, part);
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
    shift = IO<T>::load1(x + first_off);
  }
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
    const A shift = IO<T>::load1(x + c * chan_stride);
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
  const uint32_t total = sh.N * sh.C * sh.S;
  const bool vec_ok = aligned16(in0) && aligned16(in1) && aligned16(out) &&
      (sh.nchw ? sh.S % kVec == 0 : sh.C % kVec == 0);
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
// Training forward and backward read every tensor once. A channel is cut into
// K slices; a 256-thread workgroup keeps its slice in registers as raw packets
// (up to 16 per thread, 64 KB per slice), writes the slice's two partial sums
// into the channel's K pairs in HBM and waits until the channel's other K-1
// slices have done the same. Every workgroup of the channel then forms the
// same totals from the K pairs in a fixed order and normalises its slice out
// of registers.
//
// Work item w = c*K + k is taken by workgroup w % grid, and a workgroup walks
// its items in ascending order. All `grid` workgroups are resident at once
// (the grid is never larger than the occupancy query reports), so a workgroup
// that waits for the peers of its item waits for workgroups that are running:
// each of them holds a slice of the same channel or an item of an earlier
// channel, which by induction completes. The wait is bounded all the same (a
// thread that runs out of patience goes on with what it has read), so every
// wavefront reaches the end of the kernel whatever happens.
//
// A small kernel fills the pairs with the "unset" pattern before every launch.
constexpr int kCoopThreads = 256;

// A wait that gave up is reported through one word of pinned host memory that
// the kernels write and the host reads without synchronising: the outputs of
// that launch are invalid, and every later single-read launch is refused with
// DRAGON_HIP_ETIMEOUT until the word is cleared. Allocated on first use (once
// per process; before any stream capture, like the cached launch plans).
struct ExchangeState {
  uint32_t* host_word = nullptr;
  uint32_t* device_word = nullptr;
  uint32_t patience = 0;  // 0: the default
};
inline ExchangeState& exchange_state() {
  static ExchangeState st = [] {
    ExchangeState e;
    void* p = nullptr;
    if (hipHostMalloc(&p, sizeof(uint32_t), hipHostMallocMapped | hipHostMallocPortable) ==
        hipSuccess) {
      e.host_word = static_cast<uint32_t*>(p);
      *e.host_word = 0u;
      void* dp = nullptr;
      if (hipHostGetDevicePointer(&dp, p, 0) == hipSuccess) e.device_word = static_cast<uint32_t*>(dp);
    }
    (void)hipGetLastError();
    return e;
  }();
  return st;
}
constexpr uint32_t kCoopPatience = 1u << 20;  // polls of about 0.2 us each

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
inline uint32_t coop_grid(int r, int kIn) { return r * kIn > 16 ? kNumCUs * 3 : kNumCUs * 4; }

template <typename T>
CoopPlan plan_coop(const ChannelShape& sh, int kIn) {
  constexpr int kVec = IO<T>::kVec;
  CoopPlan p = {false, 0, 0, 0};
  if (!sh.nchw || sh.S % kVec != 0) return p;
  const uint32_t pps = sh.S / kVec;
  if (pps < 16) return p;  // runs shorter than 256 bytes: left to the split reduction
  const int64_t P = static_cast<int64_t>(sh.N) * pps;  // packets per channel
  const int rmax = coop_rmax(kIn);
  const int64_t grid = coop_grid(rmax, kIn);
  const int64_t kmin = ceil_div(P, static_cast<int64_t>(rmax) * kCoopThreads);
  if (kmin > 1024) return p;
  // Slices of at least four packets per thread, unless the channel is smaller.
  int64_t kmax = P / (4 * kCoopThreads);
  if (kmax < kmin) kmax = kmin;
  if (kmax > 1024) kmax = 1024;
  if (kmax > kmin + 64) kmax = kmin + 64;
  // The K whose C*K items fill whole rounds of the resident grid best.
  int64_t best = kmin;
  double best_util = 0;
  for (int64_t k = kmin; k <= kmax; ++k) {
    const int64_t items = static_cast<int64_t>(sh.C) * k;
    const double util = static_cast<double>(items) / (ceil_div(items, grid) * grid);
    if (util > best_util + 1e-9) best = k, best_util = util;
    if (util >= 0.96) break;
  }
  p.K = static_cast<uint32_t>(best);
  p.slice = static_cast<uint32_t>(ceil_div(P, best));
  p.r = static_cast<int>(ceil_div(p.slice, kCoopThreads));
  p.ok = true;
  return p;
}

template <typename T>
size_t coop_scratch_bytes(const ChannelShape& sh) {
  using A = typename IO<T>::Acc;
  size_t need = 0;
  for (int in = 1; in <= 2; ++in) {
    const CoopPlan p = plan_coop<T>(sh, in);
    if (!p.ok) continue;
    const size_t bytes = static_cast<size_t>(sh.C) * p.K * 2 * sizeof(A);
    if (bytes > need) need = bytes;
  }
  return need;
}

struct CoopShape {
  uint32_t C, S, K, slice;
  uint32_t pps;          // packets per segment (S / kVec)
  uint32_t P;            // packets per channel
  uint32_t seg_stride;   // elements between two samples of a channel (C * S)
  uint32_t step_seg, step_p;  // kCoopThreads packets further on = step_seg segments and step_p packets
  uint32_t items;        // C * K
  uint32_t patience;     // polls of a slot before a thread gives up
  uint32_t* timed_out;   // set to 1 by a thread that gave up (may be null)
};

template <typename T>
CoopShape make_coop_shape(const ChannelShape& sh, const CoopPlan& p) {
  constexpr int kVec = IO<T>::kVec;
  CoopShape d;
  d.C = sh.C, d.S = sh.S, d.K = p.K, d.slice = p.slice;
  d.pps = sh.S / kVec;
  d.P = sh.N * d.pps;
  d.seg_stride = sh.C * sh.S;
  d.step_seg = kCoopThreads / d.pps, d.step_p = kCoopThreads % d.pps;
  d.items = sh.C * p.K;
  const ExchangeState& ex = exchange_state();
  d.patience = ex.patience ? ex.patience : kCoopPatience;
  d.timed_out = ex.device_word;
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

// Bit pattern of a partial sum that has not been published yet (a NaN that no
// arithmetic here produces; the slots are filled with it before every launch).
template <typename A>
struct Unset;
template <>
struct Unset<float> {
  using Bits = uint32_t;
  static constexpr Bits kValue = 0xffffffffu;
};
template <>
struct Unset<double> {
  using Bits = unsigned long long;
  static constexpr Bits kValue = ~0ull;
};

template <typename Bits>
__global__ __launch_bounds__(256) void fill_words(Bits* p, uint32_t n, Bits value) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = value;
}

// Publishes this slice's pair, waits for the channel's K pairs and returns
// their sums (the same bits in every workgroup of the channel). The pairs are
// written and read with device-scope atomic accesses, which go past the
// per-XCD L2 caches without flushing or invalidating them; a slot is complete
// as soon as it no longer holds the unset pattern, so no counter or fence
// orders the exchange.
template <typename A>
__device__ __forceinline__ void coop_channel_totals(const CoopShape& d, uint32_t c, uint32_t w,
                                                    A& a, A& b, A* partial, A* lds_a, A* lds_b) {
  using Bits = typename Unset<A>::Bits;
  block_reduce_pair(a, b, lds_a);
  Bits* slots = reinterpret_cast<Bits*>(partial);
  if (threadIdx.x == 0) {
    __hip_atomic_store(slots + 2 * static_cast<size_t>(w), __builtin_bit_cast(Bits, a),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(slots + 2 * static_cast<size_t>(w) + 1, __builtin_bit_cast(Bits, b),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  A ta = A(0), tb = A(0);
  const Bits* pairs = slots + 2 * static_cast<size_t>(c) * d.K;
  for (uint32_t q = threadIdx.x; q < d.K; q += kCoopThreads) {
    Bits ua, ub;
    uint32_t patience = d.patience;
    for (;;) {
      ua = __hip_atomic_load(pairs + 2 * q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ub = __hip_atomic_load(pairs + 2 * q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (ua != Unset<A>::kValue && ub != Unset<A>::kValue) break;
      if (--patience == 0) {
        if (d.timed_out) {
          __hip_atomic_store(d.timed_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        break;
      }
      __builtin_amdgcn_s_sleep(8);
    }
    ta += __builtin_bit_cast(A, ua);
    tb += __builtin_bit_cast(A, ub);
  }
  block_reduce_pair(ta, tb, lds_b);
  a = ta, b = tb;
}

// The two passes of an item over its slice, written once for the forward
// (Op = CoopForward) and the backward (Op = CoopBackward). Op provides
//   kIn                          tensors held (x; x and dy)
//   begin(c, base, in0)          per-item setup
//   add(x, dy, a, b)             one element's terms of the two sums
//   finish(c, leader, a, b)      coefficients from the channel totals; the
//                                item's first slice also writes the [C] outputs
//   map(x, dy)                   one output element
template <typename T>
struct CoopForward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
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
    shift = IO<T>::load1(x + base);  // one sample of the channel
  }
  __device__ __forceinline__ void add(A x, A, A& a, A& b) const {
    const A t = x - shift;
    a += t;
    b += t * t;
  }
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
  __device__ __forceinline__ A map(A x, A) const { return x * sc + bi; }
};

template <typename T>
struct CoopBackward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 2;
  A normalizer;
  const A* mu;
  const A* rsig;
  const A* gamma;
  A* dgamma;
  A* dbeta;
  A m, r, gr, ca, cb;
  __device__ __forceinline__ void begin(uint32_t c, uint32_t, const T*) { m = mu[c], r = rsig[c]; }
  __device__ __forceinline__ void add(A x, A dy, A& a, A& b) const {
    a += dy * (x - m);
    b += dy;
  }
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
  __device__ __forceinline__ A map(A x, A dy) const { return gr * dy + (ca * (x - m) + cb); }
};

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
    base = c * d.S;
  }
  __device__ __forceinline__ bool has(int i) const { return i * kCoopThreads + threadIdx.x < len; }
};

template <typename T, int kR, int kIn>
__device__ __forceinline__ void coop_load(const CoopShape& d, uint32_t w, const T* in0, const T* in1,
                                          CoopSlice<T, kR, kIn>& s) {
  constexpr int kVec = IO<T>::kVec;
  const CoopItem it(d, w);
  CoopCursor cur(d, it.j0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    const uint32_t off = it.has(i) ? cur.template offset<kVec>(d, it.base) : it.base;
    s.p0[i] = load_packet(in0 + off);
    if constexpr (kIn == 2) s.p1[i] = load_packet(in1 + off);
    cur.advance(d);
  }
}

// `next` is the item this workgroup takes after w (>= d.items: none): its
// packets are requested one by one into the registers the second pass has just
// written out, so they travel while the rest of this item is stored.
template <typename T, int kR, typename Op>
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
  A a = A(0), b = A(0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    if (it.has(i)) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
#pragma unroll
      for (int e = 0; e < kVec; ++e) op.add(xv[e], Op::kIn == 2 ? dv[e] : A(0), a, b);
    }
  }
  coop_channel_totals(d, it.c, w, a, b, partial, lds_a, lds_b);
  op.finish(it.c, it.k == 0 && threadIdx.x == 0, a, b);
  // convert the packets again instead of keeping every converted element
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    asm volatile("" : "+v"(s.p0[i]));
    if constexpr (Op::kIn == 2) asm volatile("" : "+v"(s.p1[i]));
  }
  const bool more = next < d.items;  // uniform over the workgroup
  const CoopItem nit(d, more ? next : w);
  CoopCursor cur(d, it.j0), ncur(d, nit.j0);
#pragma unroll
  for (int i = 0; i < kR; ++i) {
    if (it.has(i)) {
      A xv[kVec], dv[kVec];
      IO<T>::unpack(s.p0[i], xv);
      if constexpr (Op::kIn == 2) IO<T>::unpack(s.p1[i], dv);
#pragma unroll
      for (int e = 0; e < kVec; ++e) xv[e] = op.map(xv[e], Op::kIn == 2 ? dv[e] : A(0));
      store_packet(out + cur.template offset<kVec>(d, it.base), IO<T>::pack(xv));
    }
    cur.advance(d);
    if (more) {
      const uint32_t off = nit.has(i) ? ncur.template offset<kVec>(d, nit.base) : nit.base;
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
template <typename T, int kR, typename Op>
__global__ __launch_bounds__(kCoopThreads, kR * Op::kIn > 16 ? 3 : 4) void channel_slices(
    const CoopShape d, const T* __restrict__ in0, const T* __restrict__ in1, T* __restrict__ out,
    const Op op, typename IO<T>::Acc* __restrict__ partial) {
  using A = typename IO<T>::Acc;
  __shared__ A lds_a[2 * kReduceWaves];
  __shared__ A lds_b[2 * kReduceWaves];
  CoopSlice<T, kR, Op::kIn> s;
  if (blockIdx.x < d.items) coop_load<T, kR, Op::kIn>(d, blockIdx.x, in0, in1, s);
  for (uint32_t w = blockIdx.x; w < d.items; w += gridDim.x) {
    coop_process<T, kR, Op>(d, w, w + gridDim.x, in0, in1, out, op, s, partial, lds_a, lds_b);
  }
}

template <typename A>
inline void fill_unset(A* pairs, const CoopShape& d, hipStream_t stream) {
  using Bits = typename Unset<A>::Bits;
  const uint32_t n = d.items * 2;
  hipLaunchKernelGGL((fill_words<Bits>), dim3(static_cast<unsigned>(ceil_div(n, 256))), dim3(256), 0,
                     stream, reinterpret_cast<Bits*>(pairs), n, Unset<A>::kValue);
}

// DRAGON_HIP_OK when the single-read kernel was launched, kNotApplicable when
// the shape or alignment leaves the call to the split path, or an error.
constexpr int kNotApplicable = 1;
template <typename T, typename Op>
int try_channel_slices(const ChannelShape& sh, const Op& op, const T* in0, const T* in1, T* out,
                       typename IO<T>::Acc* scratch, hipStream_t stream) {
  const CoopPlan p = plan_coop<T>(sh, Op::kIn);
  if (!p.ok || !aligned16(in0) || !aligned16(in1) || !aligned16(out)) return kNotApplicable;
  const ExchangeState& ex = exchange_state();
  if (ex.host_word && *static_cast<volatile uint32_t*>(ex.host_word) != 0u) {
    return DRAGON_HIP_ETIMEOUT;
  }
  const CoopShape d = make_coop_shape<T>(sh, p);
  fill_unset(scratch, d, stream);
#define LAUNCH(R)                                                                              \
  {                                                                                            \
    auto kernel = channel_slices<T, R, Op>;                                                    \
    const unsigned resident = resident_grid(kernel, kCoopThreads, 0);                          \
    const unsigned want = coop_grid(coop_rmax(Op::kIn), Op::kIn);                              \
    const unsigned cap = resident < want ? resident : want;                                    \
    hipLaunchKernelGGL(kernel, dim3(d.items < cap ? d.items : cap), dim3(kCoopThreads), 0,     \
                       stream, d, in0, in1, out, op, scratch);                                 \
  }
  constexpr int kIn = Op::kIn;
  if (p.r * kIn <= 4) LAUNCH(4 / kIn)
  else if (p.r * kIn <= 8) LAUNCH(8 / kIn)
  else if (p.r * kIn <= 16) LAUNCH(16 / kIn)
  else LAUNCH(24 / kIn)
#undef LAUNCH
  return status_of_launch();
}

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
  const int st = try_channel_slices<T>(sh, op, xp, xp, static_cast<T*>(y), static_cast<A*>(scratch),
                                       stream);
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
  int st = try_channel_slices<T>(sh, op, static_cast<const T*>(x), static_cast<const T*>(dy),
                                 static_cast<T*>(dx), static_cast<A*>(scratch), stream);
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
  const size_t coop = coop_scratch_bytes<T>(sh);
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

int dragon_hip_exchange_timed_out(void) {
  const dragon_hip::ExchangeState& ex = dragon_hip::exchange_state();
  return ex.host_word && *static_cast<volatile uint32_t*>(ex.host_word) != 0u ? 1 : 0;
}

void dragon_hip_exchange_reset(unsigned patience) {
  dragon_hip::ExchangeState& ex = dragon_hip::exchange_state();
  if (ex.host_word) *static_cast<volatile uint32_t*>(ex.host_word) = 0u;
  ex.patience = patience;
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

} // extern "C"
