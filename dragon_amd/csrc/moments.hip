// kernels::Moments (mean and biased variance) and math::ReduceSum /
// ReduceSumSqr / ReduceL1 over arbitrary axes for gfx950.
//
// Replaces kernels::Moments<T, AccT, Context>
// (dragon/kernels/math/op_kernels.h:106-115; CPU
// dragon/kernels/math/cpu/moments_kernel.cc:10-189 with the axis utilities of
// dragon/utils/math/reduce.h:96-198) and math::ReduceSum / ReduceSumSqr /
// ReduceL1 (dragon/utils/math/reduce.h:50-80; CPU
// dragon/utils/math/cpu/reduce.cc:10-236). As there, size-1 axes are dropped and
// adjacent axes of the same kind are merged first; the collapsed pattern picks
// the kernel:
//   [K,R] [R] [R,K,R] [K,R,K,R]   segmented split reduction (contiguous runs)
//   [R,K]                         column split reduction
//   anything else                 one workgroup per output, strided gather
// (K = kept extent, R = reduced extent).
//
// Variance uses sums shifted by one sample of the reduction set,
//   mean = s + sum(x-s)/n,  var = sum((x-s)^2)/n - (sum(x-s)/n)^2,
// which equals the reference's E[x^2]-E[x]^2 in exact arithmetic and keeps
// Welford-class accuracy in fp32 when |mean| >> stddev, while partial sums
// still combine by plain addition.
#include <algorithm>
#include <string>
#include <vector>

#include "reduce.h"
#include "short_rows.h"

namespace dragon_hip {
namespace {

// What is accumulated and what is written is a policy, so that Moments and
// the plain sums (math::ReduceSum / ReduceSumSqr / ReduceL1,
// dragon/utils/math/reduce.h:50-80) share the planner and the kernels.
//   kShift            subtract the first element of the reduction set first
//   term(d, a, b)     fold one (shifted) element into the pair of sums
//   Out / finish      outputs and the per-output epilogue
template <typename T>
struct MomentsPolicy {
  using A = typename IO<T>::Acc;
  static constexpr bool kShift = true;
  struct Out {
    A* mean;
    A* var;
  };
  static __device__ __forceinline__ void term(A d, A& a, A& b) {
    a += d;
    b += d * d;
  }
  static __device__ __forceinline__ void finish(const Out& out, uint32_t o, A shift, A a, A b,
                                                A inv_n) {
    const A m = a * inv_n;
    out.mean[o] = shift + m;
    out.var[o] = b * inv_n - m * m;
  }
};

enum SumKind { kSumPlain = 0, kSumSqr = 1, kSumAbs = 2 };

// y[o] = scale * sum f(x) with f = identity, square or absolute value; the sum
// is kept in the accumulator type and rounded to T once.
template <typename T, int kKind>
struct SumPolicy {
  using A = typename IO<T>::Acc;
  static constexpr bool kShift = false;
  struct Out {
    T* y;
    A scale;
  };
  static __device__ __forceinline__ void term(A d, A& a, A&) {
    a += kKind == kSumPlain ? d : (kKind == kSumSqr ? d * d : (d < A(0) ? -d : d));
  }
  static __device__ __forceinline__ void finish(const Out& out, uint32_t o, A, A a, A, A) {
    IO<T>::store1(out.y + o, a * out.scale);
  }
};

template <typename T, typename P>
struct ReduceAccum {
  using A = typename IO<T>::Acc;
  const T* x;
  A shift;
  __device__ __forceinline__ void begin(uint32_t, uint32_t first_off) {
    shift = P::kShift ? load_shift(x + first_off) : A(0);
  }
  template <int V>
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, uint32_t, const A (&x0)[V],
                                      const A (&)[V], A& a, A& b) const {
#pragma unroll
    for (int e = 0; e < V; ++e) P::term(P::kShift ? x0[e] - shift : x0[e], a, b);
  }
  __device__ __forceinline__ void add(uint32_t, uint32_t, uint32_t, A x0, A, A& a, A& b) const {
    P::term(P::kShift ? x0 - shift : x0, a, b);
  }
};

template <typename T, typename P>
struct ReduceSegEpilogue {
  using A = typename IO<T>::Acc;
  const T* x;
  SegmentedReduce d;
  A inv_n;
  typename P::Out out;
  __device__ __forceinline__ void operator()(uint32_t o, A a, A b) const {
    const uint32_t o1 = o / d.outer2;
    const uint32_t o2 = o - o1 * d.outer2;
    const A shift = P::kShift ? load_shift(x + o1 * d.stride1 + o2 * d.stride2) : A(0);
    P::finish(out, o, shift, a, b, inv_n);
  }
};

template <typename T, typename P>
struct ReduceColEpilogue {
  using A = typename IO<T>::Acc;
  const T* x;
  A inv_n;
  typename P::Out out;
  __device__ __forceinline__ void operator()(uint32_t c, A a, A b) const {
    const A shift = P::kShift ? load_shift(x + c) : A(0);
    P::finish(out, c, shift, a, b, inv_n);
  }
};

constexpr int kMaxDims = 8;
struct GatherDims {
  int n_keep, n_red;
  uint32_t keep_dim[kMaxDims], keep_stride[kMaxDims];
  uint32_t red_dim[kMaxDims], red_stride[kMaxDims];
  uint32_t n_out, n_red_elems;
};

// One workgroup per output; the reduced index is unravelled over the reduced
// extents (last fastest, the order the reference walks them in).
template <typename T, typename P>
__global__ __launch_bounds__(kReduceThreads) void reduce_gather(
    const GatherDims g, const T* __restrict__ x, const typename P::Out out) {
  using A = typename IO<T>::Acc;
  __shared__ A lds[2 * kReduceWaves];
  for (uint32_t o = blockIdx.x; o < g.n_out; o += gridDim.x) {
    uint32_t base = 0, r = o;
    for (int d = g.n_keep - 1; d >= 0; --d) {
      base += (r % g.keep_dim[d]) * g.keep_stride[d];
      r /= g.keep_dim[d];
    }
    const A shift = P::kShift ? load_shift(x + base) : A(0);
    A a = A(0), b = A(0);
    for (uint32_t j = threadIdx.x; j < g.n_red_elems; j += kReduceThreads) {
      uint32_t off = base, q = j;
      for (int d = g.n_red - 1; d >= 0; --d) {
        off += (q % g.red_dim[d]) * g.red_stride[d];
        q /= g.red_dim[d];
      }
      P::term(IO<T>::load1(x + off) - shift, a, b);
    }
    block_reduce_pair(a, b, lds);
    if (threadIdx.x == 0) P::finish(out, o, shift, a, b, A(1) / A(g.n_red_elems));
    __syncthreads();
  }
}

// Rows of up to 1024 contiguous elements (a trailing axis of a few or a few
// hundred elements, millions of outputs): a policy of the LDS-staged short-row
// kernel (short_rows.h), several rows per wavefront, the epilogue applied by
// the row's first lane. A workgroup per output would need more workgroups
// than a launch can hold.
template <typename T, int kE, typename P>
struct ReduceRowOp {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  static constexpr bool kReadOnly = true;
  typename P::Out out;
  A inv_n;
  // sums only: any element order (element 0 stays v[0] of lane 0 in both)
  __device__ __forceinline__ void set_packed(bool) {}
  template <int kL>
  static constexpr bool packed_ok() { return true; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int, int) {}
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A*, int l, int width, A (&v)[kE],
                                      const A (&)[kE]) const {
    // the row's first element, which lane 0 holds as v[0]
    const A shift = P::kShift ? finite_or_zero(__shfl(v[0], (threadIdx.x & (kWaveSize - 1)) / kL * kL, kWaveSize)) : A(0);
    A a = A(0), b = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      if (l + j * kL < width) P::term(v[j] - shift, a, b);
    }
    a = group_allreduce<kL>(a, SumOp());
    b = group_allreduce<kL>(b, SumOp());
    if (l == 0) P::finish(out, static_cast<uint32_t>(r), shift, a, b, inv_n);
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};
template <typename P>
struct ReduceRowsOf {
  template <typename T, int kE>
  using Op = ReduceRowOp<T, kE, P>;
};

// One reduced axis between kept ones ([N, C, S] over C): a thread per output
// walks its C elements S apart; adjacent threads read adjacent addresses.
template <typename T, typename P>
__global__ __launch_bounds__(kReduceThreads) void reduce_strided_columns(
    const uint32_t N, const uint32_t C, const uint32_t S, const T* __restrict__ x,
    const typename P::Out out) {
  using A = typename IO<T>::Acc;
  const uint32_t total = N * S;
  for (uint32_t o = blockIdx.x * kReduceThreads + threadIdx.x; o < total;
       o += gridDim.x * kReduceThreads) {
    const uint32_t n = o / S;
    const T* col = x + static_cast<size_t>(n) * C * S + (o - n * S);
    const A shift = P::kShift ? load_shift(col) : A(0);
    A a = A(0), b = A(0);
#pragma unroll 8
    for (uint32_t k = 0; k < C; ++k) P::term(IO<T>::load1(col + static_cast<size_t>(k) * S) - shift, a, b);
    P::finish(out, o, shift, a, b, A(1) / A(C));
  }
}

// Rows of a few thousand contiguous elements, thousands of them: one wavefront
// per row (four rows per workgroup), no LDS and no second stage. A row is read
// as the aligned 16-byte packets that cover it, whatever its width and address;
// of its first and last packet only the row's own elements are folded in.
template <typename T, typename P>
__global__ __launch_bounds__(kReduceThreads) void reduce_wave_rows(
    const uint32_t rows, const uint32_t len, const T* __restrict__ x, const typename P::Out out,
    const typename IO<T>::Acc inv_n) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const uint32_t wave = threadIdx.x / kWaveSize;
  const int n = static_cast<int>(len);
  for (uint32_t row = blockIdx.x * kReduceWaves + wave; row < rows; row += gridDim.x * kReduceWaves) {
    const T* r = x + static_cast<size_t>(row) * len;
    const A shift = P::kShift ? load_shift(r) : A(0);
    const int lead = static_cast<int>((reinterpret_cast<uintptr_t>(r) & 15u) / sizeof(T));
    const int packets = (lead + n + kVec - 1) / kVec;
    A a = A(0), b = A(0);
#pragma unroll 4
    for (int p = lane; p < packets; p += kWaveSize) {
      const int pe = p * kVec - lead;  // the packet's first element, in the row
      A v[kVec];
      load_unpack_keep<T>(r + pe, v);
      if (pe >= 0 && pe + kVec <= n) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) P::term(P::kShift ? v[e] - shift : v[e], a, b);
      } else {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          if (pe + e >= 0 && pe + e < n) P::term(P::kShift ? v[e] - shift : v[e], a, b);
        }
      }
    }
    a = wave_allreduce(a, SumOp());
    b = wave_allreduce(b, SumOp());
    if (lane == 0) P::finish(out, row, shift, a, b, inv_n);
  }
}

enum PlanKind { kPlanSegments, kPlanColumns, kPlanGather, kPlanShortRows, kPlanStrided, kPlanWaveRows };
struct MomentsPlan {
  PlanKind kind;
  SegmentedReduce seg;
  ColumnReduce col;
  GatherDims gather;
  int64_t n_out, n_red;
  size_t scratch_bytes;
};

// Restates what CollapseReduceAxes does to the shape (drop extents of one,
// merge neighbours of the same kind) and classifies the result.
int make_plan(int dtype, int num_dims, const int64_t* dims, int num_axes, const int64_t* axes,
              MomentsPlan* plan) {
  if (num_dims < 0 || num_axes < 0 || (num_dims > 0 && !dims) || (num_axes > 0 && !axes)) {
    return DRAGON_HIP_EINVAL;
  }
  std::vector<char> is_red(num_dims, 0);
  for (int i = 0; i < num_axes; ++i) {
    if (axes[i] < 0 || axes[i] >= num_dims) return DRAGON_HIP_EINVAL;
    is_red[axes[i]] = 1;
  }
  std::vector<int64_t> ext;
  std::vector<char> red;
  int64_t total = 1;
  for (int i = 0; i < num_dims; ++i) {
    if (dims[i] < 0) return DRAGON_HIP_EINVAL;
    total *= dims[i];
    if (dims[i] == 1) continue;
    if (!ext.empty() && red.back() == is_red[i]) {
      ext.back() *= dims[i];
    } else {
      ext.push_back(dims[i]);
      red.push_back(is_red[i]);
    }
  }
  if (!fits_int32(total)) return DRAGON_HIP_EINVAL;
  const size_t acc_bytes = dtype == DRAGON_HIP_F64 ? 8 : 4;
  std::vector<int64_t> stride(ext.size(), 1);
  for (int i = static_cast<int>(ext.size()) - 2; i >= 0; --i) stride[i] = stride[i + 1] * ext[i + 1];
  plan->n_out = plan->n_red = 1;
  for (size_t i = 0; i < ext.size(); ++i) (red[i] ? plan->n_red : plan->n_out) *= ext[i];
  plan->scratch_bytes = 0;
  std::string pat;
  for (char r : red) pat.push_back(r ? 'R' : 'K');
  SegmentedReduce& s = plan->seg;
  s = SegmentedReduce{static_cast<uint32_t>(plan->n_out), 1, 0, 0, 1, 0, 0, 1};
  auto u32 = [](int64_t v) { return static_cast<uint32_t>(v); };
  if (pat == "KR" && plan->n_red <= 1024 && plan->n_out >= 4096) {
    plan->kind = kPlanShortRows;
  } else if (pat == "KRK" && plan->n_out >= 16384) {
    // enough outputs to fill the device with a thread each
    plan->kind = kPlanStrided;
    s.nseg = u32(ext[0]), s.seglen = u32(ext[1]), s.seg_stride = u32(ext[2]);  // N, C, S
  } else if (pat == "KR" && plan->n_out >= 2048 && dtype != DRAGON_HIP_F64 &&
             plan->n_red * (dtype == DRAGON_HIP_F32 ? 4 : 2) <= 20 * 1024) {
    // Rows of up to 20 KB, 2048 of them or more: a wavefront each. Measured against
    // a workgroup per row: fp32 [65536,1025] 49 us against 83, [16384,4097] 46
    // against 53, [8192,8192] 51 against 47 (left to the workgroups); bf16
    // [32768,2048] 27 against 37, [8192,8192] 26 against 28; with 2048 rows of
    // 128 KB the wavefronts are too few (78 us against 50).
    plan->kind = kPlanWaveRows;
  } else if (pat == "R" || pat == "KR") {
    plan->kind = kPlanSegments;
    s.stride1 = u32(plan->n_red), s.seglen = u32(plan->n_red);
  } else if (pat == "RKR") {
    plan->kind = kPlanSegments;
    s.outer2 = u32(ext[1]), s.stride2 = u32(ext[2]);
    s.nseg = u32(ext[0]), s.seg_stride = u32(stride[0]), s.seglen = u32(ext[2]);
  } else if (pat == "KRKR") {
    plan->kind = kPlanSegments;
    s.outer2 = u32(ext[2]), s.stride1 = u32(stride[0]), s.stride2 = u32(ext[3]);
    s.nseg = u32(ext[1]), s.seg_stride = u32(stride[1]), s.seglen = u32(ext[3]);
  } else if (pat == "RK") {
    plan->kind = kPlanColumns;
    plan->col = ColumnReduce{u32(ext[0]), u32(ext[1]), 1};
    plan->col.split = column_split_bound(ext[0], ext[1]);  // upper bound: sizes the scratch
    plan->scratch_bytes = static_cast<size_t>(plan->col.split) * ext[1] * 2 * acc_bytes;
  } else {
    if (ext.size() > kMaxDims) return DRAGON_HIP_EINVAL;
    plan->kind = kPlanGather;
    GatherDims& g = plan->gather;
    g.n_keep = g.n_red = 0;
    for (size_t i = 0; i < ext.size(); ++i) {
      if (red[i]) {
        g.red_dim[g.n_red] = u32(ext[i]), g.red_stride[g.n_red++] = u32(stride[i]);
      } else {
        g.keep_dim[g.n_keep] = u32(ext[i]), g.keep_stride[g.n_keep++] = u32(stride[i]);
      }
    }
    g.n_out = u32(plan->n_out), g.n_red_elems = u32(plan->n_red);
  }
  if (plan->kind == kPlanSegments) {
    s.split = pick_split(plan->n_out, plan->n_red);
    plan->scratch_bytes = static_cast<size_t>(plan->n_out) * s.split * 2 * acc_bytes;
  }
  return DRAGON_HIP_OK;
}

template <typename T, typename P>
int launch_reduce(const MomentsPlan& plan, const void* x, const typename P::Out& out, void* scratch,
                  hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* xp = static_cast<const T*>(x);
  A* part = static_cast<A*>(scratch);
  const A inv_n = A(1) / A(plan.n_red);
  const unsigned fin_grid = static_cast<unsigned>(ceil_div(plan.n_out, kReduceThreads));
  using Accum = ReduceAccum<T, P>;
  if (plan.kind == kPlanShortRows) {
    ShortPlan sp;
    if (!plan_short_rows(plan.n_red, sizeof(T), 4, aligned16(x), &sp)) return DRAGON_HIP_EINVAL;
    using Holder = ReduceRowsOf<P>;
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16;
    T* none = nullptr;
    DRAGON_HIP_SHORT_LAUNCH(T, typename Holder::template Op, sp, lds,
                            short_grid(plan.n_out, sp.rows_per_chunk), stream, plan.n_out,
                            static_cast<int>(plan.n_red), xp, xp, none, out, inv_n);
  } else if (plan.kind == kPlanWaveRows) {
    if (sizeof(T) > 4) return DRAGON_HIP_EINVAL;  // the planner keeps fp64 on the segment kernels
    const int64_t want = ceil_div(plan.n_out, kReduceWaves);
    const int64_t cap = static_cast<int64_t>(num_cus()) * 32;
    hipLaunchKernelGGL((reduce_wave_rows<T, P>), dim3(static_cast<unsigned>(want < cap ? want : cap)),
                       dim3(kReduceThreads), 0, stream, static_cast<uint32_t>(plan.n_out),
                       static_cast<uint32_t>(plan.n_red), xp, out, inv_n);
  } else if (plan.kind == kPlanStrided) {
    const SegmentedReduce& s = plan.seg;
    const unsigned grid = static_cast<unsigned>(
        std::min<int64_t>(ceil_div(plan.n_out, kReduceThreads), static_cast<int64_t>(num_cus()) * 32));
    hipLaunchKernelGGL((reduce_strided_columns<T, P>), dim3(grid), dim3(kReduceThreads), 0, stream,
                       s.nseg, s.seglen, s.seg_stride, xp, out);
  } else if (plan.kind == kPlanSegments) {
    const SegmentedReduce& s = plan.seg;
    const bool vec_ok = aligned16(x) && s.seglen % kVec == 0 && s.stride1 % kVec == 0 &&
        s.stride2 % kVec == 0 && s.seg_stride % kVec == 0;
    Accum f{xp, A(0)};
    const dim3 grid(s.n_out * s.split);
    if (vec_ok) {
      hipLaunchKernelGGL((reduce2_segments<T, 1, kVec, Accum>), grid, dim3(kReduceThreads), 0,
                         stream, s, xp, xp, f, part);
    } else if (s.seglen >= 4 * kVec && sizeof(T) <= 4) {
      // segments that are not whole aligned packets, through the packets that cover them
      hipLaunchKernelGGL((reduce2_segments_windows<T, 1, Accum>), grid, dim3(kReduceThreads), 0,
                         stream, s, xp, xp, f, part);
    } else {
      hipLaunchKernelGGL((reduce2_segments<T, 1, 1, Accum>), grid, dim3(kReduceThreads), 0, stream,
                         s, xp, xp, f, part);
    }
    ReduceSegEpilogue<T, P> e{xp, s, inv_n, out};
    hipLaunchKernelGGL((reduce2_finalize<A, ReduceSegEpilogue<T, P>>), dim3(fin_grid),
                       dim3(kReduceThreads), 0, stream, s.n_out, s.split, true, part, e);
  } else if (plan.kind == kPlanColumns) {
    const ColumnReduce& c = plan.col;
    Accum f{xp, A(0)};
    const uint32_t split = launch_reduce2_columns<T, 1, Accum>(c.rows, c.cols, xp, xp, f, part,
                                                               stream);
    ReduceColEpilogue<T, P> e{xp, inv_n, out};
    launch_reduce2_finalize<A, ReduceColEpilogue<T, P>>(c.cols, split, false, part, e, stream);
  } else {
    const unsigned grid = static_cast<unsigned>(plan.n_out < 65536 ? plan.n_out : 65536);
    hipLaunchKernelGGL((reduce_gather<T, P>), dim3(grid), dim3(kReduceThreads), 0, stream,
                       plan.gather, xp, out);
  }
  return status_of_launch();
}

template <typename T>
int launch_moments(const MomentsPlan& plan, const void* x, void* mean, void* var, void* scratch,
                   hipStream_t stream) {
  using A = typename IO<T>::Acc;
  using P = MomentsPolicy<T>;
  return launch_reduce<T, P>(plan, x, typename P::Out{static_cast<A*>(mean), static_cast<A*>(var)},
                             scratch, stream);
}

template <typename T>
int launch_sum(int kind, const MomentsPlan& plan, float scale, const void* x, void* y,
               void* scratch, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  T* yp = static_cast<T*>(y);
  const A sc = static_cast<A>(scale);
  switch (kind) {
    case kSumPlain: {
      using P = SumPolicy<T, kSumPlain>;
      return launch_reduce<T, P>(plan, x, typename P::Out{yp, sc}, scratch, stream);
    }
    case kSumSqr: {
      using P = SumPolicy<T, kSumSqr>;
      return launch_reduce<T, P>(plan, x, typename P::Out{yp, sc}, scratch, stream);
    }
    default: {
      using P = SumPolicy<T, kSumAbs>;
      return launch_reduce<T, P>(plan, x, typename P::Out{yp, sc}, scratch, stream);
    }
  }
}

// Shared body of the three sum entry points. A reduction over no element (an
// extent of zero among the reduced axes) writes zeros, the reducer's identity.
int reduce_sum_entry(int kind, int dtype, int num_dims, const int64_t* dims, int num_axes,
                     const int64_t* axes, float scale, const void* x, void* y, void* scratch,
                     size_t scratch_bytes, void* stream) {
  MomentsPlan plan;
  const int st = make_plan(dtype, num_dims, dims, num_axes, axes, &plan);
  if (st != DRAGON_HIP_OK) return st;
  if (plan.n_out == 0) return DRAGON_HIP_OK;
  if (!y) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (plan.n_red == 0) return dragon_hip_set(dtype, plan.n_out, 0.f, y, stream);
  if (!x) return DRAGON_HIP_EINVAL;
  if (plan.scratch_bytes > 0 && (!scratch || scratch_bytes < plan.scratch_bytes)) {
    return DRAGON_HIP_ESCRATCH;
  }
  DRAGON_HIP_DISPATCH_DTYPE(dtype, launch_sum, kind, plan, scale, x, y, scratch, s);
}

} // namespace
} // namespace dragon_hip

extern "C" {

size_t dragon_hip_moments_scratch_bytes(int dtype, int num_dims, const int64_t* dims,
                                        int num_axes, const int64_t* axes) {
  dragon_hip::MomentsPlan plan;
  if (dragon_hip::make_plan(dtype, num_dims, dims, num_axes, axes, &plan) != DRAGON_HIP_OK) return 0;
  return plan.scratch_bytes;
}

int dragon_hip_moments(int dtype, int num_dims, const int64_t* dims, int num_axes,
                       const int64_t* axes, const void* x, void* mean, void* var, void* scratch,
                       size_t scratch_bytes, void* stream) {
  dragon_hip::MomentsPlan plan;
  const int st = dragon_hip::make_plan(dtype, num_dims, dims, num_axes, axes, &plan);
  if (st != DRAGON_HIP_OK) return st;
  if (plan.n_out * plan.n_red == 0) return DRAGON_HIP_OK;
  if (!x || !mean || !var) return DRAGON_HIP_EINVAL;
  if (plan.scratch_bytes > 0 && (!scratch || scratch_bytes < plan.scratch_bytes)) {
    return DRAGON_HIP_ESCRATCH;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_moments, plan, x, mean, var, scratch, s);
}

size_t dragon_hip_reduce_scratch_bytes(int dtype, int num_dims, const int64_t* dims, int num_axes,
                                       const int64_t* axes) {
  return dragon_hip_moments_scratch_bytes(dtype, num_dims, dims, num_axes, axes);
}

int dragon_hip_reduce_sum(int dtype, int num_dims, const int64_t* dims, int num_axes,
                          const int64_t* axes, float scale, const void* x, void* y, void* scratch,
                          size_t scratch_bytes, void* stream) {
  return dragon_hip::reduce_sum_entry(dragon_hip::kSumPlain, dtype, num_dims, dims, num_axes, axes,
                                      scale, x, y, scratch, scratch_bytes, stream);
}

int dragon_hip_reduce_sum_sqr(int dtype, int num_dims, const int64_t* dims, int num_axes,
                              const int64_t* axes, float scale, const void* x, void* y,
                              void* scratch, size_t scratch_bytes, void* stream) {
  return dragon_hip::reduce_sum_entry(dragon_hip::kSumSqr, dtype, num_dims, dims, num_axes, axes,
                                      scale, x, y, scratch, scratch_bytes, stream);
}

int dragon_hip_reduce_l1(int dtype, int num_dims, const int64_t* dims, int num_axes,
                         const int64_t* axes, float scale, const void* x, void* y, void* scratch,
                         size_t scratch_bytes, void* stream) {
  return dragon_hip::reduce_sum_entry(dragon_hip::kSumAbs, dtype, num_dims, dims, num_axes, axes,
                                      scale, x, y, scratch, scratch_bytes, stream);
}

} // extern "C"
