// LayerNorm forward for gfx950.
//
// Replaces kernels::LayerNorm<T, AccT, Context>
// (dragon/kernels/normalization/op_kernels.h:191-202; CPU loop
// dragon/kernels/normalization/cpu/layer_norm_kernel.cc:10-39): per row,
//   mu = mean(x), rsig = 1/sqrt(var_biased(x) + eps),
//   y  = (x - mu) * rsig * gamma + beta.
//
// HBM traffic per row: C elements in, C elements out, plus mu/rsig. The row is
// held in registers between the statistics and the normalisation, so x is read
// once. Variance is the centred sum sum((x-mu)^2)/C computed from the
// register copy: same quantity as the reference's E[x^2]-E[x]^2 without its
// cancellation.
#include "row_loop.h"
#include "row_tile.h"
#include "short_rows.h"

namespace dragon_hip {
namespace {

// A wavefront that holds a whole row in one or two packets per lane takes two
// neighbouring rows at a time: their dependent cross-lane reduction steps
// interleave, and one fetch of gamma and beta serves both.
template <typename T, int kTPR, int kVPT, bool kRagged>
__global__ __launch_bounds__(row_threads(kTPR)) void layer_norm_rows(
    const int64_t N, const int C, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT, row_threads(kTPR), kRagged>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  constexpr int kR = wave_rows_at_a_time<kTPR, kVPT>();
  constexpr int kRowsPerStep = Tile::kRowsPerBlock * kR;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = Tile::extent_of(C);
  const A inv_c = A(1) / A(C);
  const int lane = Tile::lane();

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kRowsPerStep + Tile::sub_row() * kR;
       row < N; row += static_cast<int64_t>(gridDim.x) * kRowsPerStep) {
    Tile t[kR];
    bool on[kR];  // uniform over the row's threads
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      on[r] = row + r < N;
      t[r].load(x + (on[r] ? row + r : row) * C, npackets, A(0));
    }

    A mean[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      mean[r] = A(0);
#pragma unroll
      for (int i = 0; i < kVPT; ++i)
#pragma unroll
        for (int e = 0; e < kVec; ++e) mean[r] += t[r].v[i][e];
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) mean[r] = Tile::reduce(mean[r], SumOp(), slots[0]) * inv_c;

    A rs[kR];
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      rs[r] = A(0);
#pragma unroll
      for (int i = 0; i < kVPT; ++i) {
        if (Tile::active(i, npackets)) {
#pragma unroll
          for (int e = 0; e < kVec; ++e) {
            const A d = t[r].v[i][e] - mean[r];
            if (Tile::elem_active(i, e, npackets)) rs[r] += d * d;
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < kR; ++r) {
      const A var = Tile::reduce(rs[r], SumOp(), slots[1]) * inv_c;
      rs[r] = acc_rsqrt_exact(var + eps);
      if (lane == 0 && on[r]) {
        mu[row + r] = mean[r];
        rsig[row + r] = rs[r];
      }
    }

#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        const int col = (i * kTPR + lane) * kVec;
        A g[kVec], b[kVec];
        if constexpr (kRagged) {
          load_params_ragged<kVec>(gamma + col, C - col, g);
          load_params_ragged<kVec>(beta + col, C - col, b);
        } else {
          load_params<kVec>(gamma + col, g);
          load_params<kVec>(beta + col, b);
        }
#pragma unroll
        for (int r = 0; r < kR; ++r)
#pragma unroll
          for (int e = 0; e < kVec; ++e)
            t[r].v[i][e] = (t[r].v[i][e] - mean[r]) * rs[r] * g[e] + b[e];
      }
    }
#pragma unroll
    for (int r = 0; r < kR; ++r)
      if (on[r]) t[r].store(y + (row + r) * C, npackets);
    if (kTPR != kWaveSize) __syncthreads();  // slots are reused by the next row
  }
}

// Rows spanning several wavefronts: gamma and beta no longer fit the 32 KB L1
// next to the streamed rows, and re-reading them from L2 for every row would
// move more bytes than the row itself (fp32 parameters against 16-bit data).
// A persistent workgroup stages both in LDS once and then walks its rows.
// A workgroup of kThreads threads holds kThreads / kTPR rows at a time; the
// 1024-thread workgroups, of which a compute unit holds two at most, also
// request their next rows' packets before they reduce the current ones.
template <typename T, int kTPR, int kVPT, int kThreads = kTPR>
__global__ __launch_bounds__(kThreads) void layer_norm_wide_rows(
    const int64_t N, const int C, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT, kThreads>;
  using Raw = RawRowTile<T, kTPR, kVPT, kThreads>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  constexpr int kGroups = Tile::kRowsPerBlock;
  constexpr int kPerPacket = 16 / sizeof(A);  // parameters per 16-byte LDS word
  constexpr bool kPrefetch = kThreads == 1024;
  extern __shared__ u32x4 staged[];  // gamma[C] then beta[C]
  __shared__ A slots[2][Tile::kSlots];
  A* lds_gamma = reinterpret_cast<A*>(staged);
  A* lds_beta = lds_gamma + C;
  const int npackets = C / kVec;
  // Rows of 8-element packets against 4-float LDS words: the first halves of
  // all packets, then the second halves, so that the lanes of a wavefront read
  // adjacent 16-byte words (eight consecutive floats per lane put lanes l and
  // l + 8 on the same banks: a two-way conflict on every access).
  constexpr bool kSplit = kVec == 2 * kPerPacket;
  for (int i = threadIdx.x; i < C / kPerPacket; i += kThreads) {
    const int at = kSplit ? (i & 1) * npackets + (i >> 1) : i;
    staged[at] = load_packet_keep(gamma + i * kPerPacket);
    staged[C / kPerPacket + at] = load_packet_keep(beta + i * kPerPacket);
  }
  __syncthreads();
  // the kVec parameters of packet `packet` of the row
  auto params_of = [&](const A* lds, const int packet, A(&v)[kVec]) {
    if constexpr (kSplit) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(lds + packet * 4);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(lds + (npackets + packet) * 4);
      v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
      v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    } else {
      load_params<kVec>(lds + packet * kVec, v);
    }
  };

  const A inv_c = A(1) / A(C);
  const int lane = Tile::lane();
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kGroups;
  int64_t row = static_cast<int64_t>(blockIdx.x) * kGroups + Tile::sub_row();
  Raw cur;
  if (kPrefetch) cur.load(x + (row < N ? row : 0) * C, npackets, row < N);
  // Uniform trip count over the workgroup: the row reductions hold barriers.
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kGroups; base < N; base += stride) {
    const bool valid = row < N;
    Raw nxt;
    if (kPrefetch) {
      const bool more = row + stride < N;
      nxt.load(x + (more ? row + stride : 0) * C, npackets, more);
    } else {
      cur.load(x + (valid ? row : 0) * C, npackets, valid);
    }
    Tile t;
    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      cur.unpack(i, t.v[i]);
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += t.v[i][e];
    }
    const A mean = Tile::reduce(s, SumOp(), slots[0]) * inv_c;
    A q = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
          const A d = t.v[i][e] - mean;
          q += d * d;
        }
      }
    }
    const A var = Tile::reduce(q, SumOp(), slots[1]) * inv_c;
    const A rs = acc_rsqrt_exact(var + eps);
    if (lane == 0 && valid) {
      mu[row] = mean;
      rsig[row] = rs;
    }
#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        A g[kVec], b[kVec];
        params_of(lds_gamma, i * kTPR + lane, g);
        params_of(lds_beta, i * kTPR + lane, b);
#pragma unroll
        for (int e = 0; e < kVec; ++e) t.v[i][e] = (t.v[i][e] - mean) * rs * g[e] + b[e];
      }
    }
    if (kPrefetch) {
      nxt.wait_ready();
      cur = nxt;
    }
    if (valid) t.store(y + row * C, npackets);
    row += stride;
  }
}

// Rows too long for the register tiles: two passes per row. Pass one
// accumulates sums shifted by the row's first element (mean = s + sum(x-s)/C,
// var = sum((x-s)^2)/C - (sum(x-s)/C)^2: no cancellation against a large mean),
// pass two normalises; gamma and beta are read element-wise (any alignment).
template <typename T>
__global__ __launch_bounds__(kLoopThreads) void layer_norm_rows_looped(
    const int64_t N, const int64_t C, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using A = typename IO<T>::Acc;
  using Loop = RowLoop<T>;
  constexpr int kVec = Loop::kVec;
  __shared__ A slots[2][kLoopWaves];
  const A inv_c = A(1) / A(C);
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const T* xr = x + row * C;
    T* yr = y + row * C;
    const A shift = load_shift(xr);
    A s = A(0), q = A(0);
    Loop::visit(xr, C, shift, [&](int64_t, const A(&v)[kVec], int) {
#pragma unroll
      for (int e = 0; e < kVec; ++e) {
        const A d = v[e] - shift;  // padding holds `shift`: adds nothing
        s += d;
        q += d * d;
      }
    });
    s = block_allreduce<kLoopWaves>(s, SumOp(), slots[0]);
    q = block_allreduce<kLoopWaves>(q, SumOp(), slots[1]);
    const A dm = s * inv_c;
    const A mean = shift + dm;
    const A rs = acc_rsqrt_exact((q * inv_c - dm * dm) + eps);
    if (threadIdx.x == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    Loop::visit(xr, C, A(0), [&](int64_t col, const A(&v)[kVec], int n) {
      A o[kVec], g[kVec], b[kVec];
      load_params_ragged<kVec>(gamma + col, n, g);
      load_params_ragged<kVec>(beta + col, n, b);
#pragma unroll
      for (int e = 0; e < kVec; ++e) o[e] = (v[e] - mean) * rs * g[e] + b[e];
      Loop::store(yr, col, o, n);
    });
    __syncthreads();  // slots are reused by the next row
  }
}

// Short rows (per-head normalisations, odd widths): a policy of the LDS-staged
// kernel (short_rows.h). Mean, then the centred sum of squares, over the kL
// lanes of a row; gamma / beta of a thread's elements live in registers.
template <typename T, int kE>
struct LayerNormShortForward {
  using A = typename IO<T>::Acc;
  static constexpr int kIn = 1;
  static constexpr size_t kEndBytes = 0;
  static constexpr int kSideWords = 0;
  A inv_c, eps;
  const A* gamma;
  const A* beta;
  A* mu;
  A* rsig;
  A g[kE], b[kE];
  bool packed = false;  // lane l owns elements l * kE + j instead of l + j * kL
  __device__ __forceinline__ void set_packed(bool on) { packed = on; }
  // Measured on MI355X: the packed order gains 6-9% on 16-bit rows of up to 64
  // elements and loses 3-15% on longer or fp32 rows, where the parameters held
  // per lane leave the registers no room for both orders.
  template <int kL>
  static constexpr bool packed_ok() { return sizeof(T) == 2 && kL <= 8; }
  __device__ __forceinline__ A fill0() const { return A(0); }
  __device__ __forceinline__ A fill1() const { return A(0); }
  template <int kL>
  __device__ __forceinline__ void begin(int l, int C) {
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const int e = packed ? l * kE + j : l + j * kL;
      g[j] = e < C ? gamma[e] : A(0);
      b[j] = e < C ? beta[e] : A(0);
    }
  }
  template <int kL>
  __device__ __forceinline__ void row(int64_t r, const A*, int l, int C, A (&v)[kE], const A (&)[kE]) const {
    A s = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) s += v[j];  // lanes past the row hold 0
    const A mean = group_allreduce<kL>(s, SumOp()) * inv_c;
    A q = A(0);
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      const A d = v[j] - mean;
      q += l + j * kL < C ? d * d : A(0);
    }
    const A rs = acc_rsqrt_exact(group_allreduce<kL>(q, SumOp()) * inv_c + eps);
    if (l == 0) {
      mu[r] = mean;
      rsig[r] = rs;
    }
#pragma unroll
    for (int j = 0; j < kE; ++j) v[j] = (v[j] - mean) * rs * g[j] + b[j];
  }
  template <int kL>
  __device__ __forceinline__ void end(A*, int) const {}
};

// Rows of up to 512 bytes, and rows of up to 1024 elements that are not whole
// aligned packets, take the staged kernel (as for softmax).
inline bool layer_norm_short_rows(int64_t C, size_t elem_bytes, const void* x, const void* y) {
  if (C > 1024 || !congruent16(x, y)) return false;
  const size_t row_bytes = static_cast<size_t>(C) * elem_bytes;
  return row_bytes <= 512 || row_bytes % 16 != 0 || !aligned16(x);
}

template <typename T>
int launch_layer_norm(int64_t N, int64_t C, float eps, const void* x, const void* gamma,
                      const void* beta, void* mu, void* rsig, void* y, hipStream_t stream) {
  using A = typename IO<T>::Acc;
  constexpr int kVec = IO<T>::kVec;
  const T* xp = static_cast<const T*>(x);
  T* yp = static_cast<T*>(y);
  const A* gp = static_cast<const A*>(gamma);
  const A* bp = static_cast<const A*>(beta);
  A* mp = static_cast<A*>(mu);
  A* rp = static_cast<A*>(rsig);
  ShortPlan sp;
  if (layer_norm_short_rows(C, sizeof(T), x, y) && plan_short_rows(C, sizeof(T), 4, aligned16(x), &sp)) {
    const size_t lds = static_cast<size_t>(sp.stage_packets) * 16;
    DRAGON_HIP_SHORT_LAUNCH(T, LayerNormShortForward, sp, lds, short_grid(N, sp.rows_per_chunk),
                            stream, N, static_cast<int>(C), xp, xp, yp, A(1) / A(C), A(eps), gp, bp,
                            mp, rp, {}, {});
    return status_of_launch();
  }
  RowConfig cfg;
  // Eight 16-bit packets per thread of a 1024-thread tile (64 fp32 values and
  // as many parameters) do not fit the 128 registers of such a workgroup:
  // those rows take the looped kernel.
  const bool fits = pick_row_config(ceil_div(C, kVec), 8, &cfg) &&
      !(sizeof(T) == 2 && cfg.tpr == 1024 && cfg.vpt == 8);
  const bool packets_ok = fits && C % kVec == 0 && aligned16(x) && aligned16(y) &&
      aligned16(gamma) && aligned16(beta);
  const size_t staged_bytes = 2 * static_cast<size_t>(C) * sizeof(A);
  if (packets_ok && cfg.tpr > kWaveSize && staged_bytes <= kMaxStagedParamBytes) {
    // 256-thread tiles need several workgroups per compute unit to hide HBM
    // latency; when the staged parameters leave room for fewer than four, use
    // the 1024-thread tile (which prefetches instead).
    // the same with 16-bit rows of up to 1024 packets: four rows at a time on
    // 256 threads each, so that a 1024-thread workgroup is not mostly idle
    bool four_rows = false;
    if (cfg.tpr == 256 && staged_bytes * 4 > kMaxStagedParamBytes) {
      const int64_t need = ceil_div(C / kVec, 1024);
      four_rows = sizeof(T) == 2 && need == 1;
      cfg.tpr = 1024;
      cfg.vpt = need <= 2 ? 2 : (need <= 4 ? 4 : 8);
    }
#define LAUNCH_T(TPR, VPT, THREADS)                                                          \
  {                                                                                          \
    note_flavour("layer_norm_wide_rows<" #TPR "," #VPT "," #THREADS ">");                    \
    auto kernel = layer_norm_wide_rows<T, TPR, VPT, THREADS>;                                \
    const int64_t groups = ceil_div(N, static_cast<int64_t>(THREADS / TPR));                 \
    const unsigned resident = resident_grid(kernel, THREADS, staged_bytes);                  \
    const unsigned grid =                                                                    \
        groups < static_cast<int64_t>(resident) ? static_cast<unsigned>(groups) : resident;  \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(THREADS), staged_bytes, stream, N,           \
                       static_cast<int>(C), A(eps), xp, gp, bp, mp, rp, yp);                 \
  }
#define LAUNCH(TPR, VPT) LAUNCH_T(TPR, VPT, TPR)
    if (four_rows) LAUNCH_T(256, 4, 1024)
    else if (cfg.tpr == 256 && cfg.vpt == 2) LAUNCH(256, 2)
    else if (cfg.tpr == 256 && cfg.vpt == 4) LAUNCH(256, 4)
    else if (cfg.tpr == 256 && cfg.vpt == 8) LAUNCH(256, 8)
    else if (cfg.tpr == 1024 && cfg.vpt == 2) LAUNCH(1024, 2)
    else if (cfg.tpr == 1024 && cfg.vpt == 4) LAUNCH(1024, 4)
    else LAUNCH(1024, 8)
#undef LAUNCH
#undef LAUNCH_T
  } else if (packets_ok) {
#define LAUNCH(TPR, VPT)                                                                   \
  {                                                                                        \
    using Tile = RowTile<T, TPR, VPT>;                                                     \
    hipLaunchKernelGGL((layer_norm_rows<T, TPR, VPT, false>),                              \
                       dim3(row_grid(N, Tile::kRowsPerBlock * wave_rows_at_a_time<TPR, VPT>())), \
                       dim3(Tile::kThreads), 0, stream,                                    \
                       N, static_cast<int>(C), A(eps), xp, gp, bp, mp, rp, yp);            \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  } else if (fits) {
    // any width, any alignment: ragged tiles, parameters read element-wise
#define LAUNCH(TPR, VPT)                                                                   \
  {                                                                                        \
    using Tile = RowTile<T, TPR, VPT>;                                                     \
    hipLaunchKernelGGL((layer_norm_rows<T, TPR, VPT, true>),                               \
                       dim3(row_grid(N, Tile::kRowsPerBlock * wave_rows_at_a_time<TPR, VPT>())), \
                       dim3(Tile::kThreads), 0, stream,                                    \
                       N, static_cast<int>(C), A(eps), xp, gp, bp, mp, rp, yp);            \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  } else {
    hipLaunchKernelGGL((layer_norm_rows_looped<T>), dim3(loop_grid(N)), dim3(kLoopThreads), 0,
                       stream, N, C, A(eps), xp, gp, bp, mp, rp, yp);
  }
  return status_of_launch();
}

} // namespace
} // namespace dragon_hip

extern "C" int dragon_hip_layer_norm(int dtype, int64_t N, int64_t C, float eps, const void* x,
                                     const void* gamma, const void* beta, void* mu, void* rsig,
                                     void* y, void* stream) {
  if (N < 0 || C <= 0) return DRAGON_HIP_EINVAL;
  if (N == 0) return DRAGON_HIP_OK;
  if (!x || !gamma || !beta || !mu || !rsig || !y) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::launch_layer_norm, N, C, eps, x, gamma, beta, mu,
                            rsig, y, s);
}
