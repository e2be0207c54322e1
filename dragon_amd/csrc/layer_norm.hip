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
#include "row_tile.h"

namespace dragon_hip {
namespace {

template <typename T, int kTPR, int kVPT>
__global__ __launch_bounds__(row_threads(kTPR)) void layer_norm_rows(
    const int64_t N, const int C, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using Tile = RowTile<T, kTPR, kVPT>;
  using A = typename Tile::A;
  constexpr int kVec = Tile::kVec;
  __shared__ A slots[2][Tile::kSlots];
  const int npackets = C / kVec;
  const A inv_c = A(1) / A(C);
  const int lane = Tile::lane();

  for (int64_t row = static_cast<int64_t>(blockIdx.x) * Tile::kRowsPerBlock + Tile::sub_row();
       row < N; row += static_cast<int64_t>(gridDim.x) * Tile::kRowsPerBlock) {
    Tile t;
    t.load(x + row * C, npackets, A(0));

    A s = A(0);
#pragma unroll
    for (int i = 0; i < kVPT; ++i)
#pragma unroll
      for (int e = 0; e < kVec; ++e) s += t.v[i][e];
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
    if (lane == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }

#pragma unroll
    for (int i = 0; i < kVPT; ++i) {
      if (Tile::active(i, npackets)) {
        const int col = (i * kTPR + lane) * kVec;
        A g[kVec], b[kVec];
        load_params<kVec>(gamma + col, g);
        load_params<kVec>(beta + col, b);
#pragma unroll
        for (int e = 0; e < kVec; ++e) t.v[i][e] = (t.v[i][e] - mean) * rs * g[e] + b[e];
      }
    }
    t.store(y + row * C, npackets);
    if (kTPR != kWaveSize) __syncthreads();  // slots are reused by the next row
  }
}

// Any width, any alignment: one 256-thread workgroup per row, three strided
// passes over the row with element-wise accesses (the second and third hit L2).
template <typename T>
__global__ __launch_bounds__(256) void layer_norm_rows_looped(
    const int64_t N, const int64_t C, const typename IO<T>::Acc eps, const T* __restrict__ x,
    const typename IO<T>::Acc* __restrict__ gamma, const typename IO<T>::Acc* __restrict__ beta,
    typename IO<T>::Acc* __restrict__ mu, typename IO<T>::Acc* __restrict__ rsig,
    T* __restrict__ y) {
  using A = typename IO<T>::Acc;
  __shared__ A slots[2][4];
  const A inv_c = A(1) / A(C);
  for (int64_t row = blockIdx.x; row < N; row += gridDim.x) {
    const T* xr = x + row * C;
    T* yr = y + row * C;
    A s = A(0);
    for (int64_t j = threadIdx.x; j < C; j += 256) s += IO<T>::load1(xr + j);
    const A mean = block_allreduce<4>(s, SumOp(), slots[0]) * inv_c;
    A q = A(0);
    for (int64_t j = threadIdx.x; j < C; j += 256) {
      const A d = IO<T>::load1(xr + j) - mean;
      q += d * d;
    }
    const A var = block_allreduce<4>(q, SumOp(), slots[1]) * inv_c;
    const A rs = acc_rsqrt_exact(var + eps);
    if (threadIdx.x == 0) {
      mu[row] = mean;
      rsig[row] = rs;
    }
    for (int64_t j = threadIdx.x; j < C; j += 256) {
      IO<T>::store1(yr + j, (IO<T>::load1(xr + j) - mean) * rs * gamma[j] + beta[j]);
    }
    __syncthreads();
  }
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
  RowConfig cfg;
  const bool packets_ok = C % kVec == 0 && aligned16(x) && aligned16(y) && aligned16(gamma) &&
      aligned16(beta) && pick_row_config(C / kVec, &cfg);
  if (packets_ok) {
#define LAUNCH(TPR, VPT)                                                                   \
  {                                                                                        \
    using Tile = RowTile<T, TPR, VPT>;                                                     \
    hipLaunchKernelGGL((layer_norm_rows<T, TPR, VPT>), dim3(row_grid(N, Tile::kRowsPerBlock)), \
                       dim3(Tile::kThreads), 0, stream, N, static_cast<int>(C), A(eps), xp, gp, \
                       bp, mp, rp, yp);                                                    \
  }
    DRAGON_HIP_ROW_SWITCH(cfg, LAUNCH);
#undef LAUNCH
  } else {
    hipLaunchKernelGGL((layer_norm_rows_looped<T>), dim3(row_grid(N, 1)), dim3(256), 0, stream, N,
                       C, A(eps), xp, gp, bp, mp, rp, yp);
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
