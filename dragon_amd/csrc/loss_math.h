// Pieces the loss kernels and the softmax kernels that fold the loss gather in
// share: SparseCrossEntropy's clamp and its notion of a valid class index
// (dragon/kernels/loss/cpu/cross_entropy_kernel.cc:25-57).
#pragma once

#include <cfloat>

#include "common.h"

namespace dragon_hip {

template <typename A>
__device__ __forceinline__ A neg_log_clamped(A p) {
  const A lo = static_cast<A>(FLT_MIN);
  return -acc_log(p > lo ? p : lo);
}

template <typename TargetT>
__device__ __forceinline__ bool target_valid(TargetT tgt, int64_t ignore_index, int64_t C) {
  const int64_t t = static_cast<int64_t>(tgt);
  return t != ignore_index && t >= 0 && t < C;
}

// Softmax along C of [N, C, S], S > 1, with the per-position loss and mask of
// SparseCrossEntropy written by the thread that holds the target class
// (softmax.hip). DRAGON_HIP_OK when launched, 1 when no column tile holds C rows.
template <typename T, typename TargetT>
int launch_softmax_cols_with_loss(int64_t N, int64_t S, int64_t C, int64_t ignore_index,
                                  const T* x, const TargetT* target, T* prob, T* loss, T* mask,
                                  hipStream_t stream);

} // namespace dragon_hip
