// The kernels:: and math:: function templates the operators call, declared
// with the reference's signatures (dragon/kernels/normalization/op_kernels.h:36-202,
// dragon/kernels/activation/op_kernels.h:211-247, dragon/kernels/math/op_kernels.h:106-115,
// dragon/utils/math/elementwise.h:48, dragon/utils/math/blas.h) and explicitly
// specialised for HIPContext in kernels_hip.cc, where each specialisation is a
// forward to the C-ABI entry point of the same name.
//
// Three additions have no counterpart among the reference's kernels:: functions:
// GroupNormForward, BatchNormTrainingForward and BatchNormTrainingBackward run
// a sequence an operator body issues (Moments, InvStd, ... ; WGrad,
// TrainingGrad) as one call, so that x (and dy) is read once where the device
// can keep the reduction unit on-die.
#pragma once

#include "core/common.h"
#include "core/context.h"

namespace dragon {

namespace math {

template <typename T, class Context>
void InvStd(const int N, const float eps, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void Axpby(const int N, const float alpha, const T* x, const float beta, T* y, Context* ctx);

template <typename T, class Context>
void Copy(const int N, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void Set(const int N, const T value, T* y, Context* ctx);

template <typename T, class Context>
void Square(const int N, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void Sub(const int N, const T* a, const T* b, T* y, Context* ctx);

// y = scale * sum(x) over `axes` (dragon/utils/math/reduce.h:50-58).
template <typename T, class Context>
void ReduceSum(const int num_dims, const int64_t* dims, const int num_axes, const int64_t* axes,
               const float scale, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void ReduceSumSqr(const int num_dims, const int64_t* dims, const int num_axes, const int64_t* axes,
                  const float scale, const T* x, T* y, Context* ctx);

} // namespace math

namespace kernels {

template <typename T, typename AccT, class Context>
void Moments(const int num_dims, const int64_t* dims, const int num_axes, const int64_t* axes,
             const T* x, AccT* mean, AccT* var, Context* ctx);

template <typename T, typename AccT, class Context>
void LayerNorm(const int N, const int C, const float epsilon, const T* x, const AccT* gamma,
               const AccT* beta, AccT* mu, AccT* rsig, T* y, Context* ctx);

template <typename T, typename AccT, class Context>
void GroupNorm(const int N, const int G, const int D, const int S, const string& data_format,
               const T* x, const AccT* mu, const AccT* rsig, const AccT* gamma, const AccT* beta,
               T* y, Context* ctx);

template <typename T, typename AccT, class Context>
void GroupNormGrad(const int N, const int G, const int D, const int S, const string& data_format,
                   const T* x, const AccT* mu, const AccT* rsig, const AccT* gamma, const T* dy,
                   AccT* ds, AccT* db, AccT* dgamma, AccT* dbeta, T* dx, Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNormExpectation(const int N, const int C, const int S, const float normalizer,
                          const string& data_format, const T* x, AccT* ex, AccT* ex2, Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNorm(const int N, const int C, const int S, const string& data_format, const T* x,
               const AccT* mu, const AccT* rsig, const AccT* gamma, const AccT* beta, AccT* scale,
               AccT* bias, T* y, Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNormWGrad(const int N, const int C, const int S, const string& data_format, const T* x,
                    const AccT* mu, const AccT* rsig, const T* dy, AccT* dgamma, AccT* dbeta,
                    Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNormTrainingGrad(const int N, const int C, const int S, const float normalizer,
                           const string& data_format, const T* x, const AccT* mu, const AccT* rsig,
                           const AccT* gamma, const AccT* dgamma, const AccT* dbeta, const T* dy,
                           T* dx, Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNormInferenceGrad(const int N, const int C, const int S, const string& data_format,
                            const T* x, const AccT* mu, const AccT* rsig, const AccT* gamma,
                            const T* dy, AccT* dgamma, AccT* dbeta, T* dx, Context* ctx);

template <typename T, class Context>
void Softmax(const int N, const int S, const int C, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void LogSoftmax(const int N, const int S, const int C, const T* x, T* y, Context* ctx);

template <typename T, class Context>
void SoftmaxGrad(const int N, const int S, const int C, const T* dy, const T* y, T* dx, Context* ctx);

template <typename T, class Context>
void LogSoftmaxGrad(const int N, const int S, const int C, const T* dy, const T* y, T* dx,
                    Context* ctx);

template <typename T, class Context>
void L1Norm(const int N, const int S, const int C, const float normalizer, const float epsilon,
            const T* x, T* y, Context* ctx);

template <typename T, class Context>
void L1NormGrad(const int N, const int S, const int C, const float normalizer, const float epsilon,
                const T* dy, const T* x, T* dx, Context* ctx);

template <typename T, class Context>
void L2Norm(const int N, const int S, const int C, const float normalizer, const float epsilon,
            const T* x, T* y, Context* ctx);

template <typename T, class Context>
void L2NormGrad(const int N, const int S, const int C, const float normalizer, const float epsilon,
                const T* dy, const T* x, T* dx, Context* ctx);

// Loss kernels (dragon/kernels/loss/op_kernels.h:25-32,51-69,95-113,179-189).
template <typename T, class Context>
void CrossEntropy(const int N, const T* input, const T* target, T* loss, Context* ctx);

template <typename InputT, typename TargetT, class Context>
void CrossEntropy(const int N, const int S, const int C, const int ignore_index,
                  const InputT* input, const TargetT* target, InputT* loss, InputT* mask,
                  Context* ctx);

template <typename InputT, typename TargetT, class Context>
void SoftmaxCrossEntropyGrad(const int N, const int S, const int C, const int ignore_index,
                             const InputT* input, const TargetT* target, InputT* dx, InputT* mask,
                             Context* ctx);

template <typename T, class Context>
void ReduceLoss(const int N, const int num_masks, const float normalizer, const T* x, const T* mask,
                T* y, Context* ctx);

template <typename T, class Context>
void ReduceLossGrad(const int N, const int num_masks, const float normalizer, const T* dl,
                    const T* mask, T* dx, Context* ctx);

template <typename T, class Context>
void BroadcastLossGrad(const int N, const int S, const int C, const T* dl, T* dx, Context* ctx);

// Fused operator bodies (see the header comment).
template <typename T, typename AccT, class Context>
void GroupNormForward(const int N, const int G, const int D, const int S, const string& data_format,
                      const float epsilon, const T* x, const AccT* gamma, const AccT* beta,
                      AccT* mu, AccT* rsig, T* y, Context* ctx);

// SoftmaxCrossEntropyLossOp / ...GradientOp bodies for class-index targets;
// reduction is "NONE", "SUM", "MEAN", "BATCH_MEAN" or "VALID".
template <typename InputT, typename TargetT, class Context>
void SoftmaxCrossEntropyLossForward(const int N, const int S, const int C, const int ignore_index,
                                    const string& reduction, const InputT* x, const TargetT* target,
                                    InputT* prob, InputT* loss, Context* ctx);

template <typename InputT, typename TargetT, class Context>
void SoftmaxCrossEntropyLossBackward(const int N, const int S, const int C, const int ignore_index,
                                     const string& reduction, const InputT* prob,
                                     const TargetT* target, const InputT* dl, InputT* dx,
                                     Context* ctx);

template <typename T, typename AccT, class Context>
void BatchNormTrainingForward(const int N, const int C, const int S, const string& data_format,
                              const float momentum, const float epsilon, const T* x,
                              const AccT* gamma, const AccT* beta, AccT* running_mean,
                              AccT* running_var, AccT* mu, AccT* rsig, AccT* params, T* y,
                              Context* ctx);

// BatchNormWGrad followed by BatchNormTrainingGrad (dgamma == dbeta means
// dbeta = dgamma + C, as for the two kernels).
template <typename T, typename AccT, class Context>
void BatchNormTrainingBackward(const int N, const int C, const int S, const float normalizer,
                               const string& data_format, const T* x, const AccT* mu,
                               const AccT* rsig, const AccT* gamma, const T* dy, AccT* dgamma,
                               AccT* dbeta, T* dx, Context* ctx);

} // namespace kernels

} // namespace dragon
