// kernels::X<T, AccT, HIPContext> and math::X<T, HIPContext>: one-line forwards
// to the C ABI (include/dragon_hip.h). Scratch for split reductions comes from
// the context's scratch workspace under its own buffer name, so it never
// clobbers the "BufferShared" tensor an operator may be holding
// (GroupNormGradientOp keeps ds/db there, group_norm_op.cc:64-65).
#include "kernels/op_kernels.h"

#include "core/workspace.h"
#include "dragon_hip.h"

namespace dragon {

namespace {

template <typename T>
constexpr int Tag() {
  return static_cast<int>(TypeOf<T>::value);
}

int LayoutTag(const string& data_format) {
  if (data_format == "NCHW") return DRAGON_HIP_NCHW;
  if (data_format == "NHWC") return DRAGON_HIP_NHWC;
  LOG(FATAL) << "Unknown DataFormat: " << data_format;
  return -1;
}

void* Scratch(HIPContext* ctx, size_t bytes) {
  if (bytes == 0) return nullptr;
  return ctx->workspace()->template data<uint8_t, HIPContext>(bytes, "BufferKernel", ctx);
}

} // namespace

namespace math {

#define DEFINE_MATH_FUNCS(T)                                                                     \
  template <>                                                                                    \
  void InvStd<T, HIPContext>(const int N, const float eps, const T* x, T* y, HIPContext* ctx) {  \
    HIP_CHECK(dragon_hip_inv_std(Tag<T>(), N, eps, x, y, ctx->hip_stream()));                    \
  }                                                                                              \
  template <>                                                                                    \
  void Axpby<T, HIPContext>(const int N, const float alpha, const T* x, const float beta, T* y,  \
                            HIPContext* ctx) {                                                   \
    HIP_CHECK(dragon_hip_axpby(Tag<T>(), N, alpha, x, beta, y, ctx->hip_stream()));              \
  }                                                                                              \
  template <>                                                                                    \
  void Copy<T, HIPContext>(const int N, const T* x, T* y, HIPContext* ctx) {                     \
    HIP_CHECK(dragon_hip_copy(Tag<T>(), N, x, y, ctx->hip_stream()));                            \
  }                                                                                              \
  template <>                                                                                    \
  void Square<T, HIPContext>(const int N, const T* x, T* y, HIPContext* ctx) {                   \
    HIP_CHECK(dragon_hip_square(Tag<T>(), N, x, y, ctx->hip_stream()));                          \
  }                                                                                              \
  template <>                                                                                    \
  void Sub<T, HIPContext>(const int N, const T* a, const T* b, T* y, HIPContext* ctx) {          \
    HIP_CHECK(dragon_hip_sub(Tag<T>(), N, a, b, y, ctx->hip_stream()));                          \
  }

DEFINE_MATH_FUNCS(float16);
DEFINE_MATH_FUNCS(bfloat16);
DEFINE_MATH_FUNCS(float);
DEFINE_MATH_FUNCS(double);
#undef DEFINE_MATH_FUNCS

template <>
void Set<float, HIPContext>(const int N, const float value, float* y, HIPContext* ctx) {
  HIP_CHECK(dragon_hip_set(Tag<float>(), N, value, y, ctx->hip_stream()));
}
template <>
void Set<double, HIPContext>(const int N, const double value, double* y, HIPContext* ctx) {
  HIP_CHECK(dragon_hip_set(Tag<double>(), N, static_cast<float>(value), y, ctx->hip_stream()));
}

} // namespace math

namespace kernels {

#define DEFINE_KERNEL_LAUNCHERS(T, AccT)                                                          \
  template <>                                                                                     \
  void Moments<T, AccT, HIPContext>(const int num_dims, const int64_t* dims, const int num_axes,  \
                                    const int64_t* axes, const T* x, AccT* mean, AccT* var,       \
                                    HIPContext* ctx) {                                            \
    const size_t bytes = dragon_hip_moments_scratch_bytes(Tag<T>(), num_dims, dims, num_axes, axes); \
    HIP_CHECK(dragon_hip_moments(Tag<T>(), num_dims, dims, num_axes, axes, x, mean, var,          \
                                 Scratch(ctx, bytes), bytes, ctx->hip_stream()));                 \
  }                                                                                               \
  template <>                                                                                     \
  void LayerNorm<T, AccT, HIPContext>(const int N, const int C, const float epsilon, const T* x,  \
                                      const AccT* gamma, const AccT* beta, AccT* mu, AccT* rsig,  \
                                      T* y, HIPContext* ctx) {                                    \
    HIP_CHECK(dragon_hip_layer_norm(Tag<T>(), N, C, epsilon, x, gamma, beta, mu, rsig, y,         \
                                    ctx->hip_stream()));                                          \
  }                                                                                               \
  template <>                                                                                     \
  void GroupNorm<T, AccT, HIPContext>(const int N, const int G, const int D, const int S,         \
                                      const string& data_format, const T* x, const AccT* mu,      \
                                      const AccT* rsig, const AccT* gamma, const AccT* beta, T* y, \
                                      HIPContext* ctx) {                                          \
    HIP_CHECK(dragon_hip_group_norm(Tag<T>(), N, G, D, S, LayoutTag(data_format), x, mu, rsig,    \
                                    gamma, beta, y, ctx->hip_stream()));                          \
  }                                                                                               \
  template <>                                                                                     \
  void GroupNormGrad<T, AccT, HIPContext>(                                                        \
      const int N, const int G, const int D, const int S, const string& data_format, const T* x,  \
      const AccT* mu, const AccT* rsig, const AccT* gamma, const T* dy, AccT* ds, AccT* db,       \
      AccT* dgamma, AccT* dbeta, T* dx, HIPContext* ctx) {                                        \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_group_norm_grad_scratch_bytes(Tag<T>(), N, G, D, S, layout);  \
    HIP_CHECK(dragon_hip_group_norm_grad(Tag<T>(), N, G, D, S, layout, x, mu, rsig, gamma, dy, ds, \
                                         db, dgamma, dbeta, dx, Scratch(ctx, bytes), bytes,       \
                                         ctx->hip_stream()));                                     \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormExpectation<T, AccT, HIPContext>(                                                 \
      const int N, const int C, const int S, const float normalizer, const string& data_format,   \
      const T* x, AccT* ex, AccT* ex2, HIPContext* ctx) {                                         \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_batch_norm_reduce_scratch_bytes(Tag<T>(), N, C, S, layout);   \
    HIP_CHECK(dragon_hip_batch_norm_expectation(Tag<T>(), N, C, S, normalizer, layout, x, ex, ex2, \
                                                Scratch(ctx, bytes), bytes, ctx->hip_stream()));  \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNorm<T, AccT, HIPContext>(const int N, const int C, const int S,                      \
                                      const string& data_format, const T* x, const AccT* mu,      \
                                      const AccT* rsig, const AccT* gamma, const AccT* beta,      \
                                      AccT* scale, AccT* bias, T* y, HIPContext* ctx) {           \
    HIP_CHECK(dragon_hip_batch_norm(Tag<T>(), N, C, S, LayoutTag(data_format), x, mu, rsig, gamma, \
                                    beta, scale, bias, y, ctx->hip_stream()));                    \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormWGrad<T, AccT, HIPContext>(const int N, const int C, const int S,                 \
                                           const string& data_format, const T* x, const AccT* mu, \
                                           const AccT* rsig, const T* dy, AccT* dgamma,           \
                                           AccT* dbeta, HIPContext* ctx) {                        \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_batch_norm_reduce_scratch_bytes(Tag<T>(), N, C, S, layout);   \
    HIP_CHECK(dragon_hip_batch_norm_wgrad(Tag<T>(), N, C, S, layout, x, mu, rsig, dy, dgamma,     \
                                          dbeta, Scratch(ctx, bytes), bytes, ctx->hip_stream())); \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormTrainingGrad<T, AccT, HIPContext>(                                                \
      const int N, const int C, const int S, const float normalizer, const string& data_format,   \
      const T* x, const AccT* mu, const AccT* rsig, const AccT* gamma, const AccT* dgamma,        \
      const AccT* dbeta, const T* dy, T* dx, HIPContext* ctx) {                                   \
    HIP_CHECK(dragon_hip_batch_norm_training_grad(Tag<T>(), N, C, S, normalizer,                  \
                                                  LayoutTag(data_format), x, mu, rsig, gamma,     \
                                                  dgamma, dbeta, dy, dx, ctx->hip_stream()));     \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormInferenceGrad<T, AccT, HIPContext>(                                               \
      const int N, const int C, const int S, const string& data_format, const T* x,               \
      const AccT* mu, const AccT* rsig, const AccT* gamma, const T* dy, AccT* dgamma,             \
      AccT* dbeta, T* dx, HIPContext* ctx) {                                                      \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_batch_norm_reduce_scratch_bytes(Tag<T>(), N, C, S, layout);   \
    HIP_CHECK(dragon_hip_batch_norm_inference_grad(Tag<T>(), N, C, S, layout, x, mu, rsig, gamma, \
                                                   dy, dgamma, dbeta, dx, Scratch(ctx, bytes),    \
                                                   bytes, ctx->hip_stream()));                    \
  }                                                                                               \
  template <>                                                                                     \
  void GroupNormForward<T, AccT, HIPContext>(                                                     \
      const int N, const int G, const int D, const int S, const string& data_format,              \
      const float epsilon, const T* x, const AccT* gamma, const AccT* beta, AccT* mu, AccT* rsig, \
      T* y, HIPContext* ctx) {                                                                    \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_group_norm_forward_scratch_bytes(Tag<T>(), N, G, D, S, layout); \
    HIP_CHECK(dragon_hip_group_norm_forward(Tag<T>(), N, G, D, S, layout, epsilon, x, gamma, beta, \
                                            mu, rsig, y, Scratch(ctx, bytes), bytes,              \
                                            ctx->hip_stream()));                                  \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormTrainingForward<T, AccT, HIPContext>(                                             \
      const int N, const int C, const int S, const string& data_format, const float momentum,     \
      const float epsilon, const T* x, const AccT* gamma, const AccT* beta, AccT* running_mean,   \
      AccT* running_var, AccT* mu, AccT* rsig, AccT* params, T* y, HIPContext* ctx) {             \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_batch_norm_reduce_scratch_bytes(Tag<T>(), N, C, S, layout);   \
    HIP_CHECK(dragon_hip_batch_norm_training_forward(                                             \
        Tag<T>(), N, C, S, layout, momentum, epsilon, x, gamma, beta, running_mean, running_var,  \
        mu, rsig, params, y, Scratch(ctx, bytes), bytes, ctx->hip_stream()));                     \
  }                                                                                               \
  template <>                                                                                     \
  void BatchNormTrainingBackward<T, AccT, HIPContext>(                                            \
      const int N, const int C, const int S, const float normalizer, const string& data_format,   \
      const T* x, const AccT* mu, const AccT* rsig, const AccT* gamma, const T* dy, AccT* dgamma, \
      AccT* dbeta, T* dx, HIPContext* ctx) {                                                      \
    const int layout = LayoutTag(data_format);                                                    \
    const size_t bytes = dragon_hip_batch_norm_reduce_scratch_bytes(Tag<T>(), N, C, S, layout);   \
    HIP_CHECK(dragon_hip_batch_norm_training_backward(                                            \
        Tag<T>(), N, C, S, normalizer, layout, x, mu, rsig, gamma, dy, dgamma, dbeta, dx,         \
        Scratch(ctx, bytes), bytes, ctx->hip_stream()));                                          \
  }

DEFINE_KERNEL_LAUNCHERS(float16, float);
DEFINE_KERNEL_LAUNCHERS(bfloat16, float);
DEFINE_KERNEL_LAUNCHERS(float, float);
DEFINE_KERNEL_LAUNCHERS(double, double);
#undef DEFINE_KERNEL_LAUNCHERS

#define DEFINE_SOFTMAX_LAUNCHERS(T)                                                               \
  template <>                                                                                     \
  void Softmax<T, HIPContext>(const int N, const int S, const int C, const T* x, T* y,            \
                              HIPContext* ctx) {                                                  \
    const size_t bytes = dragon_hip_softmax_scratch_bytes(Tag<T>(), N, S, C);                     \
    HIP_CHECK(dragon_hip_softmax(Tag<T>(), N, S, C, x, y, Scratch(ctx, bytes), bytes,             \
                                 ctx->hip_stream()));                                             \
  }                                                                                               \
  template <>                                                                                     \
  void LogSoftmax<T, HIPContext>(const int N, const int S, const int C, const T* x, T* y,         \
                                 HIPContext* ctx) {                                               \
    const size_t bytes = dragon_hip_softmax_scratch_bytes(Tag<T>(), N, S, C);                     \
    HIP_CHECK(dragon_hip_log_softmax(Tag<T>(), N, S, C, x, y, Scratch(ctx, bytes), bytes,         \
                                     ctx->hip_stream()));                                         \
  }                                                                                               \
  template <>                                                                                     \
  void SoftmaxGrad<T, HIPContext>(const int N, const int S, const int C, const T* dy, const T* y, \
                                  T* dx, HIPContext* ctx) {                                       \
    const size_t bytes = dragon_hip_softmax_scratch_bytes(Tag<T>(), N, S, C);                     \
    HIP_CHECK(dragon_hip_softmax_grad(Tag<T>(), N, S, C, dy, y, dx, Scratch(ctx, bytes), bytes,   \
                                      ctx->hip_stream()));                                        \
  }                                                                                               \
  template <>                                                                                     \
  void LogSoftmaxGrad<T, HIPContext>(const int N, const int S, const int C, const T* dy,          \
                                     const T* y, T* dx, HIPContext* ctx) {                        \
    const size_t bytes = dragon_hip_softmax_scratch_bytes(Tag<T>(), N, S, C);                     \
    HIP_CHECK(dragon_hip_log_softmax_grad(Tag<T>(), N, S, C, dy, y, dx, Scratch(ctx, bytes),      \
                                          bytes, ctx->hip_stream()));                             \
  }

DEFINE_SOFTMAX_LAUNCHERS(float16);
DEFINE_SOFTMAX_LAUNCHERS(bfloat16);
DEFINE_SOFTMAX_LAUNCHERS(float);
DEFINE_SOFTMAX_LAUNCHERS(double);
#undef DEFINE_SOFTMAX_LAUNCHERS

#define DEFINE_LP_NORM_LAUNCHERS(T)                                                               \
  template <>                                                                                     \
  void L1Norm<T, HIPContext>(const int N, const int S, const int C, const float normalizer,       \
                             const float epsilon, const T* x, T* y, HIPContext* ctx) {            \
    HIP_CHECK(dragon_hip_l1_norm(Tag<T>(), N, S, C, normalizer, epsilon, x, y, ctx->hip_stream())); \
  }                                                                                               \
  template <>                                                                                     \
  void L2Norm<T, HIPContext>(const int N, const int S, const int C, const float normalizer,       \
                             const float epsilon, const T* x, T* y, HIPContext* ctx) {            \
    HIP_CHECK(dragon_hip_l2_norm(Tag<T>(), N, S, C, normalizer, epsilon, x, y, ctx->hip_stream())); \
  }                                                                                               \
  template <>                                                                                     \
  void L1NormGrad<T, HIPContext>(const int N, const int S, const int C, const float normalizer,   \
                                 const float epsilon, const T* dy, const T* x, T* dx,             \
                                 HIPContext* ctx) {                                               \
    HIP_CHECK(dragon_hip_l1_norm_grad(Tag<T>(), N, S, C, normalizer, epsilon, dy, x, dx,          \
                                      ctx->hip_stream()));                                        \
  }                                                                                               \
  template <>                                                                                     \
  void L2NormGrad<T, HIPContext>(const int N, const int S, const int C, const float normalizer,   \
                                 const float epsilon, const T* dy, const T* x, T* dx,             \
                                 HIPContext* ctx) {                                               \
    HIP_CHECK(dragon_hip_l2_norm_grad(Tag<T>(), N, S, C, normalizer, epsilon, dy, x, dx,          \
                                      ctx->hip_stream()));                                        \
  }

DEFINE_LP_NORM_LAUNCHERS(float16);
DEFINE_LP_NORM_LAUNCHERS(bfloat16);
DEFINE_LP_NORM_LAUNCHERS(float);
DEFINE_LP_NORM_LAUNCHERS(double);
#undef DEFINE_LP_NORM_LAUNCHERS

namespace {

template <typename T>
constexpr int TargetTag() {
  return sizeof(T) == 4 ? DRAGON_HIP_I32 : DRAGON_HIP_I64;
}

int ReductionTag(const string& r) {
  if (r == "NONE") return 0;
  if (r == "SUM") return 1;
  if (r == "MEAN") return 2;
  if (r == "BATCH_MEAN") return 3;
  if (r == "VALID") return 4;
  LOG(FATAL) << "Unknown reduction: " << r;
  return -1;
}

} // namespace

#define DEFINE_LOSS_LAUNCHERS(T)                                                                  \
  template <>                                                                                     \
  void CrossEntropy<T, HIPContext>(const int N, const T* input, const T* target, T* loss,         \
                                   HIPContext* ctx) {                                             \
    HIP_CHECK(dragon_hip_cross_entropy(Tag<T>(), N, input, target, loss, ctx->hip_stream()));     \
  }                                                                                               \
  template <>                                                                                     \
  void ReduceLoss<T, HIPContext>(const int N, const int num_masks, const float normalizer,        \
                                 const T* x, const T* mask, T* y, HIPContext* ctx) {              \
    const size_t bytes = dragon_hip_reduce_loss_scratch_bytes(Tag<T>());                          \
    HIP_CHECK(dragon_hip_reduce_loss(Tag<T>(), N, num_masks, normalizer, x, mask, y,              \
                                     Scratch(ctx, bytes), bytes, ctx->hip_stream()));             \
  }                                                                                               \
  template <>                                                                                     \
  void ReduceLossGrad<T, HIPContext>(const int N, const int num_masks, const float normalizer,    \
                                     const T* dl, const T* mask, T* dx, HIPContext* ctx) {        \
    const size_t bytes = dragon_hip_reduce_loss_scratch_bytes(Tag<T>());                          \
    HIP_CHECK(dragon_hip_reduce_loss_grad(Tag<T>(), N, num_masks, normalizer, dl, mask, dx,       \
                                          Scratch(ctx, bytes), bytes, ctx->hip_stream()));        \
  }                                                                                               \
  template <>                                                                                     \
  void BroadcastLossGrad<T, HIPContext>(const int N, const int S, const int C, const T* dl,       \
                                        T* dx, HIPContext* ctx) {                                 \
    HIP_CHECK(dragon_hip_broadcast_loss_grad(Tag<T>(), N, S, C, dl, dx, ctx->hip_stream()));      \
  }

DEFINE_LOSS_LAUNCHERS(float);
DEFINE_LOSS_LAUNCHERS(double);
#undef DEFINE_LOSS_LAUNCHERS

#define DEFINE_SPARSE_LOSS_LAUNCHERS(InputT, TargetT)                                             \
  template <>                                                                                     \
  void CrossEntropy<InputT, TargetT, HIPContext>(                                                 \
      const int N, const int S, const int C, const int ignore_index, const InputT* input,         \
      const TargetT* target, InputT* loss, InputT* mask, HIPContext* ctx) {                       \
    HIP_CHECK(dragon_hip_sparse_cross_entropy(Tag<InputT>(), TargetTag<TargetT>(), N, S, C,       \
                                              ignore_index, input, target, loss, mask,            \
                                              ctx->hip_stream()));                                \
  }                                                                                               \
  template <>                                                                                     \
  void SoftmaxCrossEntropyGrad<InputT, TargetT, HIPContext>(                                      \
      const int N, const int S, const int C, const int ignore_index, const InputT* input,         \
      const TargetT* target, InputT* dx, InputT* mask, HIPContext* ctx) {                         \
    HIP_CHECK(dragon_hip_softmax_cross_entropy_grad(Tag<InputT>(), TargetTag<TargetT>(), N, S, C, \
                                                    ignore_index, input, target, dx, mask,        \
                                                    ctx->hip_stream()));                          \
  }                                                                                               \
  template <>                                                                                     \
  void SoftmaxCrossEntropyLossForward<InputT, TargetT, HIPContext>(                               \
      const int N, const int S, const int C, const int ignore_index, const string& reduction,     \
      const InputT* x, const TargetT* target, InputT* prob, InputT* loss, HIPContext* ctx) {      \
    const size_t bytes = dragon_hip_softmax_cross_entropy_loss_scratch_bytes(Tag<InputT>(), N, S, C); \
    HIP_CHECK(dragon_hip_softmax_cross_entropy_loss_forward(                                      \
        Tag<InputT>(), TargetTag<TargetT>(), N, S, C, ignore_index, ReductionTag(reduction), x,   \
        target, prob, loss, Scratch(ctx, bytes), bytes, ctx->hip_stream()));                      \
  }                                                                                               \
  template <>                                                                                     \
  void SoftmaxCrossEntropyLossBackward<InputT, TargetT, HIPContext>(                              \
      const int N, const int S, const int C, const int ignore_index, const string& reduction,     \
      const InputT* prob, const TargetT* target, const InputT* dl, InputT* dx, HIPContext* ctx) { \
    const size_t bytes = dragon_hip_reduce_loss_scratch_bytes(Tag<InputT>());                     \
    HIP_CHECK(dragon_hip_softmax_cross_entropy_loss_backward(                                     \
        Tag<InputT>(), TargetTag<TargetT>(), N, S, C, ignore_index, ReductionTag(reduction),      \
        prob, target, dl, dx, Scratch(ctx, bytes), bytes, ctx->hip_stream()));                    \
  }

DEFINE_SPARSE_LOSS_LAUNCHERS(float, int);
DEFINE_SPARSE_LOSS_LAUNCHERS(float, int64_t);
DEFINE_SPARSE_LOSS_LAUNCHERS(double, int);
DEFINE_SPARSE_LOSS_LAUNCHERS(double, int64_t);
#undef DEFINE_SPARSE_LOSS_LAUNCHERS

} // namespace kernels

namespace math {

#define DEFINE_REDUCE_FUNCS(T)                                                                    \
  template <>                                                                                     \
  void ReduceSum<T, HIPContext>(const int num_dims, const int64_t* dims, const int num_axes,      \
                                const int64_t* axes, const float scale, const T* x, T* y,         \
                                HIPContext* ctx) {                                                \
    const size_t bytes = dragon_hip_reduce_scratch_bytes(Tag<T>(), num_dims, dims,       \
                                                         num_axes, axes);                         \
    HIP_CHECK(dragon_hip_reduce_sum(Tag<T>(), num_dims, dims, num_axes, axes, scale, x,  \
                                    y, Scratch(ctx, bytes), bytes, ctx->hip_stream()));  \
  }                                                                                               \
  template <>                                                                                     \
  void ReduceSumSqr<T, HIPContext>(const int num_dims, const int64_t* dims, const int num_axes,   \
                                   const int64_t* axes, const float scale, const T* x, T* y,      \
                                   HIPContext* ctx) {                                             \
    const size_t bytes = dragon_hip_reduce_scratch_bytes(Tag<T>(), num_dims, dims,       \
                                                         num_axes, axes);                         \
    HIP_CHECK(dragon_hip_reduce_sum_sqr(Tag<T>(), num_dims, dims, num_axes, axes, scale, \
                                        x, y, Scratch(ctx, bytes), bytes,                \
                                        ctx->hip_stream()));                                      \
  }

DEFINE_REDUCE_FUNCS(float16);
DEFINE_REDUCE_FUNCS(bfloat16);
DEFINE_REDUCE_FUNCS(float);
DEFINE_REDUCE_FUNCS(double);
#undef DEFINE_REDUCE_FUNCS

} // namespace math

} // namespace dragon
