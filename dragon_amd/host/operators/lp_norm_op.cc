#include "core/gradient.h"
#include "kernels/op_kernels.h"
#include "operators/lp_norm_op.h"

namespace dragon {

template <class Context>
template <typename T>
void LpNormOp<Context>::DoRunWithType() {
  Tensor& X = Input(0);
  Tensor* Y = Output(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  GET_OP_AXIS_ARG(end_axis, X.ndim(), axis);
  const int a = static_cast<int>(axis), b = static_cast<int>(end_axis);
  const int reduce_dim = static_cast<int>(X.count(a, b + 1));
  const float normalizer = reduction_ == "MEAN" ? static_cast<float>(reduce_dim) : 1.f;
  const int N = static_cast<int>(X.count(0, a)), S = static_cast<int>(X.count(b + 1));
  const T* x = X.template data<T, Context>(ctx());
  T* y = Y->ReshapeLike(X)->template mutable_data<T, Context>(ctx());
  if (p_ == 1) {
    kernels::L1Norm(N, S, reduce_dim, normalizer, static_cast<float>(epsilon_), x, y, ctx());
  } else if (p_ == 2) {
    kernels::L2Norm(N, S, reduce_dim, normalizer, static_cast<float>(epsilon_), x, y, ctx());
  } else {
    LOG(FATAL) << "Unsupported order of normalization: " << p_;
  }
}

template <class Context>
template <typename T>
void LpNormGradientOp<Context>::DoRunWithType() {
  Tensor& X = Input(0);
  Tensor& dY = Input(1);
  Tensor* dX = Output(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  GET_OP_AXIS_ARG(end_axis, X.ndim(), axis);
  const int a = static_cast<int>(axis), b = static_cast<int>(end_axis);
  const int reduce_dim = static_cast<int>(X.count(a, b + 1));
  const float normalizer = reduction_ == "MEAN" ? static_cast<float>(reduce_dim) : 1.f;
  const int N = static_cast<int>(X.count(0, a)), S = static_cast<int>(X.count(b + 1));
  const T* dy = dY.template data<T, Context>(ctx());
  const T* x = X.template data<T, Context>(ctx());
  T* dx = dX->ReshapeLike(X)->template mutable_data<T, Context>(ctx());
  if (p_ == 1) {
    kernels::L1NormGrad(N, S, reduce_dim, normalizer, static_cast<float>(epsilon_), dy, x, dx, ctx());
  } else if (p_ == 2) {
    kernels::L2NormGrad(N, S, reduce_dim, normalizer, static_cast<float>(epsilon_), dy, x, dx, ctx());
  } else {
    LOG(FATAL) << "Unsupported order of LpNormalization: " << p_;
  }
}

DEPLOY_HIP_OPERATOR(LpNorm);
DEPLOY_HIP_OPERATOR(LpNormGradient);

OPERATOR_SCHEMA(LpNorm).NumInputs(1).NumOutputs(1);          // X -> Y
OPERATOR_SCHEMA(LpNormGradient).NumInputs(2).NumOutputs(1);  // X, dY -> dX

REGISTER_GRADIENT(LpNorm, GenericGradientMaker);

} // namespace dragon
