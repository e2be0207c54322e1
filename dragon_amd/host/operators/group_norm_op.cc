#include "kernels/op_kernels.h"
#include "operators/norm_ops.h"

namespace dragon {

template <class Context>
void GroupNormOpBase<Context>::GetBaseArguments() {
  Tensor& X = Input(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  N_ = X.dim(0);
  C_ = X.dim(static_cast<int>(axis));
  S_ = (N_ * C_ > 0) ? X.count() / N_ / C_ : 0;
  G_ = OP_SINGLE_ARG(int64_t, "group", 0);
  if (G_ <= 0) G_ = C_;
  CHECK_EQ(C_ % G_, 0) << "\nThe " << C_ << " channels can not be split into " << G_ << " groups.";
  D_ = C_ / G_;
  this->data_format_ = (axis + 1 == X.ndim()) ? "NHWC" : "NCHW";
}

template <class Context>
template <typename T>
void GroupNormOp<Context>::DoRunWithType() {
  using AccT = typename math::Traits<T>::accumulator_type;
  Tensor& X = Input(0);
  Tensor& W = Input(1);
  Tensor& B = Input(2);
  Tensor* Y = Output(0);
  this->GetBaseArguments();
  INITIALIZE_TENSOR_VIA_SPEC(W, vec64_t({this->C_}), AccT);
  INITIALIZE_TENSOR_VIA_SPEC(B, vec64_t({this->C_}), AccT);
  Tensor* X_mu = Output("X_mu")->Reshape({this->N_, this->G_});
  Tensor* X_rsig = Output("X_rsig")->Reshape({this->N_, this->G_});

  // Group moments, inverse standard deviation and the affine normalisation in
  // one call; a group that fits the register file is read from HBM once.
  kernels::GroupNormForward(
      static_cast<int>(this->N_), static_cast<int>(this->G_), static_cast<int>(this->D_),
      static_cast<int>(this->S_), data_format(), static_cast<float>(this->epsilon_),
      X.template data<T, Context>(ctx()), W.template data<AccT, Context>(ctx()),
      B.template data<AccT, Context>(ctx()), X_mu->template mutable_data<AccT, Context>(ctx()),
      X_rsig->template mutable_data<AccT, Context>(ctx()),
      Y->ReshapeLike(X)->template mutable_data<T, Context>(ctx()), ctx());
}

template <class Context>
template <typename T>
void GroupNormGradientOp<Context>::DoRunWithType() {
  using AccT = typename math::Traits<T>::accumulator_type;
  Tensor& X = Input(0);
  Tensor& W = Input(1);
  Tensor& dY = Input(2);
  Tensor& X_mu = Input("X_mu");
  Tensor& X_rsig = Input("X_rsig");
  Tensor* dX = Output(0);
  Tensor* dW = Output(1);
  Tensor* dB = Output(2);
  this->GetBaseArguments();

  // ds and db of every group, packed into one 2*N*G scratch buffer that is
  // passed for both (the kernel places db behind ds).
  const int64_t num_groups = this->N_ * this->G_;
  AccT* params = ctx()->workspace()->template data<AccT, Context>(2 * num_groups, "BufferShared", ctx());

  kernels::GroupNormGrad(
      static_cast<int>(this->N_), static_cast<int>(this->G_), static_cast<int>(this->D_),
      static_cast<int>(this->S_), data_format(), X.template data<T, Context>(ctx()),
      X_mu.template data<AccT, Context>(ctx()), X_rsig.template data<AccT, Context>(ctx()),
      W.template data<AccT, Context>(ctx()), dY.template data<T, Context>(ctx()), params, params,
      dW->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx()),
      dB->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx()),
      dX->ReshapeLike(X)->template mutable_data<T, Context>(ctx()), ctx());
}

DEPLOY_HIP_OPERATOR(GroupNorm);
DEPLOY_HIP_OPERATOR(GroupNormGradient);

OPERATOR_SCHEMA(GroupNorm).NumInputs(3).NumOutputs(1);          // X, W, B -> Y
OPERATOR_SCHEMA(GroupNormGradient).NumInputs(3).NumOutputs(3);  // X, W, dY -> dX, dW, dB

} // namespace dragon
