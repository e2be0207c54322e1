#include "core/gradient.h"
#include "kernels/op_kernels.h"
#include "operators/norm_ops.h"

namespace dragon {

template <class Context>
template <typename T>
void LayerNormOp<Context>::DoRunWithType() {
  using AccT = typename math::Traits<T>::accumulator_type;
  Tensor& X = Input(0);
  Tensor& W = Input(1);
  Tensor& B = Input(2);
  Tensor* Y = Output(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);

  // Everything before `axis` indexes a row, everything from it on is normalised.
  const int64_t rows = X.count(0, axis);
  const int64_t width = X.count(axis);
  INITIALIZE_TENSOR_VIA_SPEC(W, vec64_t({width}), AccT);
  INITIALIZE_TENSOR_VIA_SPEC(B, vec64_t({width}), AccT);
  Tensor* X_mu = Output("X_mu")->Reshape({rows});
  Tensor* X_rsig = Output("X_rsig")->Reshape({rows});

  kernels::LayerNorm(
      static_cast<int>(rows), static_cast<int>(width), static_cast<float>(epsilon_),
      X.template data<T, Context>(ctx()), W.template data<AccT, Context>(ctx()),
      B.template data<AccT, Context>(ctx()), X_mu->template mutable_data<AccT, Context>(ctx()),
      X_rsig->template mutable_data<AccT, Context>(ctx()),
      Y->ReshapeLike(X)->template mutable_data<T, Context>(ctx()), ctx());
}

template <class Context>
void LayerNormGradientOp<Context>::GetBaseArguments() {
  Tensor& X = Input(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  this->N_ = X.count(0, axis);
  this->C_ = this->D_ = X.count(axis);
  this->G_ = this->S_ = 1;
  this->data_format_ = "NHWC";
}

DEPLOY_HIP_OPERATOR(LayerNorm);
DEPLOY_HIP_OPERATOR(LayerNormGradient);

OPERATOR_SCHEMA(LayerNorm).NumInputs(3).NumOutputs(1);          // X, W, B -> Y
OPERATOR_SCHEMA(LayerNormGradient).NumInputs(3).NumOutputs(3);  // X, W, dY -> dX, dW, dB

namespace {

// Shared by LayerNorm and GroupNorm: (X, W, dY) -> (dX, dW, dB).
class AffineNormGradientMaker final : public GradientMakerBase {
 public:
  using GradientMakerBase::GradientMakerBase;
  void CreateGradientDefs() override {
    AddGradientDef(def().type + "Gradient", {I(0), I(1), GO(0)}, {GI(0), GI(1), GI(2)});
  }
};

} // namespace

REGISTER_GRADIENT(LayerNorm, AffineNormGradientMaker);
REGISTER_GRADIENT(GroupNorm, AffineNormGradientMaker);

} // namespace dragon
