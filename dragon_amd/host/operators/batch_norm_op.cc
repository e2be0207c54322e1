#include "core/gradient.h"
#include "kernels/op_kernels.h"
#include "operators/norm_ops.h"

namespace dragon {

template <class Context>
void BatchNormOpBase<Context>::GetBaseArguments() {
  Tensor& X = Input(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  N_ = X.dim(0);
  C_ = X.dim(static_cast<int>(axis));
  S_ = (N_ * C_ > 0) ? X.count() / N_ / C_ : 0;
  this->data_format_ = (axis + 1 == X.ndim()) ? "NHWC" : "NCHW";
  if (use_stats_ < 0) {
    training_ = phase() == "TRAIN" ? 1 : 0;
  } else {
    training_ = use_stats_ > 0 ? 0 : 1;
  }
  // Cross-rank statistics need the collective backend, which one GPU has no
  // use for: the two all-reduces of the sync path are not part of this build.
  CHECK_EQ(sync_stats_, 0) << "\nSynchronised statistics (comm > 0) need a collective backend "
                           << "that this single-device build does not provide.";
}

template <class Context>
template <typename T>
void BatchNormOp<Context>::RunTraining() {
  using AccT = typename math::Traits<T>::accumulator_type;
  const vec64_t param_shape({this->C_});
  INITIALIZE_TENSOR_VIA_SPEC(Input(1), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(2), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(3), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(4), param_shape, AccT);
  Tensor* X_mu = Output("X_mu")->Reshape({this->C_});
  Tensor* X_rsig = Output("X_rsig")->Reshape({this->C_});
  Tensor* X_params = Output("X_params")->Reshape({this->C_ * 2});

  // One call for: batch moments; running_mean/var <- momentum * running +
  // (1 - momentum) * batch (biased variance); rsig = 1/sqrt(var + eps);
  // scale = gamma*rsig, bias = beta - scale*mu into X_params; y = x*scale + bias.
  kernels::BatchNormTrainingForward(
      static_cast<int>(this->N_), static_cast<int>(this->C_), static_cast<int>(this->S_),
      data_format(), momentum_, static_cast<float>(this->epsilon_),
      Input(0).template data<T, Context>(ctx()), Input(1).template data<AccT, Context>(ctx()),
      Input(2).template data<AccT, Context>(ctx()),
      Input(3).template mutable_data<AccT, Context>(ctx()),
      Input(4).template mutable_data<AccT, Context>(ctx()),
      X_mu->template mutable_data<AccT, Context>(ctx()),
      X_rsig->template mutable_data<AccT, Context>(ctx()),
      X_params->template mutable_data<AccT, Context>(ctx()),
      Output(0)->template mutable_data<T, Context>(ctx()), ctx());
}

template <class Context>
template <typename T>
void BatchNormOp<Context>::RunInference() {
  using AccT = typename math::Traits<T>::accumulator_type;
  const vec64_t param_shape({this->C_});
  INITIALIZE_TENSOR_VIA_SPEC(Input(1), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(2), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(3), param_shape, AccT);
  INITIALIZE_TENSOR_VIA_SPEC(Input(4), param_shape, AccT);
  // X_params = {rsig, scale, bias}: passing it as rsig, scale and bias selects
  // the three-part layout in the kernel.
  Tensor* X_params = Output("X_params")->Reshape({this->C_ * 3});
  AccT* params = X_params->template mutable_data<AccT, Context>(ctx());
  math::InvStd(static_cast<int>(this->C_), static_cast<float>(this->epsilon_),
               Input(4).template data<AccT, Context>(ctx()), params, ctx());
  kernels::BatchNorm(
      static_cast<int>(this->N_), static_cast<int>(this->C_), static_cast<int>(this->S_),
      data_format(), Input(0).template data<T, Context>(ctx()),
      Input(3).template data<AccT, Context>(ctx()), static_cast<const AccT*>(params),
      Input(1).template data<AccT, Context>(ctx()), Input(2).template data<AccT, Context>(ctx()),
      params, params, Output(0)->template mutable_data<T, Context>(ctx()), ctx());
}

template <class Context>
template <typename T>
void BatchNormGradientOp<Context>::RunTraining() {
  using AccT = typename math::Traits<T>::accumulator_type;
  Tensor* dX = Output(0);
  Tensor* dW = Output(1);
  Tensor* dB = Output(2);
  Tensor& X_mu = Input("X_mu");
  Tensor& X_rsig = Input("X_rsig");
  Tensor* X_params = Output("X_params")->Reshape({this->C_ * 2});

  const T* x = Input(0).template data<T, Context>(ctx());
  const AccT* gamma = Input(1).template data<AccT, Context>(ctx());
  const T* dy = Input(4).template data<T, Context>(ctx());
  const AccT* mu = X_mu.template data<AccT, Context>(ctx());
  const AccT* rsig = X_rsig.template data<AccT, Context>(ctx());
  AccT* params = X_params->template mutable_data<AccT, Context>(ctx());
  const int N = static_cast<int>(this->N_), C = static_cast<int>(this->C_), S = static_cast<int>(this->S_);

  // {dgamma, dbeta} packed in X_params, then copied out to the requested outputs.
  // Without cross-rank statistics nothing separates the two kernels of the
  // reference's body, so they run as one call that reads x and dy once.
  if (dX->has_name()) {
    kernels::BatchNormTrainingBackward(
        N, C, S, static_cast<float>(this->N_ * this->S_), data_format(), x, mu, rsig, gamma, dy,
        params, params, dX->template mutable_data<T, Context>(ctx()), ctx());
  } else {
    kernels::BatchNormWGrad(N, C, S, data_format(), x, mu, rsig, dy, params, params, ctx());
  }
  if (dW->has_name()) {
    math::Copy(C, static_cast<const AccT*>(params),
               dW->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx()), ctx());
  }
  if (dB->has_name()) {
    math::Copy(C, static_cast<const AccT*>(params + C),
               dB->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx()), ctx());
  }
}

template <class Context>
template <typename T>
void BatchNormGradientOp<Context>::RunInference() {
  using AccT = typename math::Traits<T>::accumulator_type;
  Tensor* dX = Output(0);
  Tensor* dW = Output(1);
  Tensor* dB = Output(2);
  Tensor* X_params = Output("X_params")->Reshape({this->C_});
  AccT* rsig = X_params->template mutable_data<AccT, Context>(ctx());
  AccT* dgamma = nullptr;
  AccT* dbeta = nullptr;
  if (dW->has_name() || dB->has_name()) {
    dgamma = dW->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx());
    dbeta = dB->Reshape({this->C_})->template mutable_data<AccT, Context>(ctx());
  }
  math::InvStd(static_cast<int>(this->C_), static_cast<float>(this->epsilon_),
               Input(3).template data<AccT, Context>(ctx()), rsig, ctx());
  kernels::BatchNormInferenceGrad(
      static_cast<int>(this->N_), static_cast<int>(this->C_), static_cast<int>(this->S_),
      data_format(), Input(0).template data<T, Context>(ctx()),
      Input(2).template data<AccT, Context>(ctx()), static_cast<const AccT*>(rsig),
      Input(1).template data<AccT, Context>(ctx()), Input(4).template data<T, Context>(ctx()),
      dgamma, dbeta, dX->template mutable_data<T, Context>(ctx()), ctx());
}

DEPLOY_HIP_OPERATOR(BatchNorm);
DEPLOY_HIP_OPERATOR(BatchNormGradient);
// SyncBatchNorm is the same pair of classes (batch_norm_op_sync.cc:5-10); with
// comm == 0 it is BatchNorm, with comm > 0 it reports the missing backend.
REGISTER_HIP_OPERATOR(SyncBatchNorm, BatchNormOp<HIPContext>);
REGISTER_HIP_OPERATOR(SyncBatchNormGradient, BatchNormGradientOp<HIPContext>);

OPERATOR_SCHEMA(BatchNorm).NumInputs(5).NumOutputs(1);          // X, W, B, M, V -> Y
OPERATOR_SCHEMA(BatchNormGradient).NumInputs(5).NumOutputs(3);  // X, W, M, V, dY -> dX, dW, dB
OPERATOR_SCHEMA(SyncBatchNorm).NumInputs(5).NumOutputs(1);
OPERATOR_SCHEMA(SyncBatchNormGradient).NumInputs(5).NumOutputs(3);

namespace {

class BatchNormGradientMaker final : public GradientMakerBase {
 public:
  using GradientMakerBase::GradientMakerBase;
  void CreateGradientDefs() override {
    AddGradientDef(def().type + "Gradient", {I(0), I(1), I(3), I(4), GO(0)}, {GI(0), GI(1), GI(2)});
  }
};

} // namespace

REGISTER_GRADIENT(BatchNorm, BatchNormGradientMaker);
REGISTER_GRADIENT(SyncBatchNorm, BatchNormGradientMaker);

} // namespace dragon
