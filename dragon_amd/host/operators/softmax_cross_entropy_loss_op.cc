#include "core/gradient.h"
#include "core/workspace.h"
#include "kernels/op_kernels.h"
#include "operators/softmax_cross_entropy_loss_op.h"

namespace dragon {

namespace {

// cross_entropy_softmax_loss_op.cc:69-78; -1 selects the count of valid targets.
int64_t LossNormalizer(const string& reduction, int64_t NxS, int64_t dim0, bool has_mask) {
  if (reduction == "VALID") return has_mask ? -1 : NxS;
  if (reduction == "BATCH_MEAN") return dim0;
  if (reduction == "MEAN") return NxS;
  return 1;
}

} // namespace

template <class Context>
template <typename T>
void SoftmaxCrossEntropyLossOp<Context>::DoRunWithType() {
  Tensor& X = Input(0);
  Tensor& Y = Input(1);
  Tensor* L = Output(0);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  const int ax = static_cast<int>(axis);
  const int C = static_cast<int>(X.dim(ax));
  const int N = static_cast<int>(X.count(0, ax));
  const int S = static_cast<int>(X.count(ax + 1));
  const int NxS = N * S;
  const int NxCxS = static_cast<int>(X.count());
  const bool target_is_dense = Y.meta() == TypeOf<T>::value;
  const int ignore_index = static_cast<int>(ignore_index_);

  Tensor* X_norm = Output("X_norm")->ReshapeLike(X);
  const T* x = X.template data<T, Context>(ctx());
  T* input = X_norm->template mutable_data<T, Context>(ctx());
  vec64_t out_dims = X.dims();
  out_dims.erase(out_dims.begin() + ax);
  if (reduction_ != "NONE") out_dims.clear();

  if (target_is_dense) {
    CHECK_EQ(Y.count(), NxCxS) << "\nNumel of X and Y must be matched.";
    kernels::Softmax(N, S, C, x, input, ctx());
    T* loss = ctx()->workspace()->template data<T, Context>(NxCxS, "BufferShared", ctx());
    kernels::CrossEntropy(NxCxS, input, Y.template data<T, Context>(ctx()), loss, ctx());
    T* out = L->Reshape(out_dims)->template mutable_data<T, Context>(ctx());
    if (reduction_ == "NONE") {
      const vec64_t dims = {N, C, S}, axes = {1};
      math::ReduceSum(3, dims.data(), 1, axes.data(), 1.f, loss, out, ctx());
    } else {
      kernels::ReduceLoss(NxCxS, 0, float(LossNormalizer(reduction_, NxS, X.dim(0), false)), loss,
                          static_cast<const T*>(nullptr), out, ctx());
    }
    return;
  }

  CHECK_EQ(Y.count(), NxS) << "\nNumel of X and Y must be matched.";
  CHECK(Y.meta() == DType::kInt32 || Y.meta() == DType::kInt64)
      << this->MessageForUnsupported(NameOf(Y.meta()), {"int32", "int64", NameOf(TypeOf<T>::value)});
  T* out = L->Reshape(out_dims)->template mutable_data<T, Context>(ctx());
  // One pass over the logits unless BATCH_MEAN divides by a leading extent
  // that is not the N of the [N, C, S] view.
  const bool fused = reduction_ != "BATCH_MEAN" || X.dim(0) == N;
  if (fused) {
    if (Y.meta() == DType::kInt32) {
      kernels::SoftmaxCrossEntropyLossForward(N, S, C, ignore_index, reduction_, x,
                                              Y.template data<int, Context>(ctx()), input, out, ctx());
    } else {
      kernels::SoftmaxCrossEntropyLossForward(N, S, C, ignore_index, reduction_, x,
                                              Y.template data<int64_t, Context>(ctx()), input, out,
                                              ctx());
    }
    return;
  }
  kernels::Softmax(N, S, C, x, input, ctx());
  T* scratch = ctx()->workspace()->template data<T, Context>(NxS * 2 + 1, "BufferShared", ctx());
  T *loss = scratch, *mask = scratch + NxS;
  if (Y.meta() == DType::kInt32) {
    kernels::CrossEntropy(N, S, C, ignore_index, input, Y.template data<int, Context>(ctx()), loss,
                          mask, ctx());
  } else {
    kernels::CrossEntropy(N, S, C, ignore_index, input, Y.template data<int64_t, Context>(ctx()),
                          loss, mask, ctx());
  }
  kernels::ReduceLoss(NxS, NxS, float(LossNormalizer(reduction_, NxS, X.dim(0), true)), loss, mask,
                      out, ctx());
}

template <class Context>
template <typename T>
void SoftmaxCrossEntropyLossGradientOp<Context>::DoRunWithType() {
  Tensor& X = Input(0);
  Tensor& Y = Input(1);
  Tensor& dL = Input(2);
  Tensor* dX = Output(0)->ReshapeLike(X);
  GET_OP_AXIS_ARG(axis, X.ndim(), -1);
  const int ax = static_cast<int>(axis);
  const int C = static_cast<int>(X.dim(ax));
  const int N = static_cast<int>(X.count(0, ax));
  const int S = static_cast<int>(X.count(ax + 1));
  const int NxS = N * S;
  const int NxCxS = static_cast<int>(X.count());
  const int ignore_index = static_cast<int>(ignore_index_);

  const T* input = Input("X_norm").template data<T, Context>(ctx());
  const T* dl = dL.template data<T, Context>(ctx());
  T* dx = dX->template mutable_data<T, Context>(ctx());

  if (Y.meta() == TypeOf<T>::value) {
    math::Sub(NxCxS, input, Y.template data<T, Context>(ctx()), dx, ctx());  // Copy + Axpy(-1)
    if (reduction_ == "NONE") {
      kernels::BroadcastLossGrad(N, S, C, dl, dx, ctx());
    } else {
      kernels::ReduceLossGrad(NxCxS, 0, float(LossNormalizer(reduction_, NxS, X.dim(0), false)), dl,
                              static_cast<const T*>(nullptr), dx, ctx());
    }
    return;
  }

  CHECK(Y.meta() == DType::kInt32 || Y.meta() == DType::kInt64)
      << this->MessageForUnsupported(NameOf(Y.meta()), {"int32", "int64", NameOf(TypeOf<T>::value)});
  const bool fused = reduction_ != "BATCH_MEAN" || X.dim(0) == N;
  if (fused) {
    if (Y.meta() == DType::kInt32) {
      kernels::SoftmaxCrossEntropyLossBackward(N, S, C, ignore_index, reduction_, input,
                                               Y.template data<int, Context>(ctx()), dl, dx, ctx());
    } else {
      kernels::SoftmaxCrossEntropyLossBackward(N, S, C, ignore_index, reduction_, input,
                                               Y.template data<int64_t, Context>(ctx()), dl, dx,
                                               ctx());
    }
    return;
  }
  math::Copy(NxCxS, input, dx, ctx());
  T* mask = ctx()->workspace()->template data<T, Context>(NxS + 1, "BufferShared", ctx());
  if (Y.meta() == DType::kInt32) {
    kernels::SoftmaxCrossEntropyGrad(N, S, C, ignore_index, input,
                                     Y.template data<int, Context>(ctx()), dx, mask, ctx());
  } else {
    kernels::SoftmaxCrossEntropyGrad(N, S, C, ignore_index, input,
                                     Y.template data<int64_t, Context>(ctx()), dx, mask, ctx());
  }
  kernels::ReduceLossGrad(NxCxS, NxS, float(LossNormalizer(reduction_, NxS, X.dim(0), true)), dl,
                          mask, dx, ctx());
}

DEPLOY_HIP_OPERATOR(SoftmaxCrossEntropyLoss);
DEPLOY_HIP_OPERATOR(SoftmaxCrossEntropyLossGradient);

OPERATOR_SCHEMA(SoftmaxCrossEntropyLoss).NumInputs(2).NumOutputs(1);          // X, Y -> L
OPERATOR_SCHEMA(SoftmaxCrossEntropyLossGradient).NumInputs(3).NumOutputs(1);  // X, Y, dL -> dX

namespace {

class LossGradientMaker final : public GradientMakerBase {
 public:
  using GradientMakerBase::GradientMakerBase;
  void CreateGradientDefs() override {
    AddGradientDef(def().type + "Gradient", {I(0), I(1), GO(0)}, {GI(0)});
  }
};

} // namespace

REGISTER_GRADIENT(SoftmaxCrossEntropyLoss, LossGradientMaker);

} // namespace dragon
