#include "core/gradient.h"
#include "kernels/op_kernels.h"
#include "operators/softmax_ops.h"

namespace dragon {

#define DEFINE_FORWARD(name, kernel)                                                     \
  template <class Context>                                                               \
  template <typename T>                                                                  \
  void name##Op<Context>::DoRunWithType() {                                              \
    Tensor& X = Input(0);                                                                \
    Tensor* Y = Output(0, {0});                                                          \
    GET_OP_AXIS_ARG(axis, X.ndim(), -1);                                                 \
    const int ax = static_cast<int>(axis);                                               \
    kernels::kernel(static_cast<int>(X.count(0, ax)), static_cast<int>(X.count(ax + 1)), \
                    static_cast<int>(X.dim(ax)), X.template data<T, Context>(ctx()),     \
                    Y->ReshapeLike(X)->template mutable_data<T, Context>(ctx()), ctx()); \
  }

#define DEFINE_BACKWARD(name, kernel)                                                    \
  template <class Context>                                                               \
  template <typename T>                                                                  \
  void name##Op<Context>::DoRunWithType() {                                              \
    Tensor& Y = Input(0);                                                                \
    Tensor& dY = Input(1);                                                               \
    Tensor* dX = Output(0, {1});                                                         \
    GET_OP_AXIS_ARG(axis, Y.ndim(), -1);                                                 \
    const int ax = static_cast<int>(axis);                                               \
    kernels::kernel(static_cast<int>(Y.count(0, ax)), static_cast<int>(Y.count(ax + 1)), \
                    static_cast<int>(Y.dim(ax)), dY.template data<T, Context>(ctx()),    \
                    Y.template data<T, Context>(ctx()),                                  \
                    dX->ReshapeLike(Y)->template mutable_data<T, Context>(ctx()), ctx()); \
  }

DEFINE_FORWARD(Softmax, Softmax)
DEFINE_FORWARD(LogSoftmax, LogSoftmax)
DEFINE_BACKWARD(SoftmaxGradient, SoftmaxGrad)
DEFINE_BACKWARD(LogSoftmaxGradient, LogSoftmaxGrad)
#undef DEFINE_FORWARD
#undef DEFINE_BACKWARD

DEPLOY_HIP_OPERATOR(Softmax);
DEPLOY_HIP_OPERATOR(SoftmaxGradient);
DEPLOY_HIP_OPERATOR(LogSoftmax);
DEPLOY_HIP_OPERATOR(LogSoftmaxGradient);

OPERATOR_SCHEMA(Softmax).NumInputs(1).NumOutputs(1).AllowInplace({{0, 0}});             // X -> Y
OPERATOR_SCHEMA(SoftmaxGradient).NumInputs(2).NumOutputs(1).AllowInplace({{1, 0}});     // Y, dY -> dX
OPERATOR_SCHEMA(LogSoftmax).NumInputs(1).NumOutputs(1).AllowInplace({{0, 0}});
OPERATOR_SCHEMA(LogSoftmaxGradient).NumInputs(2).NumOutputs(1).AllowInplace({{1, 0}});

REGISTER_GRADIENT(Softmax, InplaceGradientMaker);
REGISTER_GRADIENT(LogSoftmax, InplaceGradientMaker);

} // namespace dragon
