// Softmax and LogSoftmax operators (forward and gradient), following
// dragon/operators/activation/softmax_op.{h,cc} and log_softmax_op.{h,cc}:
// the "axis" argument (default -1) splits the shape into N = count(0, axis)
// outer slices, C = dim(axis) reduced elements and S = count(axis + 1) inner
// stride. Forward may run in place (Y over X), backward may write dX over dY.
#pragma once

#include "core/operator.h"

namespace dragon {

#define DECLARE_SOFTMAX_LIKE_OP(name)                                         \
  template <class Context>                                                    \
  class name##Op final : public Operator<Context> {                           \
   public:                                                                    \
    name##Op(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {} \
    USE_OPERATOR_FUNCTIONS;                                                   \
    void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }   \
    template <typename T>                                                     \
    void DoRunWithType();                                                     \
  };

DECLARE_SOFTMAX_LIKE_OP(Softmax)
DECLARE_SOFTMAX_LIKE_OP(SoftmaxGradient)
DECLARE_SOFTMAX_LIKE_OP(LogSoftmax)
DECLARE_SOFTMAX_LIKE_OP(LogSoftmaxGradient)
#undef DECLARE_SOFTMAX_LIKE_OP

} // namespace dragon
