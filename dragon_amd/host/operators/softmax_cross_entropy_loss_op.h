// SoftmaxCrossEntropyLoss operator (forward and gradient), following
// dragon/operators/loss/cross_entropy_loss_op.h:59-98 and
// dragon/operators/loss/cross_entropy_softmax_loss_op.cc:8-143.
//
// Inputs X (logits) and Y (targets: class indices as int32 / int64, or a dense
// distribution with the type and shape of X). The softmax of X is kept in the
// side tensor "X_norm" for the gradient. "reduction" is NONE, SUM, MEAN,
// BATCH_MEAN or VALID (default: divide by the number of positions whose target
// is not "ignore_index").
#pragma once

#include <climits>

#include "core/operator.h"

namespace dragon {

#define DECLARE_SOFTMAX_CE_OP(name)                                           \
  template <class Context>                                                    \
  class name##Op final : public Operator<Context> {                           \
   public:                                                                    \
    name##Op(const OperatorDef& def, Workspace* ws)                           \
        : Operator<Context>(def, ws),                                         \
          ignore_index_(OP_SINGLE_ARG(int64_t, "ignore_index", INT_MAX)),     \
          reduction_(OP_SINGLE_ARG(string, "reduction", "VALID")) {}          \
    USE_OPERATOR_FUNCTIONS;                                                   \
    void RunOnDevice() override { LossDispatch::Call(this, Input(0)); }       \
    template <typename T>                                                     \
    void DoRunWithType();                                                     \
                                                                              \
   protected:                                                                 \
    int64_t ignore_index_;                                                    \
    string reduction_;                                                        \
  };

DECLARE_SOFTMAX_CE_OP(SoftmaxCrossEntropyLoss)
DECLARE_SOFTMAX_CE_OP(SoftmaxCrossEntropyLossGradient)
#undef DECLARE_SOFTMAX_CE_OP

} // namespace dragon
