// LpNorm operator (forward and gradient), following
// dragon/operators/normalization/lp_norm_op.{h,cc}: y = x / max(||x||_p, eps)
// over the axes [axis, end_axis], p in {1, 2}. The "MEAN" reduction divides
// the accumulated |x|^p by the number of reduced elements before the root.
#pragma once

#include "core/operator.h"

namespace dragon {

#define DECLARE_LP_NORM_OP(name)                                              \
  template <class Context>                                                    \
  class name##Op final : public Operator<Context> {                           \
   public:                                                                    \
    name##Op(const OperatorDef& def, Workspace* ws)                           \
        : Operator<Context>(def, ws),                                         \
          p_(OP_SINGLE_ARG(int64_t, "p", 2)),                                 \
          epsilon_(OP_SINGLE_ARG(double, "epsilon", 1e-12)),                  \
          reduction_(OP_SINGLE_ARG(string, "reduction", "SUM")) {}            \
    USE_OPERATOR_FUNCTIONS;                                                   \
    void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }   \
    template <typename T>                                                     \
    void DoRunWithType();                                                     \
                                                                              \
   protected:                                                                 \
    int64_t p_;                                                               \
    double epsilon_;                                                          \
    string reduction_;                                                        \
  };

DECLARE_LP_NORM_OP(LpNorm)
DECLARE_LP_NORM_OP(LpNormGradient)
#undef DECLARE_LP_NORM_OP

} // namespace dragon
