// LayerNorm, GroupNorm and BatchNorm operators (forward and gradient) for any
// device context that provides the kernels:: functions of kernels/op_kernels.h.
//
// Argument names and defaults, shape derivation, parameter checks, side
// outputs ("<op name>/X_mu", "/X_rsig", "/X_params") and scratch use follow
// the reference operators:
//   dragon/operators/normalization/layer_norm_op.{h,cc}
//   dragon/operators/normalization/group_norm_op.{h,cc}
//   dragon/operators/normalization/batch_norm_op.{h,cc}, batch_norm_op_sync.cc
// The forward bodies of GroupNorm and training-mode BatchNorm issue one fused
// kernel call where the reference issues Moments / InvStd / Axpby / affine
// separately; results are the same sequence's results.
#pragma once

#include "core/operator.h"

namespace dragon {

// ---------------------------------------------------------------- LayerNorm

template <class Context>
class LayerNormOp final : public Operator<Context> {
 public:
  LayerNormOp(const OperatorDef& def, Workspace* ws)
      : Operator<Context>(def, ws), epsilon_(OP_SINGLE_ARG(double, "epsilon", 1e-5)) {}
  USE_OPERATOR_FUNCTIONS;

  void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }

  template <typename T>
  void DoRunWithType();

 protected:
  double epsilon_;
};

// ---------------------------------------------------------------- GroupNorm

template <class Context>
class GroupNormOpBase : public Operator<Context> {
 public:
  GroupNormOpBase(const OperatorDef& def, Workspace* ws)
      : Operator<Context>(def, ws), epsilon_(OP_SINGLE_ARG(double, "epsilon", 1e-5)) {}
  USE_OPERATOR_FUNCTIONS;

  // N = dim(0), C = dim(axis), S = everything else; "group" = 0 means one
  // group per channel (InstanceNorm); channel-last inputs are "NHWC".
  virtual void GetBaseArguments();

 protected:
  double epsilon_;
  int64_t N_ = 0, C_ = 0, G_ = 0, D_ = 0, S_ = 0;
};

template <class Context>
class GroupNormOp final : public GroupNormOpBase<Context> {
 public:
  GroupNormOp(const OperatorDef& def, Workspace* ws) : GroupNormOpBase<Context>(def, ws) {}
  USE_OPERATOR_FUNCTIONS;

  void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }

  template <typename T>
  void DoRunWithType();
};

template <class Context>
class GroupNormGradientOp : public GroupNormOpBase<Context> {
 public:
  GroupNormGradientOp(const OperatorDef& def, Workspace* ws) : GroupNormOpBase<Context>(def, ws) {}
  USE_OPERATOR_FUNCTIONS;

  void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }

  template <typename T>
  void DoRunWithType();
};

// LayerNorm backward is GroupNorm backward over rows: N = count(0, axis),
// one group of D = count(axis) channels, S = 1, channel-last.
template <class Context>
class LayerNormGradientOp final : public GroupNormGradientOp<Context> {
 public:
  LayerNormGradientOp(const OperatorDef& def, Workspace* ws) : GroupNormGradientOp<Context>(def, ws) {}
  USE_OPERATOR_FUNCTIONS;

  void GetBaseArguments() override;
};

// ---------------------------------------------------------------- BatchNorm

template <class Context>
class BatchNormOpBase : public Operator<Context> {
 public:
  BatchNormOpBase(const OperatorDef& def, Workspace* ws)
      : Operator<Context>(def, ws),
        epsilon_(OP_SINGLE_ARG(double, "epsilon", 1e-5)),
        use_stats_(OP_SINGLE_ARG(int64_t, "use_stats", -1)),
        sync_stats_(OP_SINGLE_ARG(int64_t, "comm", 0) > 0 ? 1 : 0) {}
  USE_OPERATOR_FUNCTIONS;

  // N = dim(0), C = dim(axis), S = everything else; training unless use_stats
  // says otherwise (use_stats < 0 defers to the phase).
  void GetBaseArguments();

 protected:
  double epsilon_;
  int64_t N_ = 0, C_ = 0, S_ = 0;
  int64_t use_stats_, sync_stats_;
  int64_t training_ = 1;
};

template <class Context>
class BatchNormOp final : public BatchNormOpBase<Context> {
 public:
  BatchNormOp(const OperatorDef& def, Workspace* ws)
      : BatchNormOpBase<Context>(def, ws), momentum_(OP_SINGLE_ARG(float, "momentum", 0.9f)) {}
  USE_OPERATOR_FUNCTIONS;

  void Setup() override {
    this->GetBaseArguments();
    Output(0)->ReshapeLike(Input(0));
  }
  void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }

  template <typename T>
  void RunTraining();
  template <typename T>
  void RunInference();
  template <typename T>
  void DoRunWithType() {
    if (this->training_) {
      RunTraining<T>();
    } else {
      RunInference<T>();
    }
  }

  float momentum() const { return momentum_; }

 protected:
  float momentum_;
};

template <class Context>
class BatchNormGradientOp final : public BatchNormOpBase<Context> {
 public:
  BatchNormGradientOp(const OperatorDef& def, Workspace* ws) : BatchNormOpBase<Context>(def, ws) {}
  USE_OPERATOR_FUNCTIONS;

  void Setup() override {
    this->GetBaseArguments();
    Output(0)->ReshapeLike(Input(0));
  }
  void RunOnDevice() override { FloatingDispatch::Call(this, Input(0)); }

  template <typename T>
  void RunTraining();
  template <typename T>
  void RunInference();
  template <typename T>
  void DoRunWithType() {
    if (this->training_) {
      RunTraining<T>();
    } else {
      RunInference<T>();
    }
  }
};

} // namespace dragon
