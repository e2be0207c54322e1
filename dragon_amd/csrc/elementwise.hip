// The math:: helpers Dragon's normalisation operators call on their small
// accumulator-typed buffers ([C] or [N*G] elements): InvStd, Axpby, Copy, Set,
// Square, Sub. One element per thread; these are launch-latency bound.
//
//   InvStd  dragon/utils/math/cpu/elementwise.cc:187-201   y = 1/sqrt(x + eps)
//   Axpby   dragon/utils/math/cpu/blas.cc:87-136           y = beta*y, then y += alpha*x
//   Copy    dragon/utils/math/cpu/blas.cc:8-48
//   Set     dragon/utils/math/cpu/elementwise.cc:151-186
//   Square, Sub  as used at dragon/operators/normalization/batch_norm_op.cc:45-47
#include "common.h"

namespace dragon_hip {
namespace {

enum { kInvStd, kAxpby, kCopy, kSet, kSquare, kSub };

// round(round(y * beta) + round(x * alpha)): contraction into a fused
// multiply-add is switched off so both products are rounded first.
template <typename A>
__device__ __forceinline__ A scale_then_axpy(A y, A beta, A x, A alpha) {
#pragma clang fp contract(off)
  const A scaled = y * beta;
  const A prod = x * alpha;
  return scaled + prod;
}

template <typename T, int kOp>
__global__ __launch_bounds__(256) void elementwise_kernel(
    const int64_t N, const typename IO<T>::Acc p0, const typename IO<T>::Acc p1, const T* a,
    const T* b, T* y) {
  using A = typename IO<T>::Acc;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < N;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    A r;
    if (kOp == kInvStd) {
      r = acc_rsqrt_exact(IO<T>::load1(a + i) + p0);
    } else if (kOp == kAxpby) {
      // Two roundings like the reference's Scale-then-Axpy pair, no fused multiply-add.
      r = scale_then_axpy(IO<T>::load1(y + i), p1, IO<T>::load1(a + i), p0);
    } else if (kOp == kCopy) {
      r = IO<T>::load1(a + i);
    } else if (kOp == kSet) {
      r = p0;
    } else if (kOp == kSquare) {
      const A v = IO<T>::load1(a + i);
      r = v * v;
    } else {
      r = IO<T>::load1(a + i) - IO<T>::load1(b + i);
    }
    IO<T>::store1(y + i, r);
  }
}

template <typename T, int kOp>
int launch_elementwise(int64_t N, float p0, float p1, const void* a, const void* b, void* y,
                       hipStream_t stream) {
  using A = typename IO<T>::Acc;
  if (N == 0) return DRAGON_HIP_OK;
  const int64_t blocks = ceil_div(N, 256);
  hipLaunchKernelGGL((elementwise_kernel<T, kOp>), dim3(static_cast<unsigned>(blocks < 65536 ? blocks : 65536)),
                     dim3(256), 0, stream, N, A(p0), A(p1), static_cast<const T*>(a),
                     static_cast<const T*>(b), static_cast<T*>(y));
  return status_of_launch();
}

#define DEFINE_OP(fn, op)                                                                   \
  template <typename T>                                                                     \
  int fn(int64_t N, float p0, float p1, const void* a, const void* b, void* y, hipStream_t s) { \
    return launch_elementwise<T, op>(N, p0, p1, a, b, y, s);                                \
  }
DEFINE_OP(inv_std_t, kInvStd)
DEFINE_OP(axpby_t, kAxpby)
DEFINE_OP(copy_t, kCopy)
DEFINE_OP(set_t, kSet)
DEFINE_OP(square_t, kSquare)
DEFINE_OP(sub_t, kSub)
#undef DEFINE_OP

} // namespace
} // namespace dragon_hip

extern "C" {

int dragon_hip_inv_std(int dtype, int64_t N, float eps, const void* x, void* y, void* stream) {
  if (N < 0 || (N > 0 && (!x || !y))) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::inv_std_t, N, eps, 0.f, x, nullptr, y, s);
}
int dragon_hip_axpby(int dtype, int64_t N, float alpha, const void* x, float beta, void* y,
                     void* stream) {
  if (N < 0 || (N > 0 && (!x || !y))) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::axpby_t, N, alpha, beta, x, nullptr, y, s);
}
int dragon_hip_copy(int dtype, int64_t N, const void* x, void* y, void* stream) {
  if (N < 0 || (N > 0 && (!x || !y))) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::copy_t, N, 0.f, 0.f, x, nullptr, y, s);
}
int dragon_hip_set(int dtype, int64_t N, float value, void* y, void* stream) {
  if (N < 0 || (N > 0 && !y)) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::set_t, N, value, 0.f, nullptr, nullptr, y, s);
}
int dragon_hip_square(int dtype, int64_t N, const void* x, void* y, void* stream) {
  if (N < 0 || (N > 0 && (!x || !y))) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::square_t, N, 0.f, 0.f, x, nullptr, y, s);
}
int dragon_hip_sub(int dtype, int64_t N, const void* a, const void* b, void* y, void* stream) {
  if (N < 0 || (N > 0 && (!a || !b || !y))) return DRAGON_HIP_EINVAL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DRAGON_HIP_DISPATCH_DTYPE(dtype, dragon_hip::sub_t, N, 0.f, 0.f, a, b, y, s);
}

} // extern "C"
