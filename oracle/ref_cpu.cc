// CPU oracle: a loop-for-loop restatement of Dragon's CPU kernels for
// LayerNorm, GroupNorm, BatchNorm, Moments, Softmax/LogSoftmax, L1/L2Norm,
// ReduceSum and the softmax cross-entropy loss.
//
// THIS FILE IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are
// compared against and the CPU baseline that is timed beside them. Nothing in
// the product path may link, import or call it.
//
// Every function follows one reference function (cited as file:line relative
// to the reference tree) with the same accumulation order, the same formula
// and the same pointer-aliasing conventions. Where the reference uses an Eigen
// array expression (Eigen is an un-vendored submodule, so its version is not
// pinned) the expression is restated as a scalar loop with std::exp, std::log
// and 1/std::sqrt: same semantics, last-ulp rounding may differ.
//
// Pinning status (what fixes each function independent of this restatement):
//   softmax / log_softmax (+grad)  reference test literals, test_ops.py:363-377,588-601
//   layer_norm, group_norm_grad    reference test literals, test_ops.py:4232-4291,4303-4351,4363-4397
//   moments                        numpy mean/var closed form, test_ops.py:3489-3511
//   batch_norm fwd/bwd             numpy closed forms,  test_ops.py:4127-4181
//   reduce_sum / _sum_sqr / _l1    numpy sum closed forms (the reference's reduce
//                                  tests compare with numpy, test_ops.py TestReduceOps)
//   cross_entropy*, reduce_loss*,  the numpy closed form of test_ops.py:2260-2296 (sparse
//   broadcast_loss_grad            and dense targets, reductions mean / sum / none);
//                                  ignore_index and VALID / BATCH_MEAN normalisation are
//                                  PARITY UNPINNED by any reference test, checked against
//                                  the formulas of the operator body only
//   lp_norm (+grad)                reference test literals and the numpy closed
//                                  form of test_ops.py:4480-4512
//   f16 / bf16 conversions         exhaustive comparison against numpy float16 and
//                                  a bit-level bf16 RNE over all 2^16 encodings
//   running-stat update (axpby)    the formula the reference states for its operator,
//                                  running = momentum * running + (1 - momentum) * batch
//                                  (dragon/python/core/ops/normalization_ops.py:36-39),
//                                  with the biased batch variance of batch_norm_op.cc:60-63;
//                                  no reference test asserts the running tensors
//   batch_norm_expectation         PARITY UNPINNED by any reference test (SyncBN is
//                                  never run multi-rank); checked against E[x], E[x^2]
//
// Build: make -C oracle   (g++ -O2 -std=c++14 -mavx -mavx2 -mfma -fopenmp, no
// fast-math: the flag set of the reference's cmake/MiscCheck.cmake:33-58)

#include <algorithm>
#include <array>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

// ---------------------------------------------------------------------------
// 16-bit float storage types and software conversions.
// Follows dragon/core/types.h:36-42 and dragon/utils/conversions.h:42-149.
// ---------------------------------------------------------------------------

struct half_t {
  unsigned short x;
};
struct bhalf_t {
  unsigned short x;
};

inline unsigned short float_to_half_bits(float val) {
  // dragon/utils/conversions.h:47-78 : round-to-nearest-even with the
  // overflow case expressed as "largest finite, then round up".
  unsigned int x, remainder, result;
  std::memcpy(&x, &val, sizeof(val));
  unsigned int u = (x & 0x7fffffffU);
  unsigned int sign = ((x >> 16U) & 0x8000U);
  if (u >= 0x7f800000U) {
    remainder = 0U;
    result = ((u == 0x7f800000U) ? (sign | 0x7c00U) : 0x7fffU);
  } else if (u > 0x477fefffU) {
    remainder = 0x80000000U;
    result = (sign | 0x7bffU);
  } else if (u >= 0x38800000U) {
    remainder = u << 19U;
    u -= 0x38000000U;
    result = (sign | (u >> 13U));
  } else if (u < 0x33000001U) {
    remainder = u;
    result = sign;
  } else {
    const unsigned int exponent = u >> 23U;
    const unsigned int shift = 0x7eU - exponent;
    unsigned int mantissa = (u & 0x7fffffU);
    mantissa |= 0x800000U;
    remainder = mantissa << (32U - shift);
    result = (sign | (mantissa >> shift));
    result &= 0x0000FFFFU;
  }
  unsigned short r = static_cast<unsigned short>(result);
  if ((remainder > 0x80000000U) ||
      ((remainder == 0x80000000U) && ((r & 0x1U) != 0U))) {
    r++;
  }
  return r;
}

inline float half_bits_to_float(unsigned short h) {
  // dragon/utils/conversions.h:113-141
  unsigned int sign = ((static_cast<unsigned int>(h) >> 15U) & 1U);
  unsigned int exponent = ((static_cast<unsigned int>(h) >> 10U) & 0x1fU);
  unsigned int mantissa = ((static_cast<unsigned int>(h) & 0x3ffU) << 13U);
  if (exponent == 0x1fU) {
    sign = ((mantissa != 0U) ? (sign >> 1U) : sign);
    mantissa = ((mantissa != 0U) ? 0x7fffffU : 0U);
    exponent = 0xffU;
  } else if (exponent == 0U) {
    if (mantissa != 0U) {
      unsigned int msb;
      exponent = 0x71U;
      do {
        msb = (mantissa & 0x400000U);
        mantissa <<= 1U;
        --exponent;
      } while (msb == 0U);
      mantissa &= 0x7fffffU;
    }
  } else {
    exponent += 0x70U;
  }
  const unsigned int u = ((sign << 31U) | (exponent << 23U) | mantissa);
  float ret;
  std::memcpy(&ret, &u, sizeof(u));
  return ret;
}

inline unsigned short float_to_bhalf_bits(float val) {
  // dragon/utils/conversions.h:90-106 : NaN -> 0x7fff, else RNE on bit 16.
  unsigned int x, remainder;
  unsigned short r;
  std::memcpy(&x, &val, sizeof(val));
  if ((x & 0x7fffffffU) > 0x7f800000U) {
    remainder = 0U;
    r = static_cast<unsigned short>(0x7fffU);
  } else {
    remainder = x << 16U;
    r = static_cast<unsigned short>(x >> 16U);
  }
  if ((remainder > 0x80000000U) ||
      ((remainder == 0x80000000U) && ((r & 0x1U) != 0U))) {
    r++;
  }
  return r;
}

inline float bhalf_bits_to_float(unsigned short h) {
  // dragon/utils/conversions.h:143-149
  const unsigned int u = static_cast<unsigned int>(h) << 16;
  float ret;
  std::memcpy(&ret, &u, sizeof(ret));
  return ret;
}

// convert::To<Dst>(src) restricted to the pairs the hot path uses.
template <typename D, typename S>
struct Cvt {
  static D to(S v) { return static_cast<D>(v); }
};
template <>
struct Cvt<float, half_t> {
  static float to(half_t v) { return half_bits_to_float(v.x); }
};
template <>
struct Cvt<float, bhalf_t> {
  static float to(bhalf_t v) { return bhalf_bits_to_float(v.x); }
};
template <>
struct Cvt<half_t, float> {
  static half_t to(float v) { return half_t{float_to_half_bits(v)}; }
};
template <>
struct Cvt<bhalf_t, float> {
  static bhalf_t to(float v) { return bhalf_t{float_to_bhalf_bits(v)}; }
};
template <typename D, typename S>
inline D To(S v) {
  return Cvt<D, S>::to(v);
}

// math::utils::IncreaseIndexInDims, dragon/utils/math/utils.h:254-264 :
// odometer increment, last dimension fastest. It fixes the accumulation order
// of every index-walking kernel below.
inline void increase_index(int num_dims, const int* dims, int* index) {
  for (int i = num_dims - 1; i >= 0; --i) {
    ++index[i];
    if (index[i] >= dims[i]) {
      index[i] -= dims[i];
    } else {
      break;
    }
  }
}

// ---------------------------------------------------------------------------
// LayerNorm forward. dragon/kernels/normalization/cpu/layer_norm_kernel.cc:10-39
// ---------------------------------------------------------------------------
template <typename T, typename AccT>
void layer_norm(
    const int N, const int C, const AccT epsilon, const T* x,
    const AccT* gamma, const AccT* beta, AccT* mu, AccT* rsig, T* y) {
  const AccT scale = AccT(1) / AccT(C);
  for (int i = 0; i < N; ++i) {
    const int64_t offset = int64_t(i) * C;
    AccT m_val = AccT(0), v_val = AccT(0);
    for (int j = 0; j < C; ++j) {
      const AccT val = To<AccT>(x[offset + j]);
      m_val += val;
      v_val += val * val;
    }
    mu[i] = m_val = m_val * scale;
    v_val = std::sqrt(v_val * scale - m_val * m_val + epsilon);
    rsig[i] = v_val = AccT(1) / v_val;
    for (int j = 0; j < C; ++j) {
      AccT val = To<AccT>(x[offset + j]);
      val = (val - m_val) * v_val;
      y[offset + j] = To<T>(val * gamma[j] + beta[j]);
    }
  }
}

// ---------------------------------------------------------------------------
// Moments. dragon/kernels/math/cpu/moments_kernel.cc:10-155 and the axis
// utilities of dragon/utils/math/reduce.h:96-198.
// ---------------------------------------------------------------------------
template <typename T, typename AccT>
void rowwise_moments(
    const int64_t rows, const int64_t cols, const T* x, AccT* mean, AccT* var) {
  // moments_kernel.cc:10-31 : reduce over the LEADING axis.
  const AccT scale = AccT(1) / AccT(rows);
  for (int64_t i = 0; i < cols; ++i) {
    AccT m_val = AccT(0), v_val = AccT(0);
    for (int64_t j = 0; j < rows; ++j) {
      const AccT val = To<AccT>(x[j * cols + i]);
      m_val += val;
      v_val += val * val;
    }
    m_val = m_val * scale;
    mean[i] = m_val;
    var[i] = v_val * scale - m_val * m_val;
  }
}

template <typename T, typename AccT>
void colwise_moments(
    const int64_t rows, const int64_t cols, const T* x, AccT* mean, AccT* var) {
  // moments_kernel.cc:33-54 : reduce over the TRAILING axis.
  const AccT scale = AccT(1) / AccT(cols);
  for (int64_t i = 0; i < rows; ++i) {
    const int64_t offset = i * cols;
    AccT m_val = AccT(0), v_val = AccT(0);
    for (int64_t j = 0; j < cols; ++j) {
      const AccT val = To<AccT>(x[offset + j]);
      m_val += val;
      v_val += val * val;
    }
    m_val = m_val * scale;
    mean[i] = m_val;
    var[i] = v_val * scale - m_val * m_val;
  }
}

template <typename T, typename AccT>
void generic_moments(
    const int64_t rows, const int64_t cols, const int num_dims,
    const int64_t* x_dims, const int64_t* x_strides, const T* x, AccT* mean,
    AccT* var) {
  // moments_kernel.cc:56-84 : transposed-strided gather, kept axes outermost.
  const AccT scale = AccT(1) / AccT(cols);
  for (int64_t i = 0; i < rows; ++i) {
    const int64_t offset = i * cols;
    AccT m_val = AccT(0), v_val = AccT(0);
    for (int64_t j = 0; j < cols; ++j) {
      int64_t xi = 0, c = offset + j;
      for (int d = num_dims - 1; d >= 0; --d) {
        const int64_t r = c % x_dims[d];
        c = c / x_dims[d];
        xi += r * x_strides[d];
      }
      const AccT val = To<AccT>(x[xi]);
      m_val += val;
      v_val += val * val;
    }
    m_val = m_val * scale;
    mean[i] = m_val;
    var[i] = v_val * scale - m_val * m_val;
  }
}

// reduce.h:160-198
void collapse_reduce_axes(
    const int num_dims, const int64_t* dims, const int num_axes,
    const int64_t* axes, std::vector<int64_t>& new_dims,
    std::vector<int64_t>& new_axes) {
  new_dims.clear();
  new_axes.clear();
  int64_t new_dim = 0, new_axis = 0;
  std::vector<int64_t> reduce_dims(dims, dims + num_dims);
  for (int i = 0; i < num_axes; ++i) reduce_dims[axes[i]] = -1;
  for (int i = 0; i < num_dims; ++i) {
    if (dims[i] == 1) continue;
    if (reduce_dims[i] == -1) {
      if (new_axes.empty() || new_axis != new_axes.back()) {
        if (new_dim > 0) new_dims.push_back(new_dim);
        new_dim = dims[i];
        new_axes.push_back(new_axis);
      } else {
        new_dim *= dims[i];
      }
    } else {
      if (!new_axes.empty() && new_axis == new_axes.back()) {
        if (new_dim > 0) new_dims.push_back(new_dim);
        new_dim = 0;
        new_axis += 1;
      }
      if (new_dim == 0) {
        new_dim = dims[i];
        new_axis += 1;
      } else {
        new_dim *= dims[i];
      }
    }
  }
  if (new_dim > 0) new_dims.push_back(new_dim);
}

// reduce.h:96-116
bool is_rowwise_reduce(
    const int num_dims, const int64_t* X_dims, const int64_t* Y_dims,
    int64_t* rows, int64_t* cols) {
  *rows = *cols = 1;
  int pivot = 0;
  for (; pivot < num_dims && Y_dims[pivot] == 1; ++pivot) *rows *= X_dims[pivot];
  for (int i = pivot; i < num_dims; ++i) {
    if (X_dims[i] != Y_dims[i]) return false;
    *cols *= X_dims[i];
  }
  return true;
}

// reduce.h:118-138
bool is_colwise_reduce(
    const int num_dims, const int64_t* X_dims, const int64_t* Y_dims,
    int64_t* rows, int64_t* cols) {
  *cols = *rows = 1;
  int pivot = num_dims - 1;
  for (; pivot >= 0 && Y_dims[pivot] == 1; --pivot) *cols *= X_dims[pivot];
  for (int i = pivot; i >= 0; --i) {
    if (X_dims[i] != Y_dims[i]) return false;
    *rows *= X_dims[i];
  }
  return true;
}

// reduce.h:140-158 (TransposeAxesForReduce) and the stride computation of
// ComputeTransposeStrides: kept axes first, reduced axes last, each keeping
// its source stride.
void transposed_reduce_plan(
    const std::vector<int64_t>& dims, const std::vector<int64_t>& axes,
    int64_t* rows, int64_t* cols, std::vector<int64_t>& t_dims,
    std::vector<int64_t>& t_strides) {
  const int num_dims = int(dims.size()), num_axes = int(axes.size());
  std::vector<int64_t> t_axes(num_dims);
  t_dims.assign(num_dims, 0);
  t_strides.assign(num_dims, 0);
  const int d = num_dims - num_axes;
  std::copy_n(axes.begin(), num_axes, t_axes.begin() + d);
  std::sort(t_axes.begin() + d, t_axes.end());
  int p = 0, q = d;
  for (int i = 0; i < num_dims; ++i) {
    if (q < num_dims && i == t_axes[q]) {
      ++q;
    } else {
      t_axes[p++] = i;
    }
  }
  std::vector<int64_t> strides(num_dims);
  int64_t acc = 1;
  for (int i = num_dims - 1; i >= 0; --i) {
    strides[i] = acc;
    acc *= dims[i];
  }
  *rows = *cols = 1;
  for (int i = 0; i < d; ++i) *rows *= dims[t_axes[i]];
  for (int i = d; i < num_dims; ++i) *cols *= dims[t_axes[i]];
  for (int i = 0; i < num_dims; ++i) {
    t_dims[i] = dims[t_axes[i]];
    t_strides[i] = strides[t_axes[i]];
  }
}

template <typename T, typename AccT>
void moments(
    const int num_dims_in, const int64_t* dims_in, const int num_axes_in,
    const int64_t* axes_in, const T* x, AccT* mean, AccT* var) {
  // moments_kernel.cc:160-183 then :86-135
  std::vector<int64_t> dims, axes;
  collapse_reduce_axes(num_dims_in, dims_in, num_axes_in, axes_in, dims, axes);
  const int num_dims = int(dims.size()), num_axes = int(axes.size());
  int64_t rows, cols;
  std::vector<int64_t> out_dims(dims);
  for (int i = 0; i < num_axes; ++i) out_dims[axes[i]] = 1;
  if (is_rowwise_reduce(num_dims, dims.data(), out_dims.data(), &rows, &cols)) {
    return rowwise_moments(rows, cols, x, mean, var);
  }
  if (is_colwise_reduce(num_dims, dims.data(), out_dims.data(), &rows, &cols)) {
    return colwise_moments(rows, cols, x, mean, var);
  }
  std::vector<int64_t> t_dims, t_strides;
  transposed_reduce_plan(dims, axes, &rows, &cols, t_dims, t_strides);
  generic_moments(
      rows, cols, num_dims, t_dims.data(), t_strides.data(), x, mean, var);
}

// ---------------------------------------------------------------------------
// math::ReduceSum / ReduceSumSqr / ReduceL1, dragon/utils/math/cpu/reduce.cc.
// The global, rowwise ("leading axes") and colwise ("trailing axes") cases are
// Eigen reductions there (:12-61), restated as sequential sums in T; the
// generic case is the strided walk of :62-88 in AccT = T. y = T(sum) * T(scale)
// where scale != 1 (:17,:36,:54), y = T(sum * scale) in the generic case (:86).
// kKind: 0 identity, 1 square, 2 absolute value.
// ---------------------------------------------------------------------------
template <typename T, int kKind>
inline T reduce_term(T v) {
  return kKind == 0 ? v : (kKind == 1 ? v * v : std::abs(v));
}

template <typename T, int kKind>
void reduce_sum(
    const int num_dims_in, const int64_t* dims_in, const int num_axes_in,
    const int64_t* axes_in, const float scale, const T* x, T* y) {
  // :188-212 (CollapseReduceAxes) then the dispatcher :90-160
  std::vector<int64_t> dims, axes;
  collapse_reduce_axes(num_dims_in, dims_in, num_axes_in, axes_in, dims, axes);
  const int num_dims = int(dims.size()), num_axes = int(axes.size());
  if (num_dims == num_axes) {
    int64_t n = 1;
    for (int64_t d : dims) n *= d;
    T acc = T(0);
    for (int64_t i = 0; i < n; ++i) acc += reduce_term<T, kKind>(x[i]);
    y[0] = acc;
    if (scale != 1.f) y[0] *= T(scale);
    return;
  }
  int64_t rows, cols;
  std::vector<int64_t> out_dims(dims);
  for (int i = 0; i < num_axes; ++i) out_dims[axes[i]] = 1;
  if (is_rowwise_reduce(num_dims, dims.data(), out_dims.data(), &rows, &cols)) {
    for (int64_t i = 0; i < cols; ++i) {
      T acc = T(0);
      for (int64_t j = 0; j < rows; ++j) acc += reduce_term<T, kKind>(x[j * cols + i]);
      y[i] = scale != 1.f ? acc * T(scale) : acc;
    }
    return;
  }
  if (is_colwise_reduce(num_dims, dims.data(), out_dims.data(), &rows, &cols)) {
    for (int64_t i = 0; i < rows; ++i) {
      T acc = T(0);
      for (int64_t j = 0; j < cols; ++j) acc += reduce_term<T, kKind>(x[i * cols + j]);
      y[i] = scale != 1.f ? acc * T(scale) : acc;
    }
    return;
  }
  std::vector<int64_t> t_dims, t_strides;
  transposed_reduce_plan(dims, axes, &rows, &cols, t_dims, t_strides);
  for (int64_t i = 0; i < rows; ++i) {
    T val = T(0);
    for (int64_t j = 0; j < cols; ++j) {
      int64_t xi = 0, c = i * cols + j;
      for (int d = num_dims - 1; d >= 0; --d) {
        const int64_t r = c % t_dims[d];
        c = c / t_dims[d];
        xi += r * t_strides[d];
      }
      val += reduce_term<T, kKind>(x[xi]);
    }
    y[i] = val * T(scale);
  }
}

// ---------------------------------------------------------------------------
// math::InvStd, dragon/utils/math/cpu/elementwise.cc:187-201 :
// Eigen (x + T(eps)).rsqrt(), restated as 1/sqrt in T arithmetic.
// ---------------------------------------------------------------------------
template <typename T>
void inv_std(const int64_t N, const float eps, const T* x, T* y) {
  const T e = T(eps);
  for (int64_t i = 0; i < N; ++i) y[i] = T(1) / std::sqrt(x[i] + e);
}

// ---------------------------------------------------------------------------
// math::Axpby, dragon/utils/math/cpu/blas.cc:87-136 : Scale(y = beta*y) then
// Axpy(y += alpha*x), alpha/beta narrowed to T first. The product alpha*x is
// rounded before the add (the volatile stops the compiler fusing it), as two
// separate Eigen array statements do.
// ---------------------------------------------------------------------------
template <typename T>
void axpby(const int64_t N, const float alpha, const T* x, const float beta, T* y) {
  const T a = T(alpha), b = T(beta);
  for (int64_t i = 0; i < N; ++i) y[i] = y[i] * b;
  for (int64_t i = 0; i < N; ++i) {
    volatile T prod = x[i] * a;
    y[i] = y[i] + prod;
  }
}

// ---------------------------------------------------------------------------
// GroupNorm forward. dragon/kernels/normalization/cpu/group_norm_kernel.cc:11-31
// dims = {N,G,D,S} for NCHW and {N,S,G,D} for NHWC (:100-107).
// ---------------------------------------------------------------------------
template <typename T, typename AccT, bool kNCHW>
void group_norm_impl(
    const std::array<int, 4>& dims, const T* x, const AccT* mu,
    const AccT* rsig, const AccT* gamma, const AccT* beta, T* y) {
  const int kGDim = kNCHW ? 1 : 2;
  const int kDDim = kNCHW ? 2 : 3;
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2] * dims[3];
  std::array<int, 4> index = {0, 0, 0, 0};
  for (int64_t i = 0; i < total; ++i) {
    const int ng = index[0] * dims[kGDim] + index[kGDim];
    const int c = index[kGDim] * dims[kDDim] + index[kDDim];
    AccT val = (To<AccT>(x[i]) - mu[ng]) * rsig[ng];
    y[i] = To<T>(val * gamma[c] + beta[c]);
    increase_index(4, dims.data(), index.data());
  }
}

// group_norm_kernel.cc:33-53
template <typename T, typename AccT, bool kNCHW>
void group_norm_internal_grad(
    const std::array<int, 4>& dims, const T* x, const AccT* gamma, const T* dy,
    AccT* ds, AccT* db) {
  const int kGDim = kNCHW ? 1 : 2;
  const int kDDim = kNCHW ? 2 : 3;
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2] * dims[3];
  std::array<int, 4> index = {0, 0, 0, 0};
  for (int64_t i = 0; i < total; ++i) {
    const int ng = index[0] * dims[kGDim] + index[kGDim];
    const int c = index[kGDim] * dims[kDDim] + index[kDDim];
    ds[ng] += gamma[c] * dy[i] * x[i];
    db[ng] += gamma[c] * dy[i];
    increase_index(4, dims.data(), index.data());
  }
}

// group_norm_kernel.cc:55-84
template <typename T, typename AccT, bool kNCHW>
void group_norm_grad_impl(
    const std::array<int, 4>& dims, const T* x, const AccT* mu,
    const AccT* rsig, const AccT* gamma, const AccT* ds, const AccT* db,
    const T* dy, AccT* dgamma, AccT* dbeta, T* dx) {
  const int kGDim = kNCHW ? 1 : 2;
  const int kDDim = kNCHW ? 2 : 3;
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2] * dims[3];
  const int S = kNCHW ? dims[3] : dims[1];
  const AccT denom = AccT(1) / static_cast<AccT>(dims[kDDim] * S);
  std::array<int, 4> index = {0, 0, 0, 0};
  for (int64_t i = 0; i < total; ++i) {
    const int ng = index[0] * dims[kGDim] + index[kGDim];
    const int c = index[kGDim] * dims[kDDim] + index[kDDim];
    const AccT r = rsig[ng];
    const AccT u = (db[ng] * mu[ng] - ds[ng]) * (x[i] - mu[ng]) * (r * r * r);
    const AccT v = db[ng] * rsig[ng];
    dx[i] = gamma[c] * dy[i] * rsig[ng] + (u - v) * denom;
    dgamma[c] += dy[i] * (x[i] - mu[ng]) * rsig[ng];
    dbeta[c] += dy[i];
    increase_index(4, dims.data(), index.data());
  }
}

// ---------------------------------------------------------------------------
// BatchNorm family. dragon/kernels/normalization/cpu/batch_norm_kernel.cc
// dims = {N,C,S} for NCHW and {N,S,C} for NHWC.
// ---------------------------------------------------------------------------

// :11-33
template <typename T, typename AccT, bool kNCHW>
void batch_norm_expectation_impl(
    const std::array<int, 3>& dims, const AccT normalizer, const T* x,
    AccT* ex, AccT* ex2) {
  const int kCDim = kNCHW ? 1 : 2;
  const int C = dims[kCDim];
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2];
  std::array<int, 3> index = {0, 0, 0};
  for (int64_t xi = 0; xi < total; ++xi) {
    const T val = x[xi];
    const int i = index[kCDim];
    ex[i] += val;
    ex2[i] += val * val;
    increase_index(3, dims.data(), index.data());
  }
  for (int i = 0; i < C; ++i) {
    ex[i] /= normalizer;
    ex2[i] /= normalizer;
  }
}

// :35-50 (Eigen array expression restated element-wise)
template <typename T>
void batch_norm_fused_params(
    const int C, const T* mu, const T* rsig, const T* gamma, const T* beta,
    T* scale, T* bias) {
  for (int i = 0; i < C; ++i) scale[i] = gamma[i] * rsig[i];
  for (int i = 0; i < C; ++i) {
    volatile T prod = scale[i] * mu[i];
    bias[i] = beta[i] - prod;
  }
}

// :52-85 (both layouts evaluate x*scale[c] + bias[c] per element)
template <typename T, typename AccT, bool kNCHW>
void batch_norm_affine(
    const int N, const int C, const int S, const T* x, const AccT* scale,
    const AccT* bias, T* y) {
  if (kNCHW) {
    for (int i = 0; i < N; ++i) {
      for (int j = 0; j < C; ++j) {
        for (int k = 0; k < S; ++k) {
          volatile T prod = x[k] * scale[j];
          y[k] = prod + bias[j];
        }
        x += S;
        y += S;
      }
    }
  } else {
    const int64_t NS = int64_t(N) * S;
    for (int64_t i = 0; i < NS; ++i) {
      for (int j = 0; j < C; ++j) {
        volatile T prod = x[i * C + j] * scale[j];
        y[i * C + j] = prod + bias[j];
      }
    }
  }
}

// :87-105
template <typename T, typename AccT, bool kNCHW>
void batch_norm_wgrad_impl(
    const std::array<int, 3>& dims, const T* x, const AccT* mu,
    const AccT* rsig, const T* dy, AccT* dgamma, AccT* dbeta) {
  const int kCDim = kNCHW ? 1 : 2;
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2];
  std::array<int, 3> index = {0, 0, 0};
  for (int64_t i = 0; i < total; ++i) {
    const int pi = index[kCDim];
    dgamma[pi] += dy[i] * (x[i] - mu[pi]) * rsig[pi];
    dbeta[pi] += dy[i];
    increase_index(3, dims.data(), index.data());
  }
}

// :107-129
template <typename T, typename AccT, bool kNCHW>
void batch_norm_training_grad_impl(
    const std::array<int, 3>& dims, const AccT normalizer, const T* x,
    const AccT* mu, const AccT* rsig, const AccT* gamma, const AccT* dgamma,
    const AccT* dbeta, const T* dy, T* dx) {
  const int kCDim = kNCHW ? 1 : 2;
  const int64_t total = int64_t(dims[0]) * dims[1] * dims[2];
  std::array<int, 3> index = {0, 0, 0};
  for (int64_t i = 0; i < total; ++i) {
    const int pi = index[kCDim];
    const AccT x_norm = (x[i] - mu[pi]) * rsig[pi];
    dx[i] = gamma[pi] * rsig[pi] *
        (dy[i] - (x_norm * dgamma[pi] + dbeta[pi]) / normalizer);
    increase_index(3, dims.data(), index.data());
  }
}

// :131-155 : dx = dy * (gamma * rsig)[c]
template <typename T, typename AccT, bool kNCHW>
void batch_norm_inference_grad_impl(
    const int N, const int C, const int S, const AccT* rsig, const AccT* gamma,
    const T* dy, T* dx) {
  std::vector<AccT> gr(C);
  for (int j = 0; j < C; ++j) gr[j] = gamma[j] * rsig[j];
  if (kNCHW) {
    for (int i = 0; i < N; ++i)
      for (int j = 0; j < C; ++j)
        for (int k = 0; k < S; ++k) {
          const int64_t o = (int64_t(i) * C + j) * S + k;
          dx[o] = dy[o] * gr[j];
        }
  } else {
    const int64_t NS = int64_t(N) * S;
    for (int64_t i = 0; i < NS; ++i)
      for (int j = 0; j < C; ++j) dx[i * C + j] = dy[i * C + j] * gr[j];
  }
}

// ---------------------------------------------------------------------------
// Softmax family. dragon/kernels/activation/cpu/softmax_kernel.cc:10-108.
// The reference evaluates Eigen array expressions; each is restated as the
// scalar loop with the same data flow (max, exp, sequential sum, divide).
// ---------------------------------------------------------------------------
template <typename T>
void softmax(const int N, const int S, const int C, const T* x, T* y) {
  // :11-31
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T m = x[base];
      for (int k = 1; k < C; ++k) m = std::max(m, x[base + int64_t(k) * S]);
      T sum = T(0);
      for (int k = 0; k < C; ++k) {
        const T e = std::exp(x[base + int64_t(k) * S] - m);
        y[base + int64_t(k) * S] = e;
        sum += e;
      }
      for (int k = 0; k < C; ++k) y[base + int64_t(k) * S] /= sum;
    }
  }
}

template <typename T>
void log_softmax(const int N, const int S, const int C, const T* x, T* y) {
  // :33-52
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T m = x[base];
      for (int k = 1; k < C; ++k) m = std::max(m, x[base + int64_t(k) * S]);
      T sum = T(0);
      for (int k = 0; k < C; ++k) {
        const T v = x[base + int64_t(k) * S] - m;
        y[base + int64_t(k) * S] = v;
        sum += std::exp(v);
      }
      const T l = std::log(sum);
      for (int k = 0; k < C; ++k) y[base + int64_t(k) * S] -= l;
    }
  }
}

template <typename T>
void softmax_grad(
    const int N, const int S, const int C, const T* dy, const T* y, T* dx) {
  // :54-82 : dx = (dy - sum(dy*y)) * y
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T sum = T(0);
      for (int k = 0; k < C; ++k)
        sum += dy[base + int64_t(k) * S] * y[base + int64_t(k) * S];
      for (int k = 0; k < C; ++k) {
        const int64_t o = base + int64_t(k) * S;
        dx[o] = (dy[o] - sum) * y[o];
      }
    }
  }
}

template <typename T>
void log_softmax_grad(
    const int N, const int S, const int C, const T* dy, const T* y, T* dx) {
  // :84-108 : dx = dy - exp(y) * sum(dy)
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T sum = T(0);
      for (int k = 0; k < C; ++k) sum += dy[base + int64_t(k) * S];
      for (int k = 0; k < C; ++k) {
        const int64_t o = base + int64_t(k) * S;
        dx[o] = dy[o] - std::exp(y[o]) * sum;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// L1Norm / L2Norm and gradients over [N, C, S], reduction along C.
// dragon/kernels/normalization/cpu/lp_norm_kernel.cc:10-101. The reference
// evaluates Eigen expressions (lpNorm<1>, squaredNorm, dot, array().sign());
// each is restated as a sequential scalar loop with the same data flow: the
// norm is narrowed to float, divided by the normalizer, clamped from below by
// epsilon and narrowed to T before the element-wise division.
// ---------------------------------------------------------------------------
template <typename T>
inline T sign_of(T v) {
  return T((T(0) < v) - (v < T(0)));
}

template <typename T, int kP>
void lp_norm(const int N, const int S, const int C, const float normalizer,
             const float epsilon, const T* x, T* y) {
  // :10-49
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T acc = T(0);
      for (int k = 0; k < C; ++k) {
        const T v = x[base + int64_t(k) * S];
        acc += kP == 1 ? std::abs(v) : v * v;
      }
      const float norm = kP == 1 ? float(acc) / normalizer
                                 : std::sqrt(float(acc) / normalizer);
      const T div = T(std::max(norm, epsilon));
      for (int k = 0; k < C; ++k) {
        const int64_t o = base + int64_t(k) * S;
        y[o] = x[o] / div;
      }
    }
  }
}

template <typename T, int kP>
void lp_norm_grad(const int N, const int S, const int C, const float normalizer,
                  const float eps, const T* dy, const T* x, T* dx) {
  // :51-101 : dx = dy / norm - sign(x) / (norm^2 / sum)   (p = 1)
  //           dx = dy / norm -      x  / (norm^3 / sum)   (p = 2)
  // with sum = dot(dy, x) / normalizer.
  for (int i = 0; i < N; ++i) {
    for (int j = 0; j < S; ++j) {
      const int64_t base = int64_t(i) * C * S + j;
      T acc = T(0), dot = T(0);
      for (int k = 0; k < C; ++k) {
        const int64_t o = base + int64_t(k) * S;
        acc += kP == 1 ? std::abs(x[o]) : x[o] * x[o];
        dot += dy[o] * x[o];
      }
      const float norm =
          std::max(kP == 1 ? float(acc) / normalizer
                           : std::sqrt(float(acc) / normalizer), eps);
      const float sum = float(dot) / normalizer;
      const float powed = kP == 1 ? norm * norm : std::pow(norm, 3.f);
      const T a = T(norm), b = T(powed / sum);
      for (int k = 0; k < C; ++k) {
        const int64_t o = base + int64_t(k) * S;
        dx[o] = dy[o] / a - (kP == 1 ? sign_of(x[o]) : x[o]) / b;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Softmax cross-entropy loss kernels.
// dragon/kernels/loss/cpu/cross_entropy_kernel.cc:10-42,80-108 and
// dragon/kernels/loss/cpu/generic_loss_kernel.cc:10-60. math::Sum inside
// ReduceLoss is the global Eigen sum followed by `*= T(scale)` (reduce.cc:12-19),
// restated as a sequential sum.
// ---------------------------------------------------------------------------
template <typename T>
void cross_entropy_dense(const int64_t N, const T* input, const T* target, T* loss) {
  // :10-15
  for (int64_t i = 0; i < N; ++i) {
    loss[i] = -target[i] * std::log(std::max(input[i], T(FLT_MIN)));
  }
}

template <typename InputT, typename TargetT>
void cross_entropy_sparse(
    const int N, const int S, const int C, const int ignore_index,
    const InputT* input, const TargetT* target, InputT* loss, InputT* mask) {
  // :17-42 : positions are walked n-major, s-minor.
  for (int n = 0; n < N; ++n) {
    for (int sidx = 0; sidx < S; ++sidx) {
      const int64_t i = int64_t(n) * S + sidx;
      const int tgt = int(target[i]);
      if (tgt == ignore_index) {
        loss[i] = mask[i] = InputT(0);
      } else {
        const int64_t j = (int64_t(n) * C + tgt) * S + sidx;
        loss[i] = -std::log(std::max(input[j], InputT(FLT_MIN)));
        mask[i] = InputT(1);
      }
    }
  }
}

template <typename InputT, typename TargetT>
void softmax_cross_entropy_grad(
    const int N, const int S, const int C, const int ignore_index,
    const TargetT* target, InputT* grad, InputT* mask) {
  // :80-108
  for (int n = 0; n < N; ++n) {
    for (int sidx = 0; sidx < S; ++sidx) {
      const int64_t i = int64_t(n) * S + sidx;
      const int tgt = int(target[i]);
      if (tgt == ignore_index) {
        InputT* g = grad + int64_t(n) * C * S + sidx;
        for (int k = 0; k < C; ++k) {
          *g = InputT(0);
          g += S;
        }
        mask[i] = InputT(0);
      } else {
        grad[(int64_t(n) * C + tgt) * S + sidx] -= InputT(1);
        mask[i] = InputT(1);
      }
    }
  }
}

template <typename T>
T scaled_sum(const int64_t N, const float scale, const T* x) {
  T acc = T(0);
  for (int64_t i = 0; i < N; ++i) acc += x[i];
  if (scale != 1.f) acc *= T(scale);
  return acc;
}

template <typename T>
void reduce_loss(const int64_t N, const int64_t num_masks, const float normalizer,
                 const T* x, const T* mask, T* y) {
  // generic_loss_kernel.cc:31-44
  const float inv_scale = num_masks > 0 && normalizer < 0.f
      ? float(scaled_sum(num_masks, 1.f, mask)) : normalizer;
  y[0] = scaled_sum(N, 1.f / std::max(inv_scale, 1.f), x);
}

template <typename T>
void reduce_loss_grad(const int64_t N, const int64_t num_masks, const float normalizer,
                      const T* dl, const T* mask, T* dx) {
  // generic_loss_kernel.cc:46-60 ; math::Scale is x * T(scale) (blas.cc:87-97)
  const float inv_scale = num_masks > 0 && normalizer < 0.f
      ? float(scaled_sum(num_masks, 1.f, mask)) : normalizer;
  const float scale = float(dl[0]) / std::max(inv_scale, 0.5f);
  for (int64_t i = 0; i < N; ++i) dx[i] = dx[i] * T(scale);
}

template <typename T>
void broadcast_loss_grad(const int N, const int S, const int C, const T* dl, T* dx) {
  // generic_loss_kernel.cc:10-25
  for (int n = 0; n < N; ++n)
    for (int c = 0; c < C; ++c)
      for (int sidx = 0; sidx < S; ++sidx) {
        const int64_t i = (int64_t(n) * C + c) * S + sidx;
        dx[i] = dx[i] * dl[int64_t(n) * S + sidx];
      }
}

template <typename I, typename Tg>
void sparse_ce_erased(int N, int S, int C, int ig, const void* in, const void* tg, void* loss, void* mask) {
  cross_entropy_sparse(N, S, C, ig, (const I*)in, (const Tg*)tg, (I*)loss, (I*)mask);
}
template <typename I, typename Tg>
void sce_grad_erased(int N, int S, int C, int ig, const void* tg, void* dx, void* mask) {
  softmax_cross_entropy_grad(N, S, C, ig, (const Tg*)tg, (I*)dx, (I*)mask);
}

enum { kF16 = 0, kBF16 = 1, kF32 = 2, kF64 = 3 };
enum { kNCHWLayout = 0, kNHWCLayout = 1 };
enum { kOk = 0, kBadArg = -1, kUnsupportedDtype = -2 };

} // namespace

// ===========================================================================
// C entry points. dtype: 0 f16, 1 bf16, 2 f32, 3 f64. layout: 0 NCHW, 1 NHWC.
// AccT is float for f16/bf16/f32 and double for f64
// (dragon/utils/math/types.h:69-152). A dtype the reference's CPU launcher
// rejects with CPU_UNSUPPORTED_DTYPE returns -2.
// ===========================================================================
extern "C" {

// Bulk conversions, used by tests to produce and decode 16-bit buffers with
// exactly the reference's rounding (dragon/utils/conversions.h:42-149).
void ref_float_to_half(int64_t n, const float* x, uint16_t* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = float_to_half_bits(x[i]);
}
void ref_half_to_float(int64_t n, const uint16_t* x, float* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = half_bits_to_float(x[i]);
}
void ref_float_to_bfloat16(int64_t n, const float* x, uint16_t* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = float_to_bhalf_bits(x[i]);
}
void ref_bfloat16_to_float(int64_t n, const uint16_t* x, float* y) {
  for (int64_t i = 0; i < n; ++i) y[i] = bhalf_bits_to_float(x[i]);
}

// kernels::LayerNorm launcher, layer_norm_kernel.cc:43-62 (all four dtypes).
int ref_layer_norm(
    int dtype, int64_t N, int64_t C, float eps, const void* x,
    const void* gamma, const void* beta, void* mu, void* rsig, void* y) {
  switch (dtype) {
    case kF16:
      layer_norm<half_t, float>(
          int(N), int(C), eps, (const half_t*)x, (const float*)gamma,
          (const float*)beta, (float*)mu, (float*)rsig, (half_t*)y);
      return kOk;
    case kBF16:
      layer_norm<bhalf_t, float>(
          int(N), int(C), eps, (const bhalf_t*)x, (const float*)gamma,
          (const float*)beta, (float*)mu, (float*)rsig, (bhalf_t*)y);
      return kOk;
    case kF32:
      layer_norm<float, float>(
          int(N), int(C), eps, (const float*)x, (const float*)gamma,
          (const float*)beta, (float*)mu, (float*)rsig, (float*)y);
      return kOk;
    case kF64:
      layer_norm<double, double>(
          int(N), int(C), double(eps), (const double*)x, (const double*)gamma,
          (const double*)beta, (double*)mu, (double*)rsig, (double*)y);
      return kOk;
  }
  return kUnsupportedDtype;
}

// kernels::Moments launcher, moments_kernel.cc:159-189 (all four dtypes).
int ref_moments(
    int dtype, int num_dims, const int64_t* dims, int num_axes,
    const int64_t* axes, const void* x, void* mean, void* var) {
  switch (dtype) {
    case kF16:
      moments<half_t, float>(num_dims, dims, num_axes, axes, (const half_t*)x,
                             (float*)mean, (float*)var);
      return kOk;
    case kBF16:
      moments<bhalf_t, float>(num_dims, dims, num_axes, axes,
                              (const bhalf_t*)x, (float*)mean, (float*)var);
      return kOk;
    case kF32:
      moments<float, float>(num_dims, dims, num_axes, axes, (const float*)x,
                            (float*)mean, (float*)var);
      return kOk;
    case kF64:
      moments<double, double>(num_dims, dims, num_axes, axes, (const double*)x,
                              (double*)mean, (double*)var);
      return kOk;
  }
  return kUnsupportedDtype;
}

// math::InvStd on the AccT stat buffers the operators pass (f32 / f64).
int ref_inv_std(int dtype, int64_t N, float eps, const void* x, void* y) {
  if (dtype == kF32) {
    inv_std<float>(N, eps, (const float*)x, (float*)y);
    return kOk;
  }
  if (dtype == kF64) {
    inv_std<double>(N, eps, (const double*)x, (double*)y);
    return kOk;
  }
  return kUnsupportedDtype;
}

// math::Axpby on the AccT running-stat buffers (f32 / f64).
int ref_axpby(
    int dtype, int64_t N, float alpha, const void* x, float beta, void* y) {
  if (dtype == kF32) {
    axpby<float>(N, alpha, (const float*)x, beta, (float*)y);
    return kOk;
  }
  if (dtype == kF64) {
    axpby<double>(N, alpha, (const double*)x, beta, (double*)y);
    return kOk;
  }
  return kUnsupportedDtype;
}

// kernels::GroupNorm launcher, group_norm_kernel.cc:88-110 (all four dtypes).
int ref_group_norm(
    int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
    const void* x, const void* mu, const void* rsig, const void* gamma,
    const void* beta, void* y) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
  const std::array<int, 4> nchw = {int(N), int(G), int(D), int(S)};
  const std::array<int, 4> nhwc = {int(N), int(S), int(G), int(D)};
#define REF_GN(T, AccT)                                                       \
  if (layout == kNCHWLayout)                                                  \
    group_norm_impl<T, AccT, true>(                                           \
        nchw, (const T*)x, (const AccT*)mu, (const AccT*)rsig,                \
        (const AccT*)gamma, (const AccT*)beta, (T*)y);                        \
  else                                                                        \
    group_norm_impl<T, AccT, false>(                                          \
        nhwc, (const T*)x, (const AccT*)mu, (const AccT*)rsig,                \
        (const AccT*)gamma, (const AccT*)beta, (T*)y);                        \
  return kOk;
  switch (dtype) {
    case kF16: REF_GN(half_t, float)
    case kBF16: REF_GN(bhalf_t, float)
    case kF32: REF_GN(float, float)
    case kF64: REF_GN(double, double)
  }
#undef REF_GN
  return kUnsupportedDtype;
}

// kernels::GroupNormGrad launcher, group_norm_kernel.cc:112-181. Only f32 and
// f64 exist on the reference's CPU (f16/bf16 abort, :158-181). Honours
// ds == db  =>  db = ds + N*G and zero-fills ds, db, dgamma, dbeta (:131-135).
int ref_group_norm_grad(
    int dtype, int64_t N, int64_t G, int64_t D, int64_t S, int layout,
    const void* x, const void* mu, const void* rsig, const void* gamma,
    const void* dy, void* ds, void* db, void* dgamma, void* dbeta, void* dx) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
  const std::array<int, 4> nchw = {int(N), int(G), int(D), int(S)};
  const std::array<int, 4> nhwc = {int(N), int(S), int(G), int(D)};
#define REF_GNG(T)                                                            \
  {                                                                           \
    T* ds_ = (T*)ds;                                                          \
    T* db_ = (ds == db) ? ds_ + N * G : (T*)db;                               \
    std::fill(ds_, ds_ + N * G, T(0));                                        \
    std::fill(db_, db_ + N * G, T(0));                                        \
    std::fill((T*)dgamma, (T*)dgamma + G * D, T(0));                          \
    std::fill((T*)dbeta, (T*)dbeta + G * D, T(0));                            \
    if (layout == kNCHWLayout) {                                              \
      group_norm_internal_grad<T, T, true>(                                   \
          nchw, (const T*)x, (const T*)gamma, (const T*)dy, ds_, db_);        \
      group_norm_grad_impl<T, T, true>(                                       \
          nchw, (const T*)x, (const T*)mu, (const T*)rsig, (const T*)gamma,   \
          ds_, db_, (const T*)dy, (T*)dgamma, (T*)dbeta, (T*)dx);             \
    } else {                                                                  \
      group_norm_internal_grad<T, T, false>(                                  \
          nhwc, (const T*)x, (const T*)gamma, (const T*)dy, ds_, db_);        \
      group_norm_grad_impl<T, T, false>(                                      \
          nhwc, (const T*)x, (const T*)mu, (const T*)rsig, (const T*)gamma,   \
          ds_, db_, (const T*)dy, (T*)dgamma, (T*)dbeta, (T*)dx);             \
    }                                                                         \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_GNG(float)
  if (dtype == kF64) REF_GNG(double)
#undef REF_GNG
  return kUnsupportedDtype;
}

// kernels::BatchNormExpectation launcher, batch_norm_kernel.cc:178-199.
int ref_batch_norm_expectation(
    int dtype, int64_t N, int64_t C, int64_t S, float normalizer, int layout,
    const void* x, void* ex, void* ex2) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
#define REF_BNE(T)                                                            \
  {                                                                           \
    std::fill((T*)ex, (T*)ex + C, T(0));                                      \
    std::fill((T*)ex2, (T*)ex2 + C, T(0));                                    \
    if (layout == kNCHWLayout)                                                \
      batch_norm_expectation_impl<T, T, true>(                                \
          {int(N), int(C), int(S)}, T(normalizer), (const T*)x, (T*)ex,       \
          (T*)ex2);                                                           \
    else                                                                      \
      batch_norm_expectation_impl<T, T, false>(                               \
          {int(N), int(S), int(C)}, T(normalizer), (const T*)x, (T*)ex,       \
          (T*)ex2);                                                           \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_BNE(float)
  if (dtype == kF64) REF_BNE(double)
#undef REF_BNE
  return kUnsupportedDtype;
}

// kernels::BatchNorm launcher, batch_norm_kernel.cc:228-258. Honours
// scale == rsig => scale = rsig + C, bias = rsig + 2C  (inference, 3C buffer)
// scale == bias => bias = scale + C                    (training, 2C buffer)
int ref_batch_norm(
    int dtype, int64_t N, int64_t C, int64_t S, int layout, const void* x,
    const void* mu, const void* rsig, const void* gamma, const void* beta,
    void* scale, void* bias, void* y) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
#define REF_BN(T)                                                             \
  {                                                                           \
    T* scale_ = (T*)scale;                                                    \
    T* bias_ = (T*)bias;                                                      \
    if ((const void*)scale == rsig) {                                         \
      scale_ = (T*)rsig + C, bias_ = (T*)rsig + C * 2;                        \
    } else if (scale == bias) {                                               \
      bias_ = scale_ + C;                                                     \
    }                                                                         \
    batch_norm_fused_params<T>(                                               \
        int(C), (const T*)mu, (const T*)rsig, (const T*)gamma,                \
        (const T*)beta, scale_, bias_);                                       \
    if (layout == kNCHWLayout)                                                \
      batch_norm_affine<T, T, true>(                                          \
          int(N), int(C), int(S), (const T*)x, scale_, bias_, (T*)y);         \
    else                                                                      \
      batch_norm_affine<T, T, false>(                                         \
          int(N), int(C), int(S), (const T*)x, scale_, bias_, (T*)y);         \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_BN(float)
  if (dtype == kF64) REF_BN(double)
#undef REF_BN
  return kUnsupportedDtype;
}

// kernels::BatchNormWGrad launcher, batch_norm_kernel.cc:282-306. Honours
// dgamma == dbeta => dbeta = dgamma + C, zero-fills both.
int ref_batch_norm_wgrad(
    int dtype, int64_t N, int64_t C, int64_t S, int layout, const void* x,
    const void* mu, const void* rsig, const void* dy, void* dgamma,
    void* dbeta) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
#define REF_BNW(T)                                                            \
  {                                                                           \
    T* dg = (T*)dgamma;                                                       \
    T* dbt = (dgamma == dbeta) ? dg + C : (T*)dbeta;                          \
    std::fill(dg, dg + C, T(0));                                              \
    std::fill(dbt, dbt + C, T(0));                                            \
    if (layout == kNCHWLayout)                                                \
      batch_norm_wgrad_impl<T, T, true>(                                      \
          {int(N), int(C), int(S)}, (const T*)x, (const T*)mu,                \
          (const T*)rsig, (const T*)dy, dg, dbt);                             \
    else                                                                      \
      batch_norm_wgrad_impl<T, T, false>(                                     \
          {int(N), int(S), int(C)}, (const T*)x, (const T*)mu,                \
          (const T*)rsig, (const T*)dy, dg, dbt);                             \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_BNW(float)
  if (dtype == kF64) REF_BNW(double)
#undef REF_BNW
  return kUnsupportedDtype;
}

// kernels::BatchNormTrainingGrad launcher, batch_norm_kernel.cc:336-361.
int ref_batch_norm_training_grad(
    int dtype, int64_t N, int64_t C, int64_t S, float normalizer, int layout,
    const void* x, const void* mu, const void* rsig, const void* gamma,
    const void* dgamma, const void* dbeta, const void* dy, void* dx) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
#define REF_BNT(T)                                                            \
  {                                                                           \
    const T* dg = (const T*)dgamma;                                           \
    const T* dbt = (dgamma == dbeta) ? dg + C : (const T*)dbeta;              \
    if (layout == kNCHWLayout)                                                \
      batch_norm_training_grad_impl<T, T, true>(                              \
          {int(N), int(C), int(S)}, T(normalizer), (const T*)x,               \
          (const T*)mu, (const T*)rsig, (const T*)gamma, dg, dbt,             \
          (const T*)dy, (T*)dx);                                              \
    else                                                                      \
      batch_norm_training_grad_impl<T, T, false>(                             \
          {int(N), int(S), int(C)}, T(normalizer), (const T*)x,               \
          (const T*)mu, (const T*)rsig, (const T*)gamma, dg, dbt,             \
          (const T*)dy, (T*)dx);                                              \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_BNT(float)
  if (dtype == kF64) REF_BNT(double)
#undef REF_BNT
  return kUnsupportedDtype;
}

// kernels::BatchNormInferenceGrad launcher, batch_norm_kernel.cc:390-417.
// dgamma == nullptr skips the parameter gradients.
int ref_batch_norm_inference_grad(
    int dtype, int64_t N, int64_t C, int64_t S, int layout, const void* x,
    const void* mu, const void* rsig, const void* gamma, const void* dy,
    void* dgamma, void* dbeta, void* dx) {
  if (layout != kNCHWLayout && layout != kNHWCLayout) return kBadArg;
  if (dtype != kF32 && dtype != kF64) return kUnsupportedDtype;
  if (dgamma != nullptr) {
    ref_batch_norm_wgrad(dtype, N, C, S, layout, x, mu, rsig, dy, dgamma, dbeta);
  }
#define REF_BNI(T)                                                            \
  {                                                                           \
    if (layout == kNCHWLayout)                                                \
      batch_norm_inference_grad_impl<T, T, true>(                             \
          int(N), int(C), int(S), (const T*)rsig, (const T*)gamma,            \
          (const T*)dy, (T*)dx);                                              \
    else                                                                      \
      batch_norm_inference_grad_impl<T, T, false>(                            \
          int(N), int(C), int(S), (const T*)rsig, (const T*)gamma,            \
          (const T*)dy, (T*)dx);                                              \
    return kOk;                                                               \
  }
  if (dtype == kF32) REF_BNI(float)
  REF_BNI(double)
#undef REF_BNI
}

// kernels::Softmax / LogSoftmax / SoftmaxGrad / LogSoftmaxGrad launchers,
// softmax_kernel.cc:112-157. The reference evaluates f16/bf16 in Eigen's
// half types; this oracle offers f32 and f64 only: 16-bit I/O is checked
// against the f32 kernel run on the 16-bit-rounded inputs.
#define REF_SM_FWD(name, fn)                                                  \
  int name(int dtype, int64_t N, int64_t S, int64_t C, const void* x,         \
           void* y) {                                                         \
    if (dtype == kF32) {                                                      \
      fn<float>(int(N), int(S), int(C), (const float*)x, (float*)y);          \
      return kOk;                                                             \
    }                                                                         \
    if (dtype == kF64) {                                                      \
      fn<double>(int(N), int(S), int(C), (const double*)x, (double*)y);       \
      return kOk;                                                             \
    }                                                                         \
    return kUnsupportedDtype;                                                 \
  }
#define REF_SM_BWD(name, fn)                                                  \
  int name(int dtype, int64_t N, int64_t S, int64_t C, const void* dy,        \
           const void* y, void* dx) {                                         \
    if (dtype == kF32) {                                                      \
      fn<float>(int(N), int(S), int(C), (const float*)dy, (const float*)y,    \
                (float*)dx);                                                  \
      return kOk;                                                             \
    }                                                                         \
    if (dtype == kF64) {                                                      \
      fn<double>(int(N), int(S), int(C), (const double*)dy,                   \
                 (const double*)y, (double*)dx);                              \
      return kOk;                                                             \
    }                                                                         \
    return kUnsupportedDtype;                                                 \
  }
REF_SM_FWD(ref_softmax, softmax)
REF_SM_FWD(ref_log_softmax, log_softmax)
REF_SM_BWD(ref_softmax_grad, softmax_grad)
REF_SM_BWD(ref_log_softmax_grad, log_softmax_grad)
#undef REF_SM_FWD
#undef REF_SM_BWD

// kernels::L1Norm / L2Norm / L1NormGrad / L2NormGrad launchers,
// lp_norm_kernel.cc:105-157. p is 1 or 2. f32 and f64 only, as for softmax.
int ref_lp_norm(int dtype, int p, int64_t N, int64_t S, int64_t C,
                float normalizer, float epsilon, const void* x, void* y) {
  if (p != 1 && p != 2) return kBadArg;
  if (dtype == kF32) {
    if (p == 1) lp_norm<float, 1>(int(N), int(S), int(C), normalizer, epsilon, (const float*)x, (float*)y);
    else lp_norm<float, 2>(int(N), int(S), int(C), normalizer, epsilon, (const float*)x, (float*)y);
    return kOk;
  }
  if (dtype == kF64) {
    if (p == 1) lp_norm<double, 1>(int(N), int(S), int(C), normalizer, epsilon, (const double*)x, (double*)y);
    else lp_norm<double, 2>(int(N), int(S), int(C), normalizer, epsilon, (const double*)x, (double*)y);
    return kOk;
  }
  return kUnsupportedDtype;
}

int ref_lp_norm_grad(int dtype, int p, int64_t N, int64_t S, int64_t C,
                     float normalizer, float epsilon, const void* dy,
                     const void* x, void* dx) {
  if (p != 1 && p != 2) return kBadArg;
  if (dtype == kF32) {
    if (p == 1) lp_norm_grad<float, 1>(int(N), int(S), int(C), normalizer, epsilon, (const float*)dy, (const float*)x, (float*)dx);
    else lp_norm_grad<float, 2>(int(N), int(S), int(C), normalizer, epsilon, (const float*)dy, (const float*)x, (float*)dx);
    return kOk;
  }
  if (dtype == kF64) {
    if (p == 1) lp_norm_grad<double, 1>(int(N), int(S), int(C), normalizer, epsilon, (const double*)dy, (const double*)x, (double*)dx);
    else lp_norm_grad<double, 2>(int(N), int(S), int(C), normalizer, epsilon, (const double*)dy, (const double*)x, (double*)dx);
    return kOk;
  }
  return kUnsupportedDtype;
}

// math::ReduceSum (kind 0) / ReduceSumSqr (1) / ReduceL1 (2), reduce.cc:162-236.
// float16 / bfloat16 are CPU_UNSUPPORTED_DTYPE there (:162-186).
int ref_reduce_sum(int dtype, int kind, int num_dims, const int64_t* dims,
                   int num_axes, const int64_t* axes, float scale,
                   const void* x, void* y) {
  if (kind < 0 || kind > 2) return kBadArg;
  if (dtype == kF32) {
    const float* xp = (const float*)x;
    float* yp = (float*)y;
    if (kind == 0) reduce_sum<float, 0>(num_dims, dims, num_axes, axes, scale, xp, yp);
    else if (kind == 1) reduce_sum<float, 1>(num_dims, dims, num_axes, axes, scale, xp, yp);
    else reduce_sum<float, 2>(num_dims, dims, num_axes, axes, scale, xp, yp);
    return kOk;
  }
  if (dtype == kF64) {
    const double* xp = (const double*)x;
    double* yp = (double*)y;
    if (kind == 0) reduce_sum<double, 0>(num_dims, dims, num_axes, axes, scale, xp, yp);
    else if (kind == 1) reduce_sum<double, 1>(num_dims, dims, num_axes, axes, scale, xp, yp);
    else reduce_sum<double, 2>(num_dims, dims, num_axes, axes, scale, xp, yp);
    return kOk;
  }
  return kUnsupportedDtype;
}

// Loss kernels: dtype f32 / f64 only (cross_entropy_kernel.cc:110-165,
// generic_loss_kernel.cc:27-81 instantiate the 16-bit types for the reductions
// only; the softmax loss operators dispatch on float and double).
// target_dtype: 4 = int32, 5 = int64.
int ref_cross_entropy(int dtype, int64_t N, const void* input,
                      const void* target, void* loss) {
  if (dtype == kF32) { cross_entropy_dense(N, (const float*)input, (const float*)target, (float*)loss); return kOk; }
  if (dtype == kF64) { cross_entropy_dense(N, (const double*)input, (const double*)target, (double*)loss); return kOk; }
  return kUnsupportedDtype;
}

#define REF_LOSS_DISPATCH(FN, ...)                                              \
  if (dtype == kF32 && target_dtype == 4) { FN<float, int32_t>(__VA_ARGS__); return kOk; }  \
  if (dtype == kF32 && target_dtype == 5) { FN<float, int64_t>(__VA_ARGS__); return kOk; }  \
  if (dtype == kF64 && target_dtype == 4) { FN<double, int32_t>(__VA_ARGS__); return kOk; } \
  if (dtype == kF64 && target_dtype == 5) { FN<double, int64_t>(__VA_ARGS__); return kOk; } \
  return kUnsupportedDtype;

int ref_sparse_cross_entropy(int dtype, int target_dtype, int64_t N, int64_t S,
                             int64_t C, int64_t ignore_index, const void* input,
                             const void* target, void* loss, void* mask) {
  REF_LOSS_DISPATCH(sparse_ce_erased, int(N), int(S), int(C), int(ignore_index), input, target, loss, mask)
}

int ref_softmax_cross_entropy_grad(int dtype, int target_dtype, int64_t N,
                                   int64_t S, int64_t C, int64_t ignore_index,
                                   const void* target, void* dx, void* mask) {
  REF_LOSS_DISPATCH(sce_grad_erased, int(N), int(S), int(C), int(ignore_index), target, dx, mask)
}
#undef REF_LOSS_DISPATCH

int ref_reduce_loss(int dtype, int64_t N, int64_t num_masks, float normalizer,
                    const void* x, const void* mask, void* y) {
  if (dtype == kF32) { reduce_loss(N, num_masks, normalizer, (const float*)x, (const float*)mask, (float*)y); return kOk; }
  if (dtype == kF64) { reduce_loss(N, num_masks, normalizer, (const double*)x, (const double*)mask, (double*)y); return kOk; }
  return kUnsupportedDtype;
}

int ref_reduce_loss_grad(int dtype, int64_t N, int64_t num_masks,
                         float normalizer, const void* dl, const void* mask,
                         void* dx) {
  if (dtype == kF32) { reduce_loss_grad(N, num_masks, normalizer, (const float*)dl, (const float*)mask, (float*)dx); return kOk; }
  if (dtype == kF64) { reduce_loss_grad(N, num_masks, normalizer, (const double*)dl, (const double*)mask, (double*)dx); return kOk; }
  return kUnsupportedDtype;
}

int ref_broadcast_loss_grad(int dtype, int64_t N, int64_t S, int64_t C,
                            const void* dl, void* dx) {
  if (dtype == kF32) { broadcast_loss_grad(int(N), int(S), int(C), (const float*)dl, (float*)dx); return kOk; }
  if (dtype == kF64) { broadcast_loss_grad(int(N), int(S), int(C), (const double*)dl, (double*)dx); return kOk; }
  return kUnsupportedDtype;
}

} // extern "C"
