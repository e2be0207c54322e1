"""ctypes front-end of the CPU oracle (``oracle/ref_cpu.cc``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``. The product path never imports it.

Besides the one-to-one kernel wrappers, the ``op_*`` functions sequence the
kernels the way the reference's operator bodies do:

* ``op_layer_norm``            dragon/operators/normalization/layer_norm_op.cc:9-33
* ``op_layer_norm_grad``       dragon/operators/normalization/layer_norm_op.h:39-54
                               (GroupNormGradient with G=S=1, D=C, NHWC)
* ``op_group_norm`` / ``_grad``  dragon/operators/normalization/group_norm_op.cc:8-85
* ``op_batch_norm_train`` / ``op_batch_norm_infer`` / ``*_grad``
                               dragon/operators/normalization/batch_norm_op.cc:8-226
* ``op_lp_norm`` / ``_grad``     dragon/operators/normalization/lp_norm_op.cc:8-72
* ``op_softmax_cross_entropy_loss`` / ``_grad``
                               dragon/operators/loss/cross_entropy_softmax_loss_op.cc:8-143

16-bit tensors travel as ``numpy.uint16`` bit patterns together with a dtype
name (``"float16"`` / ``"bfloat16"``); ``to_bits`` / ``from_bits`` use the
reference's software rounding (dragon/utils/conversions.h:42-149).
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdragon_ref_cpu.so")

DTYPES = {"float16": 0, "bfloat16": 1, "float32": 2, "float64": 3}
LAYOUTS = {"NCHW": 0, "NHWC": 1}

_lib = None


def build():
    """Compile the oracle with the reference's CPU flag set."""
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def storage_dtype(dtype):
    """numpy dtype that holds one element of ``dtype``."""
    return {"float16": np.uint16, "bfloat16": np.uint16,
            "float32": np.float32, "float64": np.float64}[dtype]


def acc_dtype(dtype):
    """math::Traits<T>::accumulator_type, dragon/utils/math/types.h:69-152."""
    return np.float64 if dtype == "float64" else np.float32


def to_bits(a, dtype):
    """Round an fp32 array to ``dtype`` storage with the reference's rounding."""
    if dtype in ("float32", "float64"):
        return np.ascontiguousarray(a, dtype=storage_dtype(dtype))
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, np.uint16)
    fn = lib().ref_float_to_half if dtype == "float16" else lib().ref_float_to_bfloat16
    fn(ctypes.c_int64(a.size), _p(a), _p(out))
    return out


def from_bits(a, dtype):
    """Widen ``dtype`` storage to fp32 (fp64 stays fp64)."""
    if dtype in ("float32", "float64"):
        return np.asarray(a)
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    fn = lib().ref_half_to_float if dtype == "float16" else lib().ref_bfloat16_to_float
    fn(ctypes.c_int64(a.size), _p(a), _p(out))
    return out


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _check(status, name):
    if status != 0:
        raise RuntimeError("oracle %s failed with status %d" % (name, status))


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


# ---------------------------------------------------------------------------
# One-to-one kernel wrappers
# ---------------------------------------------------------------------------

def layer_norm(dtype, x, gamma, beta, eps):
    """kernels::LayerNorm: x is [N, C] storage; returns (y, mu, rsig)."""
    N, C = x.shape
    at = acc_dtype(dtype)
    x = _c(x, storage_dtype(dtype))
    gamma, beta = _c(gamma, at), _c(beta, at)
    mu, rsig = np.empty(N, at), np.empty(N, at)
    y = np.empty_like(x)
    _check(lib().ref_layer_norm(
        DTYPES[dtype], _i64(N), _i64(C), ctypes.c_float(eps), _p(x), _p(gamma),
        _p(beta), _p(mu), _p(rsig), _p(y)), "layer_norm")
    return y, mu, rsig


def moments(dtype, x, axes):
    """kernels::Moments over ``axes`` of ``x``; returns (mean, var) flat."""
    at = acc_dtype(dtype)
    x = _c(x, storage_dtype(dtype))
    dims = (ctypes.c_int64 * x.ndim)(*x.shape)
    axes = [a % x.ndim for a in axes]
    ax = (ctypes.c_int64 * len(axes))(*axes)
    n_out = int(np.prod([d for i, d in enumerate(x.shape) if i not in axes] or [1]))
    mean, var = np.empty(n_out, at), np.empty(n_out, at)
    _check(lib().ref_moments(
        DTYPES[dtype], x.ndim, dims, len(axes), ax, _p(x), _p(mean), _p(var)),
        "moments")
    return mean, var


REDUCE_KINDS = {"sum": 0, "sum_sqr": 1, "l1": 2}


def reduce_sum(dtype, x, axes, scale=1.0, kind="sum"):
    """math::ReduceSum / ReduceSumSqr / ReduceL1 over ``axes`` of ``x``; returns y flat."""
    t = storage_dtype(dtype)
    x = _c(x, t)
    dims = (ctypes.c_int64 * x.ndim)(*x.shape)
    axes = [a % x.ndim for a in axes]
    ax = (ctypes.c_int64 * len(axes))(*axes)
    n_out = int(np.prod([d for i, d in enumerate(x.shape) if i not in axes] or [1]))
    y = np.empty(n_out, t)
    _check(lib().ref_reduce_sum(
        DTYPES[dtype], REDUCE_KINDS[kind], x.ndim, dims, len(axes), ax, ctypes.c_float(scale),
        _p(x), _p(y)), "reduce_sum")
    return y


def inv_std(x, eps):
    """math::InvStd on an AccT buffer (out of place here; the ops run it in place)."""
    x = np.ascontiguousarray(x)
    dtype = "float64" if x.dtype == np.float64 else "float32"
    y = np.empty_like(x)
    _check(lib().ref_inv_std(
        DTYPES[dtype], _i64(x.size), ctypes.c_float(eps), _p(x), _p(y)), "inv_std")
    return y


def axpby(alpha, x, beta, y):
    """math::Axpby: y <- alpha*x + beta*y, IN PLACE on ``y``."""
    x = np.ascontiguousarray(x)
    assert y.flags["C_CONTIGUOUS"] and y.dtype == x.dtype
    dtype = "float64" if x.dtype == np.float64 else "float32"
    _check(lib().ref_axpby(
        DTYPES[dtype], _i64(x.size), ctypes.c_float(alpha), _p(x),
        ctypes.c_float(beta), _p(y)), "axpby")
    return y


def group_norm(dtype, N, G, D, S, layout, x, mu, rsig, gamma, beta):
    at = acc_dtype(dtype)
    x = _c(x, storage_dtype(dtype))
    y = np.empty_like(x)
    _check(lib().ref_group_norm(
        DTYPES[dtype], _i64(N), _i64(G), _i64(D), _i64(S), LAYOUTS[layout],
        _p(x), _p(_c(mu, at)), _p(_c(rsig, at)), _p(_c(gamma, at)),
        _p(_c(beta, at)), _p(y)), "group_norm")
    return y


def group_norm_grad(dtype, N, G, D, S, layout, x, mu, rsig, gamma, dy):
    """kernels::GroupNormGrad with the op's single 2*N*G scratch passed twice.

    Returns (dx, dgamma, dbeta, ds, db).
    """
    t = storage_dtype(dtype)
    x, dy = _c(x, t), _c(dy, t)
    params = np.empty(2 * N * G, t)
    dgamma, dbeta = np.empty(G * D, t), np.empty(G * D, t)
    dx = np.empty_like(x)
    _check(lib().ref_group_norm_grad(
        DTYPES[dtype], _i64(N), _i64(G), _i64(D), _i64(S), LAYOUTS[layout],
        _p(x), _p(_c(mu, t)), _p(_c(rsig, t)), _p(_c(gamma, t)), _p(dy),
        _p(params), _p(params), _p(dgamma), _p(dbeta), _p(dx)),
        "group_norm_grad")
    return dx, dgamma, dbeta, params[:N * G].copy(), params[N * G:].copy()


def batch_norm_expectation(dtype, N, C, S, normalizer, layout, x):
    t = storage_dtype(dtype)
    x = _c(x, t)
    ex, ex2 = np.empty(C, t), np.empty(C, t)
    _check(lib().ref_batch_norm_expectation(
        DTYPES[dtype], _i64(N), _i64(C), _i64(S), ctypes.c_float(normalizer),
        LAYOUTS[layout], _p(x), _p(ex), _p(ex2)), "batch_norm_expectation")
    return ex, ex2


def batch_norm(dtype, N, C, S, layout, x, mu, rsig, gamma, beta):
    """kernels::BatchNorm with the training-mode aliasing (scale == bias, 2C)."""
    t = storage_dtype(dtype)
    x = _c(x, t)
    params = np.empty(2 * C, t)
    y = np.empty_like(x)
    _check(lib().ref_batch_norm(
        DTYPES[dtype], _i64(N), _i64(C), _i64(S), LAYOUTS[layout], _p(x),
        _p(_c(mu, t)), _p(_c(rsig, t)), _p(_c(gamma, t)), _p(_c(beta, t)),
        _p(params), _p(params), _p(y)), "batch_norm")
    return y, params


def batch_norm_wgrad(dtype, N, C, S, layout, x, mu, rsig, dy):
    """kernels::BatchNormWGrad with dgamma == dbeta aliasing; returns params[2C]."""
    t = storage_dtype(dtype)
    params = np.empty(2 * C, t)
    _check(lib().ref_batch_norm_wgrad(
        DTYPES[dtype], _i64(N), _i64(C), _i64(S), LAYOUTS[layout],
        _p(_c(x, t)), _p(_c(mu, t)), _p(_c(rsig, t)), _p(_c(dy, t)),
        _p(params), _p(params)), "batch_norm_wgrad")
    return params


def batch_norm_training_grad(dtype, N, C, S, normalizer, layout, x, mu, rsig,
                             gamma, params, dy):
    t = storage_dtype(dtype)
    x = _c(x, t)
    dx = np.empty_like(x)
    params = _c(params, t)
    _check(lib().ref_batch_norm_training_grad(
        DTYPES[dtype], _i64(N), _i64(C), _i64(S), ctypes.c_float(normalizer),
        LAYOUTS[layout], _p(x), _p(_c(mu, t)), _p(_c(rsig, t)),
        _p(_c(gamma, t)), _p(params), _p(params), _p(_c(dy, t)), _p(dx)),
        "batch_norm_training_grad")
    return dx


def batch_norm_inference_grad(dtype, N, C, S, layout, x, mu, rsig, gamma, dy,
                              want_wgrad=True):
    t = storage_dtype(dtype)
    x = _c(x, t)
    dx = np.empty_like(x)
    dgamma = np.empty(C, t) if want_wgrad else None
    dbeta = np.empty(C, t) if want_wgrad else None
    _check(lib().ref_batch_norm_inference_grad(
        DTYPES[dtype], _i64(N), _i64(C), _i64(S), LAYOUTS[layout], _p(x),
        _p(_c(mu, t)), _p(_c(rsig, t)), _p(_c(gamma, t)), _p(_c(dy, t)),
        _p(dgamma), _p(dbeta), _p(dx)), "batch_norm_inference_grad")
    return dx, dgamma, dbeta


def _softmax_like(name, dtype, N, S, C, x):
    t = storage_dtype(dtype)
    x = _c(x, t)
    y = np.empty_like(x)
    _check(getattr(lib(), name)(
        DTYPES[dtype], _i64(N), _i64(S), _i64(C), _p(x), _p(y)), name)
    return y


def _softmax_grad_like(name, dtype, N, S, C, dy, y):
    t = storage_dtype(dtype)
    dy, y = _c(dy, t), _c(y, t)
    dx = np.empty_like(y)
    _check(getattr(lib(), name)(
        DTYPES[dtype], _i64(N), _i64(S), _i64(C), _p(dy), _p(y), _p(dx)), name)
    return dx


def softmax(dtype, N, S, C, x):
    return _softmax_like("ref_softmax", dtype, N, S, C, x)


def log_softmax(dtype, N, S, C, x):
    return _softmax_like("ref_log_softmax", dtype, N, S, C, x)


def softmax_grad(dtype, N, S, C, dy, y):
    return _softmax_grad_like("ref_softmax_grad", dtype, N, S, C, dy, y)


def log_softmax_grad(dtype, N, S, C, dy, y):
    return _softmax_grad_like("ref_log_softmax_grad", dtype, N, S, C, dy, y)


def lp_norm(dtype, p, N, S, C, normalizer, epsilon, x):
    """kernels::L1Norm (p=1) / L2Norm (p=2), lp_norm_kernel.cc:10-49."""
    t = storage_dtype(dtype)
    x = _c(x, t)
    y = np.empty_like(x)
    _check(lib().ref_lp_norm(
        DTYPES[dtype], int(p), _i64(N), _i64(S), _i64(C), ctypes.c_float(normalizer),
        ctypes.c_float(epsilon), _p(x), _p(y)), "lp_norm")
    return y


def lp_norm_grad(dtype, p, N, S, C, normalizer, epsilon, dy, x):
    """kernels::L1NormGrad / L2NormGrad, lp_norm_kernel.cc:51-101."""
    t = storage_dtype(dtype)
    dy, x = _c(dy, t), _c(x, t)
    dx = np.empty_like(x)
    _check(lib().ref_lp_norm_grad(
        DTYPES[dtype], int(p), _i64(N), _i64(S), _i64(C), ctypes.c_float(normalizer),
        ctypes.c_float(epsilon), _p(dy), _p(x), _p(dx)), "lp_norm_grad")
    return dx


TARGET_DTYPES = {np.dtype(np.int32): 4, np.dtype(np.int64): 5}


def cross_entropy(dtype, inp, target):
    """kernels::CrossEntropy with dense targets, cross_entropy_kernel.cc:10-15."""
    t = storage_dtype(dtype)
    inp, target = _c(inp, t), _c(target, t)
    loss = np.empty_like(inp)
    _check(lib().ref_cross_entropy(DTYPES[dtype], _i64(inp.size), _p(inp), _p(target), _p(loss)),
           "cross_entropy")
    return loss


def sparse_cross_entropy(dtype, N, S, C, ignore_index, inp, target):
    """kernels::CrossEntropy with class-index targets; returns (loss, mask), each [N*S]."""
    t = storage_dtype(dtype)
    inp = _c(inp, t)
    target = np.ascontiguousarray(target)
    loss, mask = np.empty(N * S, t), np.empty(N * S, t)
    _check(lib().ref_sparse_cross_entropy(
        DTYPES[dtype], TARGET_DTYPES[target.dtype], _i64(N), _i64(S), _i64(C), _i64(ignore_index),
        _p(inp), _p(target), _p(loss), _p(mask)), "sparse_cross_entropy")
    return loss, mask


def softmax_cross_entropy_grad(dtype, N, S, C, ignore_index, target, dx):
    """kernels::SoftmaxCrossEntropyGrad: patches ``dx`` IN PLACE, returns mask [N*S]."""
    t = storage_dtype(dtype)
    assert dx.dtype == t and dx.flags.c_contiguous
    target = np.ascontiguousarray(target)
    mask = np.empty(N * S, t)
    _check(lib().ref_softmax_cross_entropy_grad(
        DTYPES[dtype], TARGET_DTYPES[target.dtype], _i64(N), _i64(S), _i64(C), _i64(ignore_index),
        _p(target), _p(dx), _p(mask)), "softmax_cross_entropy_grad")
    return mask


def reduce_loss(dtype, normalizer, x, mask=None):
    """kernels::ReduceLoss: returns the scalar as a 0-d array."""
    t = storage_dtype(dtype)
    x = _c(x, t)
    y = np.empty(1, t)
    m = None if mask is None else _c(mask, t)
    _check(lib().ref_reduce_loss(
        DTYPES[dtype], _i64(x.size), _i64(0 if m is None else m.size), ctypes.c_float(normalizer),
        _p(x), _p(m), _p(y)), "reduce_loss")
    return y.reshape(())


def reduce_loss_grad(dtype, normalizer, dl, dx, mask=None):
    """kernels::ReduceLossGrad: scales ``dx`` IN PLACE."""
    t = storage_dtype(dtype)
    assert dx.dtype == t and dx.flags.c_contiguous
    m = None if mask is None else _c(mask, t)
    _check(lib().ref_reduce_loss_grad(
        DTYPES[dtype], _i64(dx.size), _i64(0 if m is None else m.size), ctypes.c_float(normalizer),
        _p(_c(dl, t)), _p(m), _p(dx)), "reduce_loss_grad")
    return dx


def broadcast_loss_grad(dtype, N, S, C, dl, dx):
    """kernels::BroadcastLossGrad: ``dx[n, c, s] *= dl[n, s]`` IN PLACE."""
    t = storage_dtype(dtype)
    assert dx.dtype == t and dx.flags.c_contiguous
    _check(lib().ref_broadcast_loss_grad(
        DTYPES[dtype], _i64(N), _i64(S), _i64(C), _p(_c(dl, t)), _p(dx)), "broadcast_loss_grad")
    return dx


# ---------------------------------------------------------------------------
# Operator-level sequences (what the reference's op bodies run)
# ---------------------------------------------------------------------------

def _axis_split(shape, axis):
    axis = axis % len(shape)
    outer = int(np.prod(shape[:axis] or (1,)))
    inner = int(np.prod(shape[axis + 1:] or (1,)))
    return axis, outer, shape[axis], inner


def op_softmax(dtype, x, axis=-1, log=False):
    """SoftmaxOp / LogSoftmaxOp: N=count(0,axis), S=count(axis+1), C=dim(axis)."""
    _, N, C, S = _axis_split(x.shape, axis)
    fn = log_softmax if log else softmax
    return fn(dtype, N, S, C, x).reshape(x.shape)


def op_softmax_grad(dtype, y, dy, axis=-1, log=False):
    _, N, C, S = _axis_split(y.shape, axis)
    fn = log_softmax_grad if log else softmax_grad
    return fn(dtype, N, S, C, dy, y).reshape(y.shape)


def _lp_args(shape, axis, end_axis):
    """LpNormOp: N=count(0,axis), C=count(axis,end_axis+1), S=count(end_axis+1)."""
    axis = axis % len(shape)
    end_axis = axis if end_axis is None else end_axis % len(shape)
    N = int(np.prod(shape[:axis] or (1,)))
    C = int(np.prod(shape[axis:end_axis + 1]))
    S = int(np.prod(shape[end_axis + 1:] or (1,)))
    return N, C, S


def op_lp_norm(dtype, x, axis=-1, end_axis=None, p=2, eps=1e-12, reduction="sum"):
    """LpNormOp, dragon/operators/normalization/lp_norm_op.cc:8-38."""
    N, C, S = _lp_args(x.shape, axis, end_axis)
    normalizer = float(C) if reduction.upper() == "MEAN" else 1.0
    return lp_norm(dtype, p, N, S, C, normalizer, eps, x).reshape(x.shape)


def op_lp_norm_grad(dtype, x, dy, axis=-1, end_axis=None, p=2, eps=1e-12, reduction="sum"):
    """LpNormGradientOp, dragon/operators/normalization/lp_norm_op.cc:40-72."""
    N, C, S = _lp_args(x.shape, axis, end_axis)
    normalizer = float(C) if reduction.upper() == "MEAN" else 1.0
    return lp_norm_grad(dtype, p, N, S, C, normalizer, eps, dy, x).reshape(x.shape)


def _loss_normalizer(reduction, N, S, dim0, has_mask):
    """cross_entropy_softmax_loss_op.cc:69-78."""
    reduction = reduction.upper()
    if reduction == "VALID":
        return -1.0 if has_mask else float(N * S)
    if reduction == "BATCH_MEAN":
        return float(dim0)
    if reduction == "MEAN":
        return float(N * S)
    return 1.0


def op_softmax_cross_entropy_loss(dtype, x, target, axis=-1, ignore_index=None,
                                  reduction="valid"):
    """SoftmaxCrossEntropyLossOp, cross_entropy_softmax_loss_op.cc:8-88.

    ``target`` is dense when it has the dtype of ``x`` and class indices when it
    is int32 / int64. Returns (loss, prob) with prob the op's "X_norm" output.
    """
    ax, N, C, S = _axis_split(x.shape, axis)
    ignore = 2 ** 31 - 1 if ignore_index is None else int(ignore_index)
    prob = softmax(dtype, N, S, C, x)
    dense = np.asarray(target).dtype == storage_dtype(dtype)
    out_shape = tuple(d for i, d in enumerate(x.shape) if i != ax)
    if dense:
        loss, mask = cross_entropy(dtype, prob, target).ravel(), None
    else:
        loss, mask = sparse_cross_entropy(dtype, N, S, C, ignore, prob, target)
    if reduction.upper() == "NONE":
        if dense:
            loss = reduce_sum(dtype, loss.reshape(N, C, S), [1])
        return loss.reshape(out_shape), prob.reshape(x.shape)
    normalizer = _loss_normalizer(reduction, N, S, x.shape[0], mask is not None)
    return reduce_loss(dtype, normalizer, loss, mask), prob.reshape(x.shape)


def op_softmax_cross_entropy_loss_grad(dtype, prob, target, dl, axis=-1, ignore_index=None,
                                       reduction="valid"):
    """SoftmaxCrossEntropyLossGradientOp, cross_entropy_softmax_loss_op.cc:90-143."""
    ax, N, C, S = _axis_split(prob.shape, axis)
    ignore = 2 ** 31 - 1 if ignore_index is None else int(ignore_index)
    t = storage_dtype(dtype)
    dx = np.array(prob, dtype=t, order="C", copy=True)
    mask = None
    if np.asarray(target).dtype == t:
        dx -= _c(target, t).reshape(dx.shape)       # math::Axpy(-1)
    else:
        mask = softmax_cross_entropy_grad(dtype, N, S, C, ignore, target, dx)
    if reduction.upper() == "NONE":
        broadcast_loss_grad(dtype, N, S, C, dl, dx)
    else:
        normalizer = _loss_normalizer(reduction, N, S, prob.shape[0], mask is not None)
        reduce_loss_grad(dtype, normalizer, dl, dx, mask)
    return dx


def op_layer_norm(dtype, x, gamma, beta, axis=-1, eps=1e-5):
    """LayerNormOp: N=count(0,axis), C=count(axis). Returns (y, mu, rsig)."""
    axis = axis % x.ndim
    N = int(np.prod(x.shape[:axis] or (1,)))
    C = int(np.prod(x.shape[axis:]))
    y, mu, rsig = layer_norm(dtype, x.reshape(N, C), gamma, beta, eps)
    return y.reshape(x.shape), mu, rsig


def op_layer_norm_grad(dtype, x, gamma, dy, mu, rsig, axis=-1):
    """LayerNormGradientOp = GroupNormGradient(N, G=1, D=C, S=1, NHWC).

    The reference's CPU has this for f32/f64 only; 16-bit inputs must be
    widened by the caller. Returns (dx, dgamma, dbeta).
    """
    axis = axis % x.ndim
    N = int(np.prod(x.shape[:axis] or (1,)))
    C = int(np.prod(x.shape[axis:]))
    dx, dg, db, _, _ = group_norm_grad(
        dtype, N, 1, C, 1, "NHWC", x, mu, rsig, gamma, dy)
    return dx.reshape(x.shape), dg, db


def _group_args(shape, axis, group):
    """GroupNormOpBase::GetBaseArguments, group_norm_op.h:29-42."""
    axis = axis % len(shape)
    N, C = shape[0], shape[axis]
    S = int(np.prod(shape)) // N // C
    G = group if group > 0 else C
    assert C % G == 0
    layout = "NHWC" if axis + 1 == len(shape) else "NCHW"
    return N, C, S, G, C // G, layout


def op_group_norm(dtype, x, gamma, beta, axis=1, group=0, eps=1e-5):
    """GroupNormOp: Moments -> InvStd -> GroupNorm. Returns (y, mu, rsig)."""
    N, C, S, G, D, layout = _group_args(x.shape, axis, group)
    xs = _c(x, storage_dtype(dtype))
    if layout == "NCHW":
        mu, var = moments(dtype, xs.reshape(N * G, D * S), [1])
    else:
        mu, var = moments(dtype, xs.reshape(N, S, G, D), [1, 3])
    rsig = inv_std(var, eps)
    y = group_norm(dtype, N, G, D, S, layout, xs, mu, rsig, gamma, beta)
    return y.reshape(x.shape), mu, rsig


def op_group_norm_grad(dtype, x, gamma, dy, mu, rsig, axis=1, group=0):
    N, C, S, G, D, layout = _group_args(x.shape, axis, group)
    dx, dg, db, _, _ = group_norm_grad(
        dtype, N, G, D, S, layout, x, mu, rsig, gamma, dy)
    return dx.reshape(x.shape), dg, db


def _bn_args(shape, axis):
    """BatchNormOpBase::GetBaseArguments, batch_norm_op.h:38-47."""
    axis = axis % len(shape)
    N, C = shape[0], shape[axis]
    S = int(np.prod(shape)) // N // C
    layout = "NHWC" if axis + 1 == len(shape) else "NCHW"
    return N, C, S, layout


def op_batch_norm_train(dtype, x, gamma, beta, running_mean, running_var,
                        axis=1, momentum=0.9, eps=1e-5):
    """BatchNormOp::RunTraining, batch_norm_op.cc:8-83 (sync_stats == 0).

    ``running_mean`` / ``running_var`` are updated IN PLACE with the biased
    batch variance. Returns (y, mu, rsig, params[2C]).
    """
    N, C, S, layout = _bn_args(x.shape, axis)
    xs = _c(x, storage_dtype(dtype))
    if layout == "NCHW":
        mu, var = moments(dtype, xs.reshape(N, C, S), [0, 2])
    else:
        mu, var = moments(dtype, xs.reshape(N * S, C), [0])
    decay = np.float32(momentum)
    one_minus = float(np.float32(1.0) - decay)
    axpby(one_minus, mu, float(decay), running_mean)
    axpby(one_minus, var, float(decay), running_var)
    rsig = inv_std(var, eps)
    y, params = batch_norm(dtype, N, C, S, layout, xs, mu, rsig, gamma, beta)
    return y.reshape(x.shape), mu, rsig, params


def op_batch_norm_infer(dtype, x, gamma, beta, running_mean, running_var,
                        axis=1, eps=1e-5):
    """BatchNormOp::RunInference, batch_norm_op.cc:85-116. Returns y."""
    N, C, S, layout = _bn_args(x.shape, axis)
    rsig = inv_std(running_var, eps)
    y, _ = batch_norm(dtype, N, C, S, layout, x, running_mean, rsig, gamma, beta)
    return y.reshape(x.shape)


def op_batch_norm_train_grad(dtype, x, gamma, dy, mu, rsig, axis=1):
    """BatchNormGradientOp::RunTraining, batch_norm_op.cc:118-191.

    Returns (dx, dgamma, dbeta).
    """
    N, C, S, layout = _bn_args(x.shape, axis)
    params = batch_norm_wgrad(dtype, N, C, S, layout, x, mu, rsig, dy)
    dx = batch_norm_training_grad(
        dtype, N, C, S, float(N * S), layout, x, mu, rsig, gamma, params, dy)
    return dx.reshape(x.shape), params[:C].copy(), params[C:].copy()


def op_batch_norm_infer_grad(dtype, x, gamma, running_mean, running_var, dy,
                             axis=1, eps=1e-5):
    """BatchNormGradientOp::RunInference, batch_norm_op.cc:193-226."""
    N, C, S, layout = _bn_args(x.shape, axis)
    rsig = inv_std(running_var, eps)
    dx, dg, db = batch_norm_inference_grad(
        dtype, N, C, S, layout, x, running_mean, rsig, gamma, dy)
    return dx.reshape(x.shape), dg, db
