"""Python mirror of the reference's ``kernels::`` / ``math::`` free functions.

Same names (snake-cased), argument order and aliasing conventions as the C++
templates of dragon/kernels/normalization/op_kernels.h (LayerNorm, GroupNorm,
BatchNorm, L1/L2Norm), dragon/kernels/loss/op_kernels.h (softmax cross-entropy),
dragon/kernels/activation/op_kernels.h and dragon/kernels/math/op_kernels.h;
the trailing ``Context* ctx`` becomes the current torch stream. Tensors are
torch CUDA tensors used purely as device memory: every function passes raw
pointers through the C ABI (include/dragon_hip.h) to the gfx950 kernels.
"""

import ctypes

import torch

from . import _lib

_DTYPES = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2, torch.float64: 3}
_TARGET_DTYPES = {torch.int32: 4, torch.int64: 5}
REDUCTIONS = {"NONE": 0, "SUM": 1, "MEAN": 2, "BATCH_MEAN": 3, "VALID": 4}
_LAYOUTS = {"NCHW": 0, "NHWC": 1}

# Per-(device, stream) scratch, grown monotonically and never freed between
# calls: the role of the "BufferShared" tensor of the context's scratch
# workspace (dragon/core/workspace.h:81-92, dragon/core/context_cuda.cc:120-129).
_scratch = {}


def dtype_tag(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s" % t.dtype)


def target_tag(t):
    try:
        return _TARGET_DTYPES[t.dtype]
    except KeyError:
        raise TypeError("unsupported target dtype %s" % t.dtype)


def layout_tag(data_format):
    if data_format not in _LAYOUTS:
        raise ValueError("Unknown DataFormat: " + str(data_format))
    return _LAYOUTS[data_format]


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("kernel arguments must live in device memory")
    if not t.is_contiguous():
        raise ValueError("kernel arguments must be contiguous")
    return ctypes.c_void_p(t.data_ptr())


def workspace(nbytes, device):
    """Device scratch of at least ``nbytes`` for the current stream."""
    if nbytes == 0:
        return None
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    buf = _scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _scratch[key] = buf
    return buf


def _call(name, *args):
    _lib.check(name, getattr(_lib.lib(), name)(*args))


def _dims(values):
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


# ---------------------------------------------------------------- math::

def inv_std(N, eps, x, y):
    _call("dragon_hip_inv_std", dtype_tag(x), N, eps, _ptr(x), _ptr(y), _stream())


def axpby(N, alpha, x, beta, y):
    _call("dragon_hip_axpby", dtype_tag(x), N, alpha, _ptr(x), beta, _ptr(y), _stream())


def copy(N, x, y):
    _call("dragon_hip_copy", dtype_tag(x), N, _ptr(x), _ptr(y), _stream())


def set(N, value, y):  # noqa: A001 - the reference's name is math::Set
    _call("dragon_hip_set", dtype_tag(y), N, value, _ptr(y), _stream())


def square(N, x, y):
    _call("dragon_hip_square", dtype_tag(x), N, _ptr(x), _ptr(y), _stream())


def sub(N, a, b, y):
    _call("dragon_hip_sub", dtype_tag(a), N, _ptr(a), _ptr(b), _ptr(y), _stream())


def _reduce(name, dims, axes, scale, x, y):
    d, a = _dims(dims), _dims(axes)
    tag = dtype_tag(x)
    need = _lib.lib().dragon_hip_reduce_scratch_bytes(tag, len(dims), d, len(axes), a)
    ws = workspace(need, x.device)
    _call(name, tag, len(dims), d, len(axes), a, scale, _ptr(x), _ptr(y), _ptr(ws), need, _stream())


def reduce_sum(dims, axes, scale, x, y):
    _reduce("dragon_hip_reduce_sum", dims, axes, scale, x, y)


def reduce_sum_sqr(dims, axes, scale, x, y):
    _reduce("dragon_hip_reduce_sum_sqr", dims, axes, scale, x, y)


def reduce_l1(dims, axes, scale, x, y):
    _reduce("dragon_hip_reduce_l1", dims, axes, scale, x, y)


def sum(N, scale, x, y):  # noqa: A001 - the reference's name is math::Sum
    reduce_sum([N], [0], scale, x, y)


# ---------------------------------------------------------------- kernels::

def moments(dims, axes, x, mean, var):
    d, a = _dims(dims), _dims(axes)
    tag = dtype_tag(x)
    need = _lib.lib().dragon_hip_moments_scratch_bytes(tag, len(dims), d, len(axes), a)
    ws = workspace(need, x.device)
    _call("dragon_hip_moments", tag, len(dims), d, len(axes), a, _ptr(x), _ptr(mean), _ptr(var),
          _ptr(ws), need, _stream())


def layer_norm(N, C, epsilon, x, gamma, beta, mu, rsig, y):
    _call("dragon_hip_layer_norm", dtype_tag(x), N, C, epsilon, _ptr(x), _ptr(gamma), _ptr(beta),
          _ptr(mu), _ptr(rsig), _ptr(y), _stream())


def group_norm(N, G, D, S, data_format, x, mu, rsig, gamma, beta, y):
    _call("dragon_hip_group_norm", dtype_tag(x), N, G, D, S, layout_tag(data_format), _ptr(x),
          _ptr(mu), _ptr(rsig), _ptr(gamma), _ptr(beta), _ptr(y), _stream())


def group_norm_grad(N, G, D, S, data_format, x, mu, rsig, gamma, dy, ds, db, dgamma, dbeta, dx):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    need = _lib.lib().dragon_hip_group_norm_grad_scratch_bytes(tag, N, G, D, S, lay)
    ws = workspace(need, x.device)
    _call("dragon_hip_group_norm_grad", tag, N, G, D, S, lay, _ptr(x), _ptr(mu), _ptr(rsig),
          _ptr(gamma), _ptr(dy), _ptr(ds), _ptr(db), _ptr(dgamma), _ptr(dbeta), _ptr(dx),
          _ptr(ws), need, _stream())


def group_norm_grad_timeline(N, G, D, S, data_format, x, mu, rsig, gamma, dy, ds, db, dgamma, dbeta,
                             dx, workgroups=2048):
    """group_norm_grad with the phase clock of the LayerNorm backward row kernel: returns an
    int64 tensor [workgroups, 6] (start, first row summed, row loop end, end in 10 ns ticks,
    XCD, rows of the first row group); workgroups that recorded nothing stay zero."""
    tag, lay = dtype_tag(x), layout_tag(data_format)
    need = _lib.lib().dragon_hip_group_norm_grad_scratch_bytes(tag, N, G, D, S, lay)
    ws = workspace(need, x.device)
    stamps = torch.zeros((workgroups, 6), dtype=torch.int64, device=x.device)
    _call("dragon_hip_group_norm_grad_timeline", tag, N, G, D, S, lay, _ptr(x), _ptr(mu), _ptr(rsig),
          _ptr(gamma), _ptr(dy), _ptr(ds), _ptr(db), _ptr(dgamma), _ptr(dbeta), _ptr(dx),
          _ptr(ws), need, _ptr(stamps), workgroups, _stream())
    return stamps


def _bn_scratch(tag, N, C, S, lay, device):
    need = _lib.lib().dragon_hip_batch_norm_reduce_scratch_bytes(tag, N, C, S, lay)
    return workspace(need, device), need


def batch_norm_expectation(N, C, S, normalizer, data_format, x, ex, ex2):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    ws, need = _bn_scratch(tag, N, C, S, lay, x.device)
    _call("dragon_hip_batch_norm_expectation", tag, N, C, S, normalizer, lay, _ptr(x), _ptr(ex),
          _ptr(ex2), _ptr(ws), need, _stream())


def batch_norm(N, C, S, data_format, x, mu, rsig, gamma, beta, scale, bias, y):
    _call("dragon_hip_batch_norm", dtype_tag(x), N, C, S, layout_tag(data_format), _ptr(x),
          _ptr(mu), _ptr(rsig), _ptr(gamma), _ptr(beta), _ptr(scale), _ptr(bias), _ptr(y),
          _stream())


def batch_norm_wgrad(N, C, S, data_format, x, mu, rsig, dy, dgamma, dbeta):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    ws, need = _bn_scratch(tag, N, C, S, lay, x.device)
    _call("dragon_hip_batch_norm_wgrad", tag, N, C, S, lay, _ptr(x), _ptr(mu), _ptr(rsig),
          _ptr(dy), _ptr(dgamma), _ptr(dbeta), _ptr(ws), need, _stream())


def batch_norm_training_grad(N, C, S, normalizer, data_format, x, mu, rsig, gamma, dgamma, dbeta,
                             dy, dx):
    _call("dragon_hip_batch_norm_training_grad", dtype_tag(x), N, C, S, normalizer,
          layout_tag(data_format), _ptr(x), _ptr(mu), _ptr(rsig), _ptr(gamma), _ptr(dgamma),
          _ptr(dbeta), _ptr(dy), _ptr(dx), _stream())


def batch_norm_inference_grad(N, C, S, data_format, x, mu, rsig, gamma, dy, dgamma, dbeta, dx):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    ws, need = _bn_scratch(tag, N, C, S, lay, x.device)
    _call("dragon_hip_batch_norm_inference_grad", tag, N, C, S, lay, _ptr(x), _ptr(mu), _ptr(rsig),
          _ptr(gamma), _ptr(dy), _ptr(dgamma), _ptr(dbeta), _ptr(dx), _ptr(ws), need, _stream())


def _softmax_scratch(tag, N, S, C, device):
    need = _lib.lib().dragon_hip_softmax_scratch_bytes(tag, N, S, C)
    return workspace(need, device), need


def softmax(N, S, C, x, y):
    ws, need = _softmax_scratch(dtype_tag(x), N, S, C, x.device)
    _call("dragon_hip_softmax", dtype_tag(x), N, S, C, _ptr(x), _ptr(y), _ptr(ws), need, _stream())


def log_softmax(N, S, C, x, y):
    ws, need = _softmax_scratch(dtype_tag(x), N, S, C, x.device)
    _call("dragon_hip_log_softmax", dtype_tag(x), N, S, C, _ptr(x), _ptr(y), _ptr(ws), need,
          _stream())


def softmax_grad(N, S, C, dy, y, dx):
    ws, need = _softmax_scratch(dtype_tag(y), N, S, C, y.device)
    _call("dragon_hip_softmax_grad", dtype_tag(y), N, S, C, _ptr(dy), _ptr(y), _ptr(dx), _ptr(ws),
          need, _stream())


def log_softmax_grad(N, S, C, dy, y, dx):
    ws, need = _softmax_scratch(dtype_tag(y), N, S, C, y.device)
    _call("dragon_hip_log_softmax_grad", dtype_tag(y), N, S, C, _ptr(dy), _ptr(y), _ptr(dx),
          _ptr(ws), need, _stream())


def l1_norm(N, S, C, normalizer, epsilon, x, y):
    _call("dragon_hip_l1_norm", dtype_tag(x), N, S, C, normalizer, epsilon, _ptr(x), _ptr(y),
          _stream())


def l2_norm(N, S, C, normalizer, epsilon, x, y):
    _call("dragon_hip_l2_norm", dtype_tag(x), N, S, C, normalizer, epsilon, _ptr(x), _ptr(y),
          _stream())


def l1_norm_grad(N, S, C, normalizer, epsilon, dy, x, dx):
    _call("dragon_hip_l1_norm_grad", dtype_tag(x), N, S, C, normalizer, epsilon, _ptr(dy), _ptr(x),
          _ptr(dx), _stream())


def l2_norm_grad(N, S, C, normalizer, epsilon, dy, x, dx):
    _call("dragon_hip_l2_norm_grad", dtype_tag(x), N, S, C, normalizer, epsilon, _ptr(dy), _ptr(x),
          _ptr(dx), _stream())


# ---------------------------------------------------------------- kernels:: (loss)

def _loss_scratch(tag, device):
    need = _lib.lib().dragon_hip_reduce_loss_scratch_bytes(tag)
    return workspace(need, device), need


def cross_entropy(N, input, target, loss):  # dense targets
    _call("dragon_hip_cross_entropy", dtype_tag(input), N, _ptr(input), _ptr(target), _ptr(loss),
          _stream())


def sparse_cross_entropy(N, S, C, ignore_index, input, target, loss, mask):
    _call("dragon_hip_sparse_cross_entropy", dtype_tag(input), target_tag(target), N, S, C,
          ignore_index, _ptr(input), _ptr(target), _ptr(loss), _ptr(mask), _stream())


def softmax_cross_entropy_grad(N, S, C, ignore_index, input, target, dx, mask):
    _call("dragon_hip_softmax_cross_entropy_grad", dtype_tag(dx), target_tag(target), N, S, C,
          ignore_index, _ptr(input), _ptr(target), _ptr(dx), _ptr(mask), _stream())


def reduce_loss(N, num_masks, normalizer, x, mask, y):
    tag = dtype_tag(x)
    ws, need = _loss_scratch(tag, x.device)
    _call("dragon_hip_reduce_loss", tag, N, num_masks, normalizer, _ptr(x), _ptr(mask), _ptr(y),
          _ptr(ws), need, _stream())


def reduce_loss_grad(N, num_masks, normalizer, dl, mask, dx):
    tag = dtype_tag(dx)
    ws, need = _loss_scratch(tag, dx.device)
    _call("dragon_hip_reduce_loss_grad", tag, N, num_masks, normalizer, _ptr(dl), _ptr(mask),
          _ptr(dx), _ptr(ws), need, _stream())


def broadcast_loss_grad(N, S, C, dl, dx):
    _call("dragon_hip_broadcast_loss_grad", dtype_tag(dx), N, S, C, _ptr(dl), _ptr(dx), _stream())


# ---------------------------------------------------------------- fused operator bodies

def softmax_cross_entropy_loss_forward(N, S, C, ignore_index, reduction, x, target, prob, loss):
    tag = dtype_tag(x)
    need = _lib.lib().dragon_hip_softmax_cross_entropy_loss_scratch_bytes(tag, N, S, C)
    ws = workspace(need, x.device)
    _call("dragon_hip_softmax_cross_entropy_loss_forward", tag, target_tag(target), N, S, C,
          ignore_index, REDUCTIONS[reduction.upper()], _ptr(x), _ptr(target), _ptr(prob),
          _ptr(loss), _ptr(ws), need, _stream())


def softmax_cross_entropy_loss_backward(N, S, C, ignore_index, reduction, prob, target, dl, dx):
    tag = dtype_tag(prob)
    ws, need = _loss_scratch(tag, prob.device)
    _call("dragon_hip_softmax_cross_entropy_loss_backward", tag, target_tag(target), N, S, C,
          ignore_index, REDUCTIONS[reduction.upper()], _ptr(prob), _ptr(target), _ptr(dl),
          _ptr(dx), _ptr(ws), need, _stream())


def group_norm_forward(N, G, D, S, data_format, epsilon, x, gamma, beta, mu, rsig, y):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    need = _lib.lib().dragon_hip_group_norm_forward_scratch_bytes(tag, N, G, D, S, lay)
    ws = workspace(need, x.device)
    _call("dragon_hip_group_norm_forward", tag, N, G, D, S, lay, epsilon, _ptr(x), _ptr(gamma),
          _ptr(beta), _ptr(mu), _ptr(rsig), _ptr(y), _ptr(ws), need, _stream())


def batch_norm_training_forward(N, C, S, data_format, momentum, epsilon, x, gamma, beta,
                                running_mean, running_var, mu, rsig, params, y):
    tag, lay = dtype_tag(x), layout_tag(data_format)
    ws, need = _bn_scratch(tag, N, C, S, lay, x.device)
    _call("dragon_hip_batch_norm_training_forward", tag, N, C, S, lay, momentum, epsilon, _ptr(x),
          _ptr(gamma), _ptr(beta), _ptr(running_mean), _ptr(running_var), _ptr(mu), _ptr(rsig),
          _ptr(params), _ptr(y), _ptr(ws), need, _stream())


STATIC_SCRATCH_BYTES = 4 << 20  # DRAGON_HIP_STATIC_SCRATCH_BYTES


def batch_norm_training_forward_noalloc(N, C, S, data_format, momentum, epsilon, x, gamma, beta,
                                        running_mean, running_var, mu, rsig, params, y):
    """batch_norm_training_forward on the library's static scratch: allocates nothing."""
    tag, lay = dtype_tag(x), layout_tag(data_format)
    _call("dragon_hip_batch_norm_training_forward_noalloc", tag, N, C, S, lay, momentum, epsilon,
          _ptr(x), _ptr(gamma), _ptr(beta), _ptr(running_mean), _ptr(running_var), _ptr(mu),
          _ptr(rsig), _ptr(params), _ptr(y), _stream())


def batch_norm_training_backward(N, C, S, normalizer, data_format, x, mu, rsig, gamma, dy, dgamma,
                                 dbeta, dx):
    """BatchNormWGrad + BatchNormTrainingGrad in one call (x and dy read once where a
    channel slice fits the registers)."""
    tag, lay = dtype_tag(x), layout_tag(data_format)
    ws, need = _bn_scratch(tag, N, C, S, lay, x.device)
    _call("dragon_hip_batch_norm_training_backward", tag, N, C, S, normalizer, lay, _ptr(x),
          _ptr(mu), _ptr(rsig), _ptr(gamma), _ptr(dy), _ptr(dgamma), _ptr(dbeta), _ptr(dx),
          _ptr(ws), need, _stream())


def exchange_timed_out():
    """How many slices of the single-read kernels ran out of patience waiting for their
    peers' partial results, and were finished by the repair launch, since the last reset."""
    return int(_lib.lib().dragon_hip_exchange_timed_out())


def exchange_reset(patience=0):
    """Clears that count; ``patience`` polls per wait from now on (0 = the default)."""
    _lib.lib().dragon_hip_exchange_reset(int(patience))


def exchange_plan(dtype_name, units, nseg, seglen, tensors):
    """(slices per unit, packets per slice, packets per thread, grid) of the single-read
    path for ``units`` reduction units of ``nseg`` runs of ``seglen`` elements, or None
    when the shape is left to the split path. Needs no device."""
    import ctypes
    out = [ctypes.c_int(0) for _ in range(4)]
    tag = {"float16": 0, "bfloat16": 1, "float32": 2, "float64": 3}[dtype_name]
    ok = _lib.lib().dragon_hip_exchange_plan(tag, units, nseg, seglen, tensors,
                                             *[ctypes.byref(o) for o in out])
    return tuple(o.value for o in out) if ok else None


def plan_name(op, dtype_name, dims, data_format="NCHW"):
    """The kernels the entry point ``dragon_hip_<op>`` would launch for ``dims`` (its own
    size arguments, in its order), as text; ValueError when the op or the shape is
    rejected. Launches nothing and needs no device."""
    tag = {"float16": 0, "bfloat16": 1, "float32": 2, "float64": 3}[dtype_name]
    buf = ctypes.create_string_buffer(1024)
    n = _lib.lib().dragon_hip_plan_name(op.encode(), tag, layout_tag(data_format), _dims(dims),
                                        len(dims), buf, len(buf))
    if n < 0:
        raise ValueError("no plan for %s %s %s (status %d)" % (op, dtype_name, list(dims), n))
    return buf.value.decode()


# ---------------------------------------------------------------- measurement

def stream_probe_persistent(src, dst, nbytes, threads, in_flight, per_cu, depth, barrier, store_waves):
    """Two reads and one write as a *persistent* kernel would stream them: ``per_cu`` workgroups
    of ``threads`` per compute unit walk the chunks with a grid stride, ``depth`` chunks
    requested ahead into registers, optionally a workgroup barrier per chunk (as a row
    reduction has) and optionally with the stores issued by separate wavefronts fed through
    LDS (``store_waves``: half of the workgroup)."""
    _call("dragon_hip_stream_probe_persistent", int(threads), int(in_flight), int(per_cu), int(depth),
          int(bool(barrier)), int(bool(store_waves)), _ptr(src), _ptr(dst), nbytes, _stream())


def stream_probe(mode, src, dst, nbytes, shape=None):
    """Streaming read (0), copy (1), fill (2) or two reads and one write (3) of ``nbytes``
    bytes per tensor; ``shape`` = (threads per workgroup, loads in flight per thread)."""
    if shape is None:
        _call("dragon_hip_stream_probe", mode, _ptr(src), _ptr(dst), nbytes, _stream())
    else:
        _call("dragon_hip_stream_probe_shape", mode, int(shape[0]), int(shape[1]), _ptr(src), _ptr(dst),
              nbytes, _stream())
