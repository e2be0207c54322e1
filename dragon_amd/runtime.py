"""Python front end of the C++ host layer (``libdragon_hip_ops.so``).

A thin stand-in for what ``dragon.Workspace`` / ``OpLib.execute`` /
``GradientTape`` do in the reference (dragon/python/core/autograph/op_lib.py:56-235,
dragon/python/core/autograph/backprop.py:27-185): tensors are fed from numpy,
an ``OperatorDef`` is built in protobuf text format with the reference's
argument names, the C++ ``Workspace::RunOperator`` creates and runs the
operator on the HIP device, and results are fetched back to numpy. Nothing is
computed in Python.
"""

import ctypes
import itertools
import os

import numpy as np

from . import _lib

_HERE = os.path.dirname(os.path.abspath(__file__))
OPS_LIB_PATH = os.path.join(_HERE, "lib", "libdragon_hip_ops.so")
PROTO_HIP = 4

_handle = None


class DragonError(RuntimeError):
    """What the reference reports through LOG(FATAL) before aborting."""


def ops_lib():
    global _handle
    if _handle is None:
        if not os.path.exists(OPS_LIB_PATH):
            raise RuntimeError("%s is missing: run __graft_entry__.build()" % OPS_LIB_PATH)
        _lib.lib()  # binds the kernel library (and the HIP runtime torch ships) first
        h = ctypes.CDLL(OPS_LIB_PATH)
        h.dragon_c_last_error.restype = ctypes.c_char_p
        _handle = h
    return _handle


def _check(status):
    if status != 0:
        raise DragonError(ops_lib().dragon_c_last_error().decode())


def registered_operators():
    buf = ctypes.create_string_buffer(1 << 14)
    _check(ops_lib().dragon_c_registered_operators(buf, len(buf)))
    return [s for s in buf.value.decode().split("\n") if s]


def _np_storage(dtype):
    return {"float16": np.uint16, "bfloat16": np.uint16, "float32": np.float32,
            "float64": np.float64, "int64": np.int64, "int32": np.int32}[dtype]


def _quote(s):
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'


def make_def(op_type, inputs, outputs, name="", device_id=0, **args):
    """OperatorDef in protobuf text format (dragon/proto/dragon.proto:99-116)."""
    parts = []
    if name:
        parts.append("name: " + _quote(name))
    parts.append("type: " + _quote(op_type))
    parts += ["input: " + _quote(i) for i in inputs]
    parts += ["output: " + _quote(o) for o in outputs]
    for key, value in args.items():
        if value is None:
            continue
        if isinstance(value, bool):
            value = int(value)
        if isinstance(value, (int, np.integer)):
            field = "i: %d" % value
        elif isinstance(value, (float, np.floating)):
            field = "f: %r" % float(np.float32(value))
        elif isinstance(value, str):
            field = "s: " + _quote(value)
        elif isinstance(value, (list, tuple)) and all(isinstance(v, (int, np.integer)) for v in value):
            field = " ".join("ints: %d" % v for v in value)
        else:
            raise TypeError("unsupported argument %s=%r" % (key, value))
        parts.append("arg { name: %s %s }" % (_quote(key), field))
    parts.append("device_option { device_type: %d device_id: %d }" % (PROTO_HIP, device_id))
    return " ".join(parts)


class Workspace:
    """Named tensors plus operator execution on the HIP device."""

    _uid = itertools.count()

    def __init__(self, name="default"):
        self._ws = ctypes.c_void_p()
        _check(ops_lib().dragon_c_workspace_create(name.encode(), ctypes.byref(self._ws)))

    def close(self):
        if self._ws:
            ops_lib().dragon_c_workspace_destroy(self._ws)
            self._ws = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def unique_name(self, prefix):
        return "%s_%d" % (prefix, next(Workspace._uid))

    def feed(self, name, array, dtype=None):
        """Feed a numpy array; 16-bit floats travel as uint16 bit patterns with ``dtype`` given."""
        if dtype is None:
            dtype = {np.dtype(np.float16): "float16", np.dtype(np.float32): "float32",
                     np.dtype(np.float64): "float64", np.dtype(np.int64): "int64",
                     np.dtype(np.int32): "int32"}[array.dtype]
            if dtype == "float16":
                array = array.view(np.uint16)
        a = np.ascontiguousarray(array, dtype=_np_storage(dtype))
        dims = (ctypes.c_int64 * a.ndim)(*a.shape)
        _check(ops_lib().dragon_c_feed_tensor(self._ws, name.encode(), dtype.encode(), a.ndim, dims,
                                              ctypes.c_void_p(a.ctypes.data)))
        return name

    def has(self, name):
        flag = ctypes.c_int()
        _check(ops_lib().dragon_c_has_tensor(self._ws, name.encode(), ctypes.byref(flag)))
        return bool(flag.value)

    def info(self, name):
        buf = ctypes.create_string_buffer(32)
        ndim = ctypes.c_int()
        dims = (ctypes.c_int64 * 8)()
        _check(ops_lib().dragon_c_tensor_info(self._ws, name.encode(), buf, len(buf),
                                              ctypes.byref(ndim), dims))
        return buf.value.decode(), tuple(dims[i] for i in range(ndim.value))

    def fetch(self, name, raw=False):
        """numpy copy of a tensor. float16 comes back as float16, bfloat16 as uint16 bit
        patterns (``raw=True`` keeps float16 as uint16 too)."""
        dtype, shape = self.info(name)
        out = np.empty(shape, _np_storage(dtype))
        _check(ops_lib().dragon_c_fetch_tensor(self._ws, name.encode(), ctypes.c_void_p(out.ctypes.data),
                                               out.nbytes))
        if dtype == "float16" and not raw:
            return out.view(np.float16)
        return out

    def run_operator(self, def_text, stream=0, sync=True):
        _check(ops_lib().dragon_c_run_operator(self._ws, def_text.encode(), stream, int(sync)))

    def gradient_defs(self, def_text, output_grads):
        """Gradient OperatorDefs of a forward definition and the names of the input gradients."""
        arr = (ctypes.c_char_p * len(output_grads))(*[g.encode() for g in output_grads])
        defs = ctypes.create_string_buffer(1 << 16)
        gis = ctypes.create_string_buffer(1 << 14)
        _check(ops_lib().dragon_c_make_gradient_defs(def_text.encode(), arr, len(output_grads), defs,
                                                     len(defs), gis, len(gis)))
        grad_defs = [d for d in defs.value.decode().split("\n") if d.strip()]
        grad_inputs = gis.value.decode().split("\n")[:-1]
        return grad_defs, grad_inputs


class Tape:
    """Records the forward definitions run through it and replays their gradient
    definitions in reverse, like GradientTape.gradient with output_gradients."""

    def __init__(self, ws):
        self.ws = ws
        self.records = []

    def run(self, op_type, inputs, num_outputs=1, **args):
        name = self.ws.unique_name(op_type)
        outputs = ["%s/y%d" % (name, i) for i in range(num_outputs)]
        text = make_def(op_type, inputs, outputs, name=name, **args)
        self.ws.run_operator(text)
        self.records.append((text, outputs))
        return outputs[0] if num_outputs == 1 else outputs

    def gradient(self, target, sources, output_gradient):
        grads = {target: output_gradient}
        for text, outputs in reversed(self.records):
            if not any(o in grads for o in outputs):
                continue
            g_outputs = [grads.get(o, "NULL") for o in outputs]
            grad_defs, grad_inputs = self.ws.gradient_defs(text, g_outputs)
            for d in grad_defs:
                self.ws.run_operator(d)
            fwd_inputs = [p.split('"')[1] for p in text.split("input: ")[1:]]
            for src, g in zip(fwd_inputs, grad_inputs):
                if g:
                    grads[src] = g
        return [grads.get(s) for s in sources]


# ---------------------------------------------------------------------------
# Functional wrappers with the reference's names and arguments
# (dragon/python/core/ops/normalization_ops.py, activation_ops.py).
# ---------------------------------------------------------------------------

def layer_norm(tape, inputs, axis=-1, epsilon=1e-5):
    return tape.run("LayerNorm", inputs, axis=axis, epsilon=float(epsilon))


def group_norm(tape, inputs, axis=-1, group=0, epsilon=1e-5):
    return tape.run("GroupNorm", inputs, axis=axis, group=group, epsilon=float(epsilon))


def instance_norm(tape, inputs, axis=-1, epsilon=1e-5):
    return group_norm(tape, inputs, axis=axis, group=0, epsilon=epsilon)


def batch_norm(tape, inputs, axis=-1, momentum=0.9, epsilon=1e-5, use_stats=-1, op_type="BatchNorm"):
    return tape.run(op_type, inputs, axis=axis, momentum=float(momentum), epsilon=float(epsilon),
                    use_stats=int(use_stats))


def lp_norm(tape, inputs, axis=-1, end_axis=None, p=2, epsilon=1e-12, reduction="sum"):
    return tape.run("LpNorm", inputs, p=int(p), axis=axis, end_axis=end_axis, epsilon=float(epsilon),
                    reduction=reduction.upper())


def softmax_cross_entropy_loss(tape, inputs, axis=-1, ignore_index=None, reduction="valid"):
    """dragon.losses.softmax_cross_entropy_loss (dragon/python/core/ops/loss_ops.py:301-340)."""
    return tape.run("SoftmaxCrossEntropyLoss", inputs, axis=axis, ignore_index=ignore_index,
                    reduction=reduction.upper())


def softmax(tape, inputs, axis=-1):
    return tape.run("Softmax", inputs, axis=axis)


def log_softmax(tape, inputs, axis=-1):
    return tape.run("LogSoftmax", inputs, axis=axis)
