"""Python front end of the C++ host layer (``libdragon_hip_ops.so`` through its
compiled Python module, ``backend``).

A thin stand-in for what ``dragon.Workspace`` / ``OpLib.execute`` /
``GradientTape`` do in the reference (dragon/python/core/autograph/op_lib.py:56-235,
dragon/python/core/autograph/backprop.py:27-185): tensors are fed from numpy,
an ``OperatorDef`` is built in protobuf text format with the reference's
argument names, the C++ ``Workspace::RunOperator`` creates and runs the
operator on the HIP device, and results are fetched back to numpy. Nothing is
computed in Python.
"""

import itertools
import threading

import numpy as np

from . import backend

PROTO_HIP = 4
# DeviceTypeProto values by device name: the reference's table
# (dragon/python/core/framework/proto_util.py:132) with the HIP device added.
_DEVICE_TO_IDENTIFIER = {"cpu": 0, "cuda": 1, "mps": 2, "mlu": 3, "hip": PROTO_HIP}


class DragonError(RuntimeError):
    """What the reference reports through LOG(FATAL) before aborting."""


def _guard(fn, *args, **kwargs):
    """Calls into the compiled module; its fatal errors surface as DragonError."""
    try:
        return fn(*args, **kwargs)
    except RuntimeError as e:
        raise DragonError(str(e)) from None


def registered_operators():
    return list(backend.RegisteredOperators())


def get_device_option(device_type, device_index=0, random_seed=None):
    """DeviceOption in protobuf text format (proto_util.py:135-147)."""
    text = "device_type: %d device_id: %d" % (_DEVICE_TO_IDENTIFIER[device_type.lower()], device_index)
    if random_seed is not None:
        text += " random_seed: %d" % random_seed
    return "device_option { %s }" % text


def _quote(s):
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'


# ---------------------------------------------------------------------------
# Device scope and default workspace: what ``dragon.device(...)`` and
# ``dragon.get_workspace()`` give the reference's test bodies
# (dragon/python/core/framework/context.py:24-52,96-103,
# dragon/python/core/framework/workspace.py). A scope is a per-thread stack of
# (device_type, device_index); outside any scope the process-wide default of
# ``hip.set_default_device`` applies.
# ---------------------------------------------------------------------------
_tls = threading.local()


class _DeviceScope:
    def __init__(self, device_type, device_index):
        device_type = device_type.lower()
        if device_type not in _DEVICE_TO_IDENTIFIER:
            raise ValueError("Unsupported device type: " + device_type)
        self.spec = (device_type, int(device_index))

    def __enter__(self):
        _tls.__dict__.setdefault("devices", []).append(self.spec)
        return self

    def __exit__(self, *exc):
        _tls.devices.pop()
        return False


def device(device_type, device_index=0):
    """Context manager that nests the device, as ``dragon.device`` (context.py:24-52):
    operator definitions made and tensors fed inside it go to that device."""
    return _DeviceScope(device_type, device_index)


def get_device():
    """(device_type, device_index) of the innermost scope, else the process default."""
    stack = getattr(_tls, "devices", None)
    if stack:
        return stack[-1]
    from . import hip
    d = hip.default_device()
    return d["device_type"], d["device_index"]


def _operator_device_id(device_id):
    """Operators exist for the HIP device only: an explicit ``device_id`` wins, then the
    index of a "hip" scope or default; under a CPU scope or default they run on hip:0."""
    if device_id is not None:
        return int(device_id)
    device_type, index = get_device()
    return index if device_type == "hip" else 0


def make_def(op_type, inputs, outputs, name="", device_id=None, **args):
    """OperatorDef in protobuf text format (dragon/proto/dragon.proto:99-116); its device
    option is the current device scope unless ``device_id`` names a HIP device."""
    device_id = _operator_device_id(device_id)
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
    parts.append(get_device_option("hip", device_id))
    return " ".join(parts)


class Workspace:
    """Named tensors plus operator execution on the HIP device: the compiled module's
    Workspace (C++ ``dragon::Workspace``) behind the method names the tests use."""

    _uid = itertools.count()

    def __init__(self, name="default"):
        self._impl = backend.Workspace(name)

    def close(self):
        self._impl = None

    def as_default(self):
        """Context manager that makes this the workspace ``get_workspace()`` returns
        (``dragon.Workspace.as_default``)."""
        return _WorkspaceScope(self)

    def unique_name(self, prefix):
        return "%s_%d" % (prefix, next(Workspace._uid))

    def feed(self, name, array, dtype=None, device=None):
        """Feed a numpy array (``Tensor.FromNumpy``). bfloat16 travels as uint16 bit patterns
        with ``dtype`` given, and so may float16. ``device`` = ("hip", index) writes straight
        into device memory; by default the tensor moves there when an operator first reads it."""
        array = np.asarray(array)
        if dtype == "float16" and array.dtype == np.uint16:
            array, dtype = array.view(np.float16), None
        if device is None:  # a "hip" scope feeds straight into that device's memory
            scope = get_device()
            device = scope if scope[0] == "hip" else ("cpu", 0)
        device_type, device_id = device
        tensor = self._impl.CreateTensor(name)
        _guard(tensor.FromNumpy, array, dtype or "", device_type, device_id)
        return name

    def has(self, name):
        return self._impl.HasTensor(name)

    def tensor(self, name):
        """The compiled module's Tensor (name, dims, dtype, device, data pointers)."""
        t = self._impl.GetTensor(name)
        if t is None:
            raise DragonError("Tensor(%s) is not in workspace." % name)
        return t

    def info(self, name):
        t = self.tensor(name)
        return t.dtype, tuple(t.dims)

    def fetch(self, name, raw=False):
        """numpy copy of a tensor (``Tensor.ToNumpy``). float16 comes back as float16, bfloat16
        as uint16 bit patterns (``raw=True`` gives float16 as uint16 too)."""
        out = _guard(self.tensor(name).ToNumpy)
        if raw and out.dtype == np.float16:
            return out.view(np.uint16)
        return out

    def memory_allocated(self, device_type="cpu", device_index=0):
        return self._impl.MemoryAllocated(device_type, device_index)

    def run_operator(self, def_text, stream=0, sync=True):
        _guard(self._impl.RunOperator, def_text, stream, sync)

    def gradient_defs(self, def_text, output_grads):
        """Gradient OperatorDefs of a forward definition and the names of the input gradients."""
        defs, grad_inputs = _guard(backend.MakeGradientDefs, def_text, list(output_grads))
        return list(defs), list(grad_inputs)


class _WorkspaceScope:
    def __init__(self, ws):
        self.ws = ws

    def __enter__(self):
        _tls.__dict__.setdefault("workspaces", []).append(self.ws)
        return self.ws

    def __exit__(self, *exc):
        _tls.workspaces.pop()
        return False


_default_workspace = None
_default_workspace_lock = threading.Lock()


def get_workspace():
    """The innermost ``Workspace.as_default()`` of the thread, else the process-wide
    default workspace, created on first use (``dragon.get_workspace``)."""
    global _default_workspace
    stack = getattr(_tls, "workspaces", None)
    if stack:
        return stack[-1]
    with _default_workspace_lock:
        if _default_workspace is None:
            _default_workspace = Workspace("default")
        return _default_workspace


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
