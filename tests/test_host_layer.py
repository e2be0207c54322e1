"""Host-layer logic that needs no GPU: operator definitions in text format, the
HIP operator registry, schemas, gradient makers, tensor feed/fetch on the host
side, and the error behaviour (the reference LOG(FATAL)s; the C API reports the
same message as an exception)."""

import numpy as np
import pytest

from dragon_amd import runtime as rt


@pytest.fixture()
def ws():
    w = rt.Workspace("host_test")
    yield w
    w.close()


def test_registry_holds_the_ten_operator_types_and_the_sync_aliases():
    ops = set(rt.registered_operators())
    assert {"LayerNorm", "LayerNormGradient", "GroupNorm", "GroupNormGradient", "BatchNorm",
            "BatchNormGradient", "Softmax", "SoftmaxGradient", "LogSoftmax",
            "LogSoftmaxGradient", "SyncBatchNorm", "SyncBatchNormGradient", "LpNorm",
            "LpNormGradient", "SoftmaxCrossEntropyLoss", "SoftmaxCrossEntropyLossGradient"} <= ops


def test_feed_fetch_round_trip(ws):
    rng = np.random.default_rng(0)
    for dtype in (np.float32, np.float64, np.float16, np.int64):
        a = (rng.standard_normal((3, 5)) * 4).astype(dtype)
        ws.feed("t", a)
        assert ws.info("t") == (np.dtype(dtype).name, (3, 5))
        assert np.array_equal(ws.fetch("t"), a)
    bits = rng.integers(0, 65535, (4, 2)).astype(np.uint16)
    ws.feed("b", bits, dtype="bfloat16")
    assert ws.info("b") == ("bfloat16", (4, 2))
    assert np.array_equal(ws.fetch("b"), bits)
    empty = np.zeros((0, 7), np.float32)
    ws.feed("e", empty)
    assert ws.fetch("e").shape == (0, 7)


def test_gradient_definitions_follow_the_reference_makers(ws):
    fwd = rt.make_def("LayerNorm", ["x", "w", "b"], ["y"], name="ln", axis=1, epsilon=1e-3)
    defs, gis = ws.gradient_defs(fwd, ["dy"])
    assert len(defs) == 1 and gis == ["x_grad", "w_grad", "b_grad"]
    d = defs[0]
    assert 'type: "LayerNormGradient"' in d
    assert d.index('input: "x"') < d.index('input: "w"') < d.index('input: "dy"')
    assert 'arg { name: "axis" i: 1 }' in d and 'arg { name: "name" s: "ln" }' in d
    assert "device_type: 4" in d

    fwd = rt.make_def("BatchNorm", ["x", "w", "b", "rm", "rv"], ["y"], name="bn", axis=1)
    defs, gis = ws.gradient_defs(fwd, ["dy"])
    d = defs[0]
    assert 'type: "BatchNormGradient"' in d
    order = [d.index('input: "%s"' % n) for n in ("x", "w", "rm", "rv", "dy")]
    assert order == sorted(order) and 'input: "b"' not in d
    assert gis == ["x_grad", "w_grad", "b_grad", "", ""]

    fwd = rt.make_def("Softmax", ["x"], ["y"], name="sm", axis=-1)
    defs, gis = ws.gradient_defs(fwd, ["dy"])
    assert 'type: "SoftmaxGradient"' in defs[0]
    assert defs[0].index('input: "y"') < defs[0].index('input: "dy"') and gis == ["x_grad"]

    fwd = rt.make_def("SyncBatchNorm", ["x", "w", "b", "rm", "rv"], ["y"], name="sbn")
    assert 'type: "SyncBatchNormGradient"' in ws.gradient_defs(fwd, ["dy"])[0][0]


def test_schema_violations_and_unknown_operators_are_fatal(ws):
    ws.feed("x", np.zeros((2, 4), np.float32))
    with pytest.raises(rt.DragonError, match="inputs"):
        ws.run_operator(rt.make_def("LayerNorm", ["x"], ["y"]))
    with pytest.raises(rt.DragonError, match="not registered"):
        ws.run_operator(rt.make_def("ChannelNorm", ["x"], ["y"]))
    with pytest.raises(rt.DragonError, match="no gradient"):
        ws.gradient_defs(rt.make_def("SoftmaxGradient", ["y", "dy"], ["dx"]), ["g"])
    with pytest.raises(rt.DragonError, match="not in workspace"):
        ws.run_operator(rt.make_def("Softmax", ["missing"], ["y"]))
    # forward may only alias input 0 with output 0
    ws.feed("w", np.zeros(4, np.float32))
    ws.feed("b", np.zeros(4, np.float32))
    with pytest.raises(rt.DragonError, match="inplace"):
        ws.run_operator(rt.make_def("LayerNorm", ["x", "w", "b"], ["x"]))


def test_cpu_device_is_reported_unavailable(ws):
    ws.feed("x", np.zeros((2, 4), np.float32))
    text = rt.make_def("Softmax", ["x"], ["y"]).replace("device_type: 4", "device_type: 0")
    with pytest.raises(rt.DragonError, match="CPU operators are not part of this build"):
        ws.run_operator(text)
    with pytest.raises(rt.DragonError, match="Unknown device"):
        ws.run_operator(text.replace("device_type: 0", "device_type: 9"))


def test_malformed_definitions_are_fatal(ws):
    for bad in ('type "Softmax"', 'type: "Softmax" arg { name: "axis" q: 1 }', 'bogus: 1',
                'type: "Softmax" input: "x'):
        with pytest.raises(rt.DragonError):
            ws.run_operator(bad)


def test_hip_module_without_a_device():
    """Without a GPU the count is zero and every per-device query fails loudly."""
    import torch
    from dragon_amd import _lib, hip
    hip.set_default_device(0)
    assert hip.default_device() == {"device_type": "hip", "device_index": 0}
    hip.set_default_device(-1)
    assert hip.default_device()["device_type"] == "cpu"
    if not torch.cuda.is_available():
        assert hip.is_available() is False
        assert hip.get_device_count() == 0
        with pytest.raises(RuntimeError, match="no ROCm-capable device"):
            hip.get_device_name(0)


def test_compiled_module_binds_the_host_classes():
    """The pybind11 module exposes what the reference's compiled module does for this path:
    Workspace, Tensor, the device functions of dragon/modules/python/cuda.h under hip names,
    and the stream class."""
    from dragon_amd import backend
    for name in ("Workspace", "Tensor", "HIPStream", "hipIsDriverSufficient", "hipGetDevice",
                 "hipGetDeviceCount", "hipGetDeviceName", "hipGetDeviceCapability", "hipSetDevice",
                 "hipSetRandomSeed", "hipStreamSynchronize", "RegisteredOperators",
                 "MakeGradientDefs"):
        assert hasattr(backend, name), name
    assert rt._DEVICE_TO_IDENTIFIER == {"cpu": 0, "cuda": 1, "mps": 2, "mlu": 3, "hip": 4}
    assert rt.get_device_option("hip", 2) == "device_option { device_type: 4 device_id: 2 }"


def test_tensor_numpy_conversions_on_the_host_side():
    """Tensor.FromNumpy / ToNumpy (dragon/modules/python/numpy.h:31-150) for every dtype of
    this path, without a device: shape, dtype, bytes, and where the memory lives."""
    from dragon_amd import backend
    ws = backend.Workspace("numpy_test")
    rng = np.random.default_rng(3)
    for dtype in (np.float16, np.float32, np.float64, np.int64, np.int32, np.uint8):
        a = (rng.standard_normal((2, 3, 4)) * 9).astype(dtype)
        t = ws.CreateTensor("t_" + np.dtype(dtype).name)
        t.FromNumpy(a)
        assert (t.name, t.dtype, tuple(t.dims), t.size) == ("t_" + np.dtype(dtype).name,
                                                             np.dtype(dtype).name, (2, 3, 4), 24)
        assert t.itemsize == a.itemsize and t.nbytes == a.nbytes and t.capacity >= t.nbytes
        assert t.device == ("cpu", 0)
        out = t.ToNumpy()
        assert out.dtype == a.dtype and np.array_equal(out, a)
        assert t.data("cpu") != 0
    bits = rng.integers(0, 65535, (5, 3)).astype(np.uint16)
    b = ws.CreateTensor("b")
    b.FromNumpy(bits, "bfloat16")
    assert b.dtype == "bfloat16" and np.array_equal(b.ToNumpy(), bits)
    # a non-contiguous array is made contiguous, as PyArray_GETCONTIGUOUS does
    a = rng.standard_normal((6, 4)).astype(np.float32)
    t = ws.CreateTensor("strided")
    t.FromNumpy(a.T)
    assert np.array_equal(t.ToNumpy(), a.T)
    assert ws.MemoryAllocated("cpu", 0) >= a.nbytes and ws.MemoryAllocated("hip", 0) == 0
    assert ws.GetTensor("missing") is None and not ws.HasTensor("missing")
    with pytest.raises(RuntimeError, match="cannot hold"):
        b.FromNumpy(bits.astype(np.uint8), "bfloat16")
    with pytest.raises(RuntimeError, match="Unsupported numpy type"):
        b.FromNumpy(np.zeros(3, np.complex64))
    with pytest.raises(RuntimeError, match="empty tensor"):
        ws.CreateTensor("never_written").ToNumpy()


def test_c_runtime_api_still_answers():
    """The C API of the host layer (host/capi/dragon_c_api.h, the counterpart of the
    reference's C++ runtime API) beside the compiled Python module: registry, feed, fetch,
    and a fatal error reported as a message."""
    import ctypes
    import os
    from dragon_amd import _lib
    _lib.lib()
    here = os.path.dirname(os.path.abspath(rt.__file__))
    api = ctypes.CDLL(os.path.join(here, "lib", "libdragon_hip_ops.so"))
    api.dragon_c_last_error.restype = ctypes.c_char_p
    buf = ctypes.create_string_buffer(1 << 14)
    assert api.dragon_c_registered_operators(buf, len(buf)) == 0
    assert "LayerNorm" in buf.value.decode().split("\n")
    ws = ctypes.c_void_p()
    assert api.dragon_c_workspace_create(b"capi", ctypes.byref(ws)) == 0
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    dims = (ctypes.c_int64 * 2)(3, 4)
    assert api.dragon_c_feed_tensor(ws, b"a", b"float32", 2, dims, ctypes.c_void_p(a.ctypes.data)) == 0
    out = np.empty_like(a)
    assert api.dragon_c_fetch_tensor(ws, b"a", ctypes.c_void_p(out.ctypes.data), out.nbytes) == 0
    assert np.array_equal(out, a)
    assert api.dragon_c_run_operator(ws, b'type: "Nope" device_option { device_type: 4 }', 0, 1) == -1
    assert b"not registered" in api.dragon_c_last_error()
    assert api.dragon_c_workspace_destroy(ws) == 0


def test_device_scope_and_default_workspace():
    """``runtime.device`` nests like ``dragon.device`` (context.py:24-52) and operator
    definitions follow it; ``get_workspace`` / ``Workspace.as_default`` give
    ``hip.memory_allocated()`` the workspace the reference's takes (cuda.py:146-169)."""
    from dragon_amd import hip
    assert rt.get_device() == ("cpu", 0)
    assert "device_id: 0" in rt.make_def("Softmax", ["x"], ["y"])
    with rt.device("hip", 3):
        assert rt.get_device() == ("hip", 3)
        assert "device_type: 4 device_id: 3" in rt.make_def("Softmax", ["x"], ["y"])
        with rt.device("hip"):
            assert rt.get_device() == ("hip", 0)
            assert "device_id: 0" in rt.make_def("Softmax", ["x"], ["y"])
        with rt.device("cpu"):
            assert "device_type: 4 device_id: 0" in rt.make_def("Softmax", ["x"], ["y"])
        assert rt.get_device() == ("hip", 3)
        assert "device_id: 1" in rt.make_def("Softmax", ["x"], ["y"], device_id=1)  # explicit wins
    assert rt.get_device() == ("cpu", 0)
    hip.set_default_device(2)
    try:
        assert rt.get_device() == ("hip", 2)
        assert "device_id: 2" in rt.make_def("Softmax", ["x"], ["y"])
    finally:
        hip.set_default_device(-1)
    with pytest.raises(ValueError):
        rt.device("tpu")
    default = rt.get_workspace()
    assert rt.get_workspace() is default
    mine = rt.Workspace("scoped")
    with mine.as_default() as w:
        assert w is mine and rt.get_workspace() is mine
    assert rt.get_workspace() is default
