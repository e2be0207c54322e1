"""Device utilities, following the reference's device tests
(test/dragon/test_device.py:28-62) with ``dragon_amd.hip`` in place of ``dragon.cuda``: the
functions are the compiled module's (pybind11 over HIPContext / HIPStream, the counterpart of
dragon/modules/python/cuda.h), and tensors move between numpy and device memory through its
Tensor.FromNumpy / ToNumpy (dragon/modules/python/numpy.h:31-150)."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from dragon_amd import hip
    return hip


def test_stream(hip):
    stream = hip.Stream(device_index=0)
    stream.synchronize()
    hip.synchronize()
    assert stream.query() is True
    assert stream.ptr and stream.index >= 1
    other = hip.Stream(device_index=0)
    assert other.index == stream.index + 1 and other.ptr != stream.ptr
    hip.synchronize(0, stream.index)  # a workspace stream by (device, index), as cuda.synchronize


def test_device(hip):
    from dragon_amd import runtime as rt
    count = hip.get_device_count()
    name = hip.get_device_name(0)
    major, minor = hip.get_device_capability(0)
    assert count >= 1
    assert (major, minor) == (9, 5)          # gfx950
    assert "gfx950" in name
    hip.set_device(0)
    assert hip.current_device() == 0
    hip.set_default_device(1)
    assert hip.default_device() == {"device_type": "hip", "device_index": 1}
    hip.set_default_device(-1)
    assert hip.default_device() == {"device_type": "cpu", "device_index": 0}
    hip.set_random_seed(seed=1337)
    assert hip.get_random_seed() == 1337
    ws = rt.Workspace("device_test")
    assert hip.memory_allocated(workspace=ws) == 0
    ws.feed("x", np.ones((256, 256), np.float32), device=("hip", 0))
    assert hip.memory_allocated(workspace=ws) >= 256 * 256 * 4
    assert hip.is_available()


def test_numpy_to_device_and_back():
    """FromNumpy with a device writes device memory directly, ToNumpy reads it from there;
    a tensor fed on the host side moves when an operator first touches it on the device."""
    from dragon_amd import runtime as rt
    ws = rt.Workspace("feed_fetch")
    rng = np.random.default_rng(5)
    for dtype in (np.float16, np.float32, np.float64, np.int64):
        a = (rng.standard_normal((7, 33)) * 5).astype(dtype)
        ws.feed("d", a, device=("hip", 0))
        t = ws.tensor("d")
        assert t.device == ("hip", 0) and t.dtype == np.dtype(dtype).name
        assert t.data("hip") != 0
        assert np.array_equal(ws.fetch("d"), a)
        assert t.device == ("hip", 0)  # a fetch copies out of device memory, it does not move the tensor
    bits = rng.integers(0, 0x7f00, (4, 16)).astype(np.uint16)
    ws.feed("b", bits, dtype="bfloat16", device=("hip", 0))
    assert ws.info("b") == ("bfloat16", (4, 16)) and np.array_equal(ws.fetch("b"), bits)
    # host-side feed, operator on the device, result fetched from the device
    x = rng.standard_normal((16, 64)).astype(np.float32)
    ws.feed("x", x)
    assert ws.tensor("x").device == ("cpu", 0)
    ws.run_operator(rt.make_def("Softmax", ["x"], ["y"], axis=-1))
    assert ws.tensor("y").device == ("hip", 0)
    e = np.exp(x - x.max(1, keepdims=True))
    assert np.allclose(ws.fetch("y"), e / e.sum(1, keepdims=True), atol=1e-6)


def test_work_enqueued_on_a_stream_object_runs_there(hip):
    import torch
    from dragon_amd import kernels as K
    stream = hip.Stream()
    x = torch.randn(64, 512, device="cuda")
    y = torch.empty_like(x)
    torch.cuda.synchronize()
    with torch.cuda.stream(torch.cuda.ExternalStream(stream.ptr)):
        K.softmax(64, 1, 512, x, y)
    stream.synchronize()
    assert np.allclose(y.sum(1).cpu().numpy(), 1.0, atol=1e-5)


def test_operator_on_a_stream_index(hip):
    """Workspace.RunOperator(def, stream): the operator runs on the device objects' stream of
    that index, the one a Stream object reports (test_device.py:31-36)."""
    from dragon_amd import runtime as rt
    stream = hip.Stream(device_index=0)
    ws = rt.Workspace("stream_test")
    x = np.random.default_rng(6).standard_normal((32, 128)).astype(np.float32)
    ws.feed("x", x)
    ws.run_operator(rt.make_def("Softmax", ["x"], ["y"], axis=-1), stream=stream.index, sync=False)
    stream.synchronize()
    assert stream.query() is True
    assert np.allclose(ws.fetch("y").sum(1), 1.0, atol=1e-5)


def test_reference_style_device_wrapper(hip):
    """The reference re-enters a test body under ``with dragon.device("cuda")``
    (test/dragon/test_ops.py:4183-4204). The same wrapper with the hip device: the body names
    no device, tensors fed inside the scope land in device memory, operators run there, and
    ``hip.memory_allocated()`` reads the current (default) workspace."""
    from dragon_amd import runtime as rt

    def body():  # a device-agnostic test body: LayerNorm of the reference's literal (test_ops.py:4363-4397)
        ws = rt.get_workspace()
        tape = rt.Tape(ws)
        x = ws.feed("x", np.arange(4, dtype=np.float32).reshape(1, 4) * 0.1)
        w = ws.feed("w", np.arange(1, 5, dtype=np.float32) * 0.1)
        b = ws.feed("b", np.arange(4, dtype=np.float32) * 0.1)
        y = rt.layer_norm(tape, [x, w, b], axis=-1, epsilon=1e-5)
        dy = ws.feed("dy", np.arange(4, dtype=np.float32).reshape(1, 4) * 10)
        dx, = tape.gradient(y, [x], output_gradient=dy)
        assert np.allclose(ws.fetch(dx), [[8.897812, -8.95499, -8.926399, 8.983574]], atol=1e-3)
        return ws, x

    scoped = rt.Workspace("wrapper")
    with rt.device("hip", 0), scoped.as_default():
        before = hip.memory_allocated()
        ws, x = body()
        assert ws is scoped and ws.tensor(x).device == ("hip", 0)
        assert hip.memory_allocated() > before
        assert hip.memory_allocated() == hip.memory_allocated(workspace=scoped)
    assert rt.get_workspace() is not scoped
