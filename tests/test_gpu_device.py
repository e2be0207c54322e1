"""Device utilities, following the reference's device tests
(test/dragon/test_device.py:28-62) with ``dragon_amd.hip`` in place of ``dragon.cuda``."""

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
    assert stream.ptr
    stream.close()


def test_device(hip):
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
    hip.set_random_seed(1337)
    assert hip.memory_allocated() >= 0
    assert hip.is_available()


def test_work_enqueued_on_a_stream_object_runs_there(hip):
    import numpy as np
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
    stream.close()
