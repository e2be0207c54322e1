"""HIP device utilities with the names and arguments of ``dragon.cuda``
(dragon/python/core/device/cuda.py:23-277): stream objects, device queries,
the default device and synchronisation, over the compiled module of the host
layer (``backend``: pybind11 bindings of HIPContext / HIPStream, the
counterpart of dragon/modules/python/cuda.h). cuBLAS / cuDNN flag setters have
no counterpart: this library has no vendor-library switches.
"""

from . import backend

# The process-wide default device of ``dragon.device`` scopes
# (dragon/python/core/framework/config.py): type "hip" with an index, or "cpu".
_default = {"device_type": "cpu", "device_index": 0}


class Stream:
    """A non-blocking HIP stream at the default priority (cuda.py:23-67): the next
    unused stream index of the calling thread's device objects."""

    def __init__(self, device_index=None):
        self.device_index = current_device() if device_index is None else int(device_index)
        self._impl = backend.HIPStream(self.device_index)

    @property
    def index(self):
        """The stream index operators are run on (``Workspace.run_operator(..., stream=index)``)."""
        return self._impl.index

    @property
    def ptr(self):
        """The ``hipStream_t`` as an integer."""
        return self._impl.ptr

    def query(self):
        """True when everything enqueued on the stream has finished."""
        return self._impl.Query()

    def synchronize(self):
        self._impl.Synchronize()

    def close(self):
        """Streams belong to the thread's device objects and are destroyed with them."""
        self._impl = None


def is_available():
    """True when the compiled module loads and sees at least one device (cuda.py:134-143)."""
    try:
        return backend.hipIsDriverSufficient() and get_device_count() > 0
    except (OSError, RuntimeError):
        return False


def get_device_count():
    return backend.hipGetDeviceCount()


def current_device():
    return backend.hipGetDevice()


def set_device(device_index=0):
    backend.hipSetDevice(int(device_index))


def get_device_name(device_index=None):
    return backend.hipGetDeviceName(-1 if device_index is None else int(device_index))


def get_device_capability(device_index=None):
    """(major, minor) of the device's ISA version, (9, 5) for gfx950 (cuda.py:82-99)."""
    return backend.hipGetDeviceCapability(-1 if device_index is None else int(device_index))


def memory_allocated(device_index=None, workspace=None):
    """Bytes of device memory held by the tensors of the current workspace (cuda.py:146-169):
    ``runtime.get_workspace()``, i.e. the innermost ``Workspace.as_default()`` or the
    process-wide default one, unless ``workspace`` names another."""
    from . import runtime
    if workspace is None:
        workspace = runtime.get_workspace()
    index = current_device() if device_index is None else int(device_index)
    return workspace.memory_allocated("hip", index)


def set_default_device(device_index=0):
    """Make "hip:<index>" the default device; a negative index restores the CPU (cuda.py:212-233)."""
    if device_index < 0:
        _default.update(device_type="cpu", device_index=0)
    else:
        _default.update(device_type="hip", device_index=int(device_index))


def default_device():
    return dict(_default)


def set_random_seed(device_index=None, seed=3):
    """The seed of a device's generator (cuda.py:248-262). No kernel on this path draws
    random numbers; the device objects keep the value for operators that would."""
    backend.hipSetRandomSeed(-1 if device_index is None else int(device_index), int(seed))


def get_random_seed(device_index=None):
    return backend.hipGetRandomSeed(-1 if device_index is None else int(device_index))


def synchronize(device_index=None, stream_index=None):
    """Wait for a workspace stream of a device (cuda.py:265-277), or for every stream of
    the device when ``stream_index`` is None."""
    index = -1 if device_index is None else int(device_index)
    if stream_index is None:
        backend.hipDeviceSynchronize(index)
    else:
        backend.hipStreamSynchronize(index, int(stream_index))
