"""HIP device utilities with the names and arguments of ``dragon.cuda``
(dragon/python/core/device/cuda.py:23-277): stream objects, device queries,
the default device and synchronisation, all over the C ABI of
``libdragon_hip.so`` (include/dragon_hip.h). cuBLAS / cuDNN flag setters have
no counterpart: this library has no vendor-library switches.
"""

import ctypes

from . import _lib

# The process-wide default device of ``dragon.device`` scopes
# (dragon/python/core/framework/config.py): type "hip" with an index, or "cpu".
_default = {"device_type": "cpu", "device_index": 0}
_seeds = {}


def _call(name, *args):
    _lib.check(name, getattr(_lib.lib(), name)(*args))


class Stream:
    """A non-blocking HIP stream at the default priority (cuda.py:23-67)."""

    def __init__(self, device_index=None):
        self.device_index = current_device() if device_index is None else int(device_index)
        prev = current_device()
        set_device(self.device_index)
        handle = ctypes.c_void_p()
        try:
            _call("dragon_hip_stream_create", ctypes.byref(handle))
        finally:
            set_device(prev)
        self._ptr = handle

    @property
    def ptr(self):
        """The ``hipStream_t`` as an integer."""
        return self._ptr.value

    def query(self):
        """True when everything enqueued on the stream has finished."""
        done = ctypes.c_int()
        _call("dragon_hip_stream_query", self._ptr, ctypes.byref(done))
        return bool(done.value)

    def synchronize(self):
        _call("dragon_hip_stream_sync", self._ptr)

    def close(self):
        if self._ptr is not None and self._ptr.value:
            _call("dragon_hip_stream_destroy", self._ptr)
        self._ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def is_available():
    """True when the kernel library loads and sees at least one device (cuda.py:134-143)."""
    try:
        return get_device_count() > 0
    except (OSError, _lib.DragonHipError):
        return False


def get_device_count():
    n = ctypes.c_int()
    _call("dragon_hip_device_count", ctypes.byref(n))
    return n.value


def current_device():
    d = ctypes.c_int()
    _call("dragon_hip_get_device", ctypes.byref(d))
    return d.value


def set_device(device_index=0):
    _call("dragon_hip_set_device", int(device_index))


def get_device_name(device_index=None):
    buf = ctypes.create_string_buffer(256)
    idx = current_device() if device_index is None else int(device_index)
    _call("dragon_hip_device_name", idx, buf, 256)
    return buf.value.decode()


def get_device_capability(device_index=None):
    """(major, minor) of the device's ISA version, (9, 5) for gfx950 (cuda.py:82-99)."""
    major, minor = ctypes.c_int(), ctypes.c_int()
    idx = current_device() if device_index is None else int(device_index)
    _call("dragon_hip_device_capability", idx, ctypes.byref(major), ctypes.byref(minor))
    return major.value, minor.value


def memory_allocated(device_index=None):
    """Bytes of device memory in use on the device (total minus free).

    ``dragon.cuda.memory_allocated`` reports the workspace pool's own bytes
    (cuda.py:146-169); this library keeps no pool, so the device-wide figure is
    the closest observable.
    """
    prev = current_device()
    if device_index is not None:
        set_device(device_index)
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    try:
        _call("dragon_hip_mem_info", ctypes.byref(free), ctypes.byref(total))
    finally:
        if device_index is not None:
            set_device(prev)
    return total.value - free.value


def set_default_device(device_index=0):
    """Make "hip:<index>" the default device; a negative index restores the CPU (cuda.py:212-233)."""
    if device_index < 0:
        _default.update(device_type="cpu", device_index=0)
    else:
        _default.update(device_type="hip", device_index=int(device_index))


def default_device():
    return dict(_default)


def set_random_seed(device_index=None, seed=3):
    """Record the seed of a device's generator (cuda.py:248-262). No kernel on
    this path draws random numbers; the value is kept for callers that query it."""
    _seeds[current_device() if device_index is None else int(device_index)] = int(seed)


def synchronize(device_index=None, stream_index=0):
    """Wait for all work on a device (cuda.py:265-277). ``stream_index`` selects a
    workspace stream in the reference; here every stream of the device is waited for."""
    prev = current_device()
    if device_index is not None:
        set_device(device_index)
    try:
        _call("dragon_hip_device_sync")
    finally:
        if device_index is not None:
            set_device(prev)
