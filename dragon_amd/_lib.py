"""Loads ``libdragon_hip.so`` (the C ABI of include/dragon_hip.h) with ctypes."""

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdragon_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float
_sz = ctypes.c_size_t
_i64p = ctypes.POINTER(ctypes.c_int64)

# name -> (restype, argtypes): exactly the declarations of include/dragon_hip.h.
SIGNATURES = {
    "dragon_hip_status_string": (ctypes.c_char_p, [_int]),
    "dragon_hip_device_count": (_int, [ctypes.POINTER(_int)]),
    "dragon_hip_set_device": (_int, [_int]),
    "dragon_hip_get_device": (_int, [ctypes.POINTER(_int)]),
    "dragon_hip_device_name": (_int, [_int, ctypes.c_char_p, _sz]),
    "dragon_hip_device_capability": (_int, [_int, ctypes.POINTER(_int), ctypes.POINTER(_int)]),
    "dragon_hip_device_sync": (_int, []),
    "dragon_hip_mem_info": (_int, [ctypes.POINTER(_sz), ctypes.POINTER(_sz)]),
    "dragon_hip_stream_create": (_int, [ctypes.POINTER(_vp)]),
    "dragon_hip_stream_destroy": (_int, [_vp]),
    "dragon_hip_stream_sync": (_int, [_vp]),
    "dragon_hip_stream_query": (_int, [_vp, ctypes.POINTER(_int)]),
    "dragon_hip_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "dragon_hip_free": (_int, [_vp]),
    "dragon_hip_host_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "dragon_hip_host_free": (_int, [_vp]),
    "dragon_hip_memset_async": (_int, [_vp, _int, _sz, _vp]),
    "dragon_hip_memcpy_async": (_int, [_vp, _vp, _sz, _int, _vp]),
    "dragon_hip_event_create": (_int, [ctypes.POINTER(_vp)]),
    "dragon_hip_event_destroy": (_int, [_vp]),
    "dragon_hip_event_record": (_int, [_vp, _vp]),
    "dragon_hip_event_sync": (_int, [_vp]),
    "dragon_hip_event_elapsed_ms": (_int, [_vp, _vp, ctypes.POINTER(_f32)]),
    "dragon_hip_inv_std": (_int, [_int, _i64, _f32, _vp, _vp, _vp]),
    "dragon_hip_axpby": (_int, [_int, _i64, _f32, _vp, _f32, _vp, _vp]),
    "dragon_hip_copy": (_int, [_int, _i64, _vp, _vp, _vp]),
    "dragon_hip_set": (_int, [_int, _i64, _f32, _vp, _vp]),
    "dragon_hip_square": (_int, [_int, _i64, _vp, _vp, _vp]),
    "dragon_hip_sub": (_int, [_int, _i64, _vp, _vp, _vp, _vp]),
    "dragon_hip_moments_scratch_bytes": (_sz, [_int, _int, _i64p, _int, _i64p]),
    "dragon_hip_moments": (_int, [_int, _int, _i64p, _int, _i64p, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_reduce_scratch_bytes": (_sz, [_int, _int, _i64p, _int, _i64p]),
    "dragon_hip_reduce_sum": (_int, [_int, _int, _i64p, _int, _i64p, _f32, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_reduce_sum_sqr": (_int, [_int, _int, _i64p, _int, _i64p, _f32, _vp, _vp, _vp, _sz,
                                         _vp]),
    "dragon_hip_reduce_l1": (_int, [_int, _int, _i64p, _int, _i64p, _f32, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_layer_norm": (_int, [_int, _i64, _i64, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dragon_hip_group_norm": (_int, [_int, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp,
                                     _vp, _vp]),
    "dragon_hip_group_norm_grad_scratch_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _int]),
    "dragon_hip_group_norm_grad": (_int, [_int, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp,
                                          _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_batch_norm_reduce_scratch_bytes": (_sz, [_int, _i64, _i64, _i64, _int]),
    "dragon_hip_batch_norm_expectation": (_int, [_int, _i64, _i64, _i64, _f32, _int, _vp, _vp, _vp,
                                                 _vp, _sz, _vp]),
    "dragon_hip_batch_norm": (_int, [_int, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp, _vp,
                                     _vp, _vp, _vp]),
    "dragon_hip_batch_norm_wgrad": (_int, [_int, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp,
                                           _vp, _vp, _sz, _vp]),
    "dragon_hip_batch_norm_training_grad": (_int, [_int, _i64, _i64, _i64, _f32, _int, _vp, _vp,
                                                   _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dragon_hip_batch_norm_inference_grad": (_int, [_int, _i64, _i64, _i64, _int, _vp, _vp, _vp,
                                                    _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_softmax_scratch_bytes": (_sz, [_int, _i64, _i64, _i64]),
    "dragon_hip_softmax": (_int, [_int, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_log_softmax": (_int, [_int, _i64, _i64, _i64, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_softmax_grad": (_int, [_int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_log_softmax_grad": (_int, [_int, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_l1_norm": (_int, [_int, _i64, _i64, _i64, _f32, _f32, _vp, _vp, _vp]),
    "dragon_hip_l2_norm": (_int, [_int, _i64, _i64, _i64, _f32, _f32, _vp, _vp, _vp]),
    "dragon_hip_l1_norm_grad": (_int, [_int, _i64, _i64, _i64, _f32, _f32, _vp, _vp, _vp, _vp]),
    "dragon_hip_l2_norm_grad": (_int, [_int, _i64, _i64, _i64, _f32, _f32, _vp, _vp, _vp, _vp]),
    "dragon_hip_cross_entropy": (_int, [_int, _i64, _vp, _vp, _vp, _vp]),
    "dragon_hip_sparse_cross_entropy": (_int, [_int, _int, _i64, _i64, _i64, _i64, _vp, _vp, _vp,
                                               _vp, _vp]),
    "dragon_hip_softmax_cross_entropy_grad": (_int, [_int, _int, _i64, _i64, _i64, _i64, _vp, _vp,
                                                     _vp, _vp, _vp]),
    "dragon_hip_reduce_loss_scratch_bytes": (_sz, [_int]),
    "dragon_hip_reduce_loss": (_int, [_int, _i64, _i64, _f32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_reduce_loss_grad": (_int, [_int, _i64, _i64, _f32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_broadcast_loss_grad": (_int, [_int, _i64, _i64, _i64, _vp, _vp, _vp]),
    "dragon_hip_softmax_cross_entropy_loss_scratch_bytes": (_sz, [_int, _i64, _i64, _i64]),
    "dragon_hip_softmax_cross_entropy_loss_forward": (_int, [_int, _int, _i64, _i64, _i64, _i64,
                                                             _int, _vp, _vp, _vp, _vp, _vp, _sz,
                                                             _vp]),
    "dragon_hip_softmax_cross_entropy_loss_backward": (_int, [_int, _int, _i64, _i64, _i64, _i64,
                                                              _int, _vp, _vp, _vp, _vp, _vp, _sz,
                                                              _vp]),
    "dragon_hip_group_norm_forward_scratch_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _int]),
    "dragon_hip_group_norm_forward": (_int, [_int, _i64, _i64, _i64, _i64, _int, _f32, _vp, _vp,
                                             _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dragon_hip_batch_norm_training_forward": (_int, [_int, _i64, _i64, _i64, _int, _f32, _f32,
                                                      _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                                      _vp, _sz, _vp]),
    "dragon_hip_batch_norm_training_backward": (_int, [_int, _i64, _i64, _i64, _f32, _int, _vp, _vp,
                                                       _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz,
                                                       _vp]),
    "dragon_hip_batch_norm_training_forward_noalloc": (_int, [_int, _i64, _i64, _i64, _int, _f32,
                                                              _f32, _vp, _vp, _vp, _vp, _vp, _vp,
                                                              _vp, _vp, _vp, _vp]),
    "dragon_hip_exchange_timed_out": (_int, []),
    "dragon_hip_exchange_reset": (None, [ctypes.c_uint]),
    "dragon_hip_exchange_plan": (_int, [_int, _i64, _i64, _i64, _int] + [ctypes.POINTER(_int)] * 4),
    "dragon_hip_group_norm_grad_timeline": (_int, [_int, _i64, _i64, _i64, _i64, _int] + [_vp] * 11 +
                                            [_sz, _vp, _sz, _vp]),
    "dragon_hip_plan_name": (_int, [ctypes.c_char_p, _int, _int, ctypes.POINTER(_i64), _int,
                                    ctypes.c_char_p, _sz]),
    "dragon_hip_stream_probe": (_int, [_int, _vp, _vp, _sz, _vp]),
    "dragon_hip_stream_probe_persistent": (_int, [_int, _int, _int, _int, _int, _int, _vp, _vp, _sz, _vp]),
    "dragon_hip_stream_probe_shape": (_int, [_int, _int, _int, _vp, _vp, _sz, _vp]),
}

_lib = None


def build(jobs=8):
    """Compile every HIP source for gfx950 into ``dragon_amd/lib/libdragon_hip.so``."""
    subprocess.check_call(["make", "-C", CSRC_DIR, "-j%d" % jobs, "-s"])


def lib():
    """The loaded library with argument types set; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)" % LIB_PATH)
        # torch ships its own HIP runtime and is the source of every device
        # pointer: import it first so this library binds to that same runtime
        # (one process must not hold two copies of libamdhip64).
        import torch  # noqa: F401
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


class DragonHipError(RuntimeError):
    """A non-zero status from the C ABI (the reference would LOG(FATAL) here)."""

    def __init__(self, fn, status):
        text = lib().dragon_hip_status_string(status)
        super().__init__("%s failed: status %d (%s)" % (fn, status, text.decode() if text else "?"))
        self.status = status


def check(fn, status):
    if status != 0:
        raise DragonHipError(fn, status)
