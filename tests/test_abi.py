"""The C-ABI library builds, loads, and exports exactly what the headers under include/ declare
(dragon_hip.h, the boundary, and dragon_hip_testing.h, the hooks that exist for tests).

Runs without a GPU: no compute entry point is called."""

import ctypes
import os
import re

import pytest

from dragon_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in ("dragon_hip.h", "dragon_hip_testing.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(dragon_hip_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def handle():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return ctypes.CDLL(_lib.LIB_PATH)


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("dragon_hip_layer_norm", "dragon_hip_group_norm", "dragon_hip_group_norm_grad",
                 "dragon_hip_batch_norm", "dragon_hip_batch_norm_wgrad",
                 "dragon_hip_batch_norm_training_grad", "dragon_hip_batch_norm_inference_grad",
                 "dragon_hip_batch_norm_expectation", "dragon_hip_moments", "dragon_hip_inv_std",
                 "dragon_hip_axpby", "dragon_hip_softmax", "dragon_hip_log_softmax",
                 "dragon_hip_softmax_grad", "dragon_hip_log_softmax_grad"):
        assert must in names


def test_library_exports_every_declared_symbol(handle):
    missing = [n for n in declared_symbols() if not hasattr(handle, n)]
    assert not missing, missing


def test_python_signatures_cover_the_header():
    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_status_strings(handle):
    handle.dragon_hip_status_string.restype = ctypes.c_char_p
    assert handle.dragon_hip_status_string(0) == b"ok"
    assert b"dtype" in handle.dragon_hip_status_string(-2)
    assert b"scratch" in handle.dragon_hip_status_string(-3)


def test_argument_errors_need_no_device(handle):
    """Bad sizes / dtypes are rejected on the host before anything is enqueued."""
    lib = _lib.lib()
    one = ctypes.c_void_p(16)
    assert lib.dragon_hip_layer_norm(2, -1, 8, 1e-5, one, one, one, one, one, one, None) == -1
    assert lib.dragon_hip_layer_norm(2, 4, 0, 1e-5, one, one, one, one, one, one, None) == -1
    assert lib.dragon_hip_layer_norm(2, 0, 8, 1e-5, None, None, None, None, None, None, None) == 0
    assert lib.dragon_hip_softmax(2, 0, 1, 8, None, None, None, 0, None) == 0
    assert lib.dragon_hip_softmax(2, 4, 1, 0, one, one, None, 0, None) == -1
    assert lib.dragon_hip_group_norm(2, 2, 2, 2, 2, 7, one, one, one, one, one, one, None) == -1
    assert lib.dragon_hip_batch_norm_training_grad(2, 1 << 20, 1 << 10, 1 << 10, 1.0, 0, one, one,
                                                   one, one, one, one, one, one, None) == -1


def test_scratch_queries_need_no_device():
    lib = _lib.lib()
    dims = (ctypes.c_int64 * 3)(64, 256, 3136)
    axes = (ctypes.c_int64 * 2)(0, 2)
    assert lib.dragon_hip_moments_scratch_bytes(2, 3, dims, 2, axes) > 0
    assert lib.dragon_hip_batch_norm_reduce_scratch_bytes(2, 64, 256, 3136, 0) > 0
    assert lib.dragon_hip_group_norm_grad_scratch_bytes(1, 8192, 1, 12288, 1, 1) > 0
    assert lib.dragon_hip_batch_norm_reduce_scratch_bytes(2, 0, 256, 3136, 0) == 0


def test_exchange_plan_never_has_more_slices_than_workgroups():
    """The K slices of a reduction unit must sit in K different workgroups of a grid that is
    resident at once, or a workgroup would wait for an item it holds itself. Sweeps channel /
    group / row sizes up to the largest the planner accepts, for both tensor counts."""
    from dragon_amd import kernels as K
    rows = 0
    for dtype, vec in (("float32", 4), ("bfloat16", 8), ("float64", 2)):
        for tensors in (1, 2):
            packets_per_unit = 64
            while packets_per_unit * vec < (1 << 31):
                for nseg in (1, 48, 768):
                    seglen = max(16, packets_per_unit // nseg) * vec
                    units = max(1, min(64, ((1 << 31) - 1) // (nseg * seglen)))
                    plan = K.exchange_plan(dtype, units, nseg, seglen, tensors)
                    if plan is None:
                        continue
                    slices, slice_packets, per_thread, grid = plan
                    rows += 1
                    assert 1 <= slices <= grid, (dtype, tensors, nseg, seglen, plan)
                    assert slices * slice_packets >= nseg * (seglen // vec)
                    assert per_thread <= (16 if tensors == 1 else 12)
                    assert slice_packets % 64 == 0 and slice_packets <= per_thread * 256
                packets_per_unit = packets_per_unit * 5 // 4 + 1
    assert rows > 300
    # the two shapes whose plans once exceeded the backward grid of 768 workgroups
    for shape in ((4, 768, 112 * 112), (3, 48, 448 * 448)):
        plan = K.exchange_plan("float32", shape[0], shape[1], shape[2], 2)
        assert plan is None or plan[0] <= plan[3]
