"""Routing guard (no GPU): which kernels every BASELINE config and every bench.py
workload is sent to, asked of the library itself through dragon_hip_plan_name (the entry
point run in a plan-only mode that launches nothing) and compared with the pinned text
in tests/golden/plan_names.json. A changed size / alignment predicate that moves one of
these shapes to a multi-pass fallback fails here, not only in a benchmark.
tests/golden/make_plan_names.py rewrites the file after a routing change that is meant."""
import json
import os

import pytest

from dragon_amd import kernels as K
from tests.plan_cases import CASES

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
with open(os.path.join(ROOT, "tests", "golden", "plan_names.json")) as f:
    GOLDEN = json.load(f)

# kernels of the multi-pass general paths: none of the pinned shapes may take them ...
FALLBACKS = ("map_flat", "reduce2_", "_looped", "channel_pair_sums", "group_grad_from_channel_sums",
             "layer_norm_wide_row_sums", "softmax_columns", "reduce_gather")
# ... except where the multi-pass path was measured to be the faster one: the backward of
# channels-last GroupNorm samples beyond one workgroup (five passes; the sliced form was slower)
MULTI_PASS_BY_CHOICE = {("group_norm_bf16_32x64x64x512_g32_nhwc", "group_norm_grad")}


def _key(op, dt, dims, layout):
    return "%s %s %s %s" % (op, dt, "x".join(str(d) for d in dims), layout)


@pytest.mark.parametrize("workload", sorted(CASES))
def test_routing_is_the_pinned_one(workload):
    assert workload in GOLDEN, "run tests/golden/make_plan_names.py"
    for op, dt, dims, layout in CASES[workload]:
        text = K.plan_name(op, dt, dims, layout)
        assert text, (workload, op)
        assert text == GOLDEN[workload][_key(op, dt, dims, layout)], (workload, op, text)
        if (workload, op) in MULTI_PASS_BY_CHOICE:
            assert any(name in text for name in FALLBACKS), (workload, op, text)
            continue
        for name in FALLBACKS:
            assert name not in text, (workload, op, text)


def test_every_bench_workload_is_pinned():
    import bench
    assert set(bench.WORKLOADS) <= set(CASES), sorted(set(bench.WORKLOADS) - set(CASES))


def test_single_read_paths_of_the_baseline_configs():
    """cfg3 / cfg4 in so many words: BatchNorm through the slice exchange (16 slices per
    channel forward, 18 backward), GroupNorm with the group in one workgroup's registers."""
    fwd = K.plan_name("batch_norm_training_forward", "float32", (64, 256, 3136), "NCHW")
    bwd = K.plan_name("batch_norm_training_backward", "float32", (64, 256, 3136), "NCHW")
    assert fwd.startswith("slices=16:") and "channel_slices<" in fwd
    assert bwd.startswith("slices=18:") and "channel_slices<" in bwd
    assert K.plan_name("group_norm_forward", "bfloat16", (32, 32, 16, 4096), "NCHW").startswith(
        "group_norm_forward_items<16,512>:")
    assert K.plan_name("group_norm_grad", "bfloat16", (32, 32, 16, 4096), "NCHW").startswith(
        "group_norm_grad_rows<1024,8,waves>:")


def test_fallbacks_are_reported_as_such():
    """The guard sees a fallback when there is one: NHWC BatchNorm is the split path."""
    text = K.plan_name("batch_norm_training_forward", "float32", (64, 256, 3136), "NHWC")
    assert "reduce2_" in text and "map_flat" in text


def test_unknown_op_and_bad_shape_are_errors():
    with pytest.raises(ValueError):
        K.plan_name("no_such_op", "float32", (4, 4))
    with pytest.raises(ValueError):
        K.plan_name("layer_norm", "float32", (4, 0))
