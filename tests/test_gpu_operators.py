"""Operator-level parity on the GPU, written the way the reference tests its
operators (test/dragon/test_ops.py): feed tensors, run the operator through
Workspace::RunOperator on the HIP device, take gradients through the gradient
definitions, and compare with the literal arrays and numpy closed forms the
reference holds. Everything below the Python test goes through the C++ host
layer and the C ABI into the gfx950 kernels.

The second half runs the BASELINE configurations at full size and checks them
against the CPU oracle and against size-independent properties.
"""

import json
import os

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests import util as U

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_test_vectors.json")) as f:
    GOLD = json.load(f)


@pytest.fixture(scope="module")
def rt():
    import torch
    assert torch.cuda.is_available()
    from dragon_amd import runtime
    return runtime


@pytest.fixture()
def ws(rt):
    w = rt.Workspace("ops_test")
    yield w
    w.close()


def arange(shape, start=0, dtype="float32"):
    return np.arange(start, start + int(np.prod(shape)), dtype=dtype).reshape(shape)


def assert_equal(got, want, prec=1e-5):
    """OpTestCase.assertEqual: max absolute error <= prec (test_ops.py:41-95)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.max(np.abs(got - want)) <= prec if got.size else True


# ---------------------------------------------------------------- reference test bodies

def test_softmax(rt, ws):
    g = GOLD["softmax"]
    data = np.array(g["probs"], "float32")
    tape = rt.Tape(ws)
    x = ws.feed("x", np.log(data))
    y = rt.softmax(tape, [x])
    (dx,) = tape.gradient(y, [x], output_gradient=x)
    assert_equal(ws.fetch(y), data, g["prec"])
    assert_equal(ws.fetch(dx), g["dx_with_dy_eq_x"], g["prec"])


def test_log_softmax(rt, ws):
    g = GOLD["log_softmax"]
    data1 = np.array(g["probs"], "float32")
    data2 = np.log(data1)
    tape = rt.Tape(ws)
    x = ws.feed("x", data2)
    y = rt.log_softmax(tape, [x])
    (dx,) = tape.gradient(y, [x], output_gradient=x)
    assert_equal(ws.fetch(y), data2, g["prec"])
    assert_equal(ws.fetch(dx), g["dx_with_dy_eq_x"], g["prec"])


def test_lp_norm(rt, ws):
    g = GOLD["lp_norm"]
    for e in g["entries"]:
        data1, data2 = arange((6,)), arange((6,)) / 10 + 1
        tape = rt.Tape(ws)
        x, dy = ws.feed("x", data1), ws.feed("dy", data2)
        y = rt.lp_norm(tape, [x], e["axis"], p=e["p"], epsilon=e["eps"], reduction=e["reduction"])
        (dx,) = tape.gradient(y, [x], output_gradient=dy)
        norm = np.abs(data1) if e["p"] == 1 else np.square(data1)
        norm = norm.sum() if e["reduction"] == "sum" else norm.mean()
        norm = norm if e["p"] == 1 else np.sqrt(norm)
        assert_equal(ws.fetch(y), data1 / max(norm, e["eps"]), g["prec"])
        assert_equal(ws.fetch(dx), e["dx"], g["prec"])


def test_lp_norm_axis_range_and_bad_order(rt, ws):
    rng = np.random.default_rng(3)
    data = rng.standard_normal((3, 4, 5, 6)).astype("float32")
    x = ws.feed("x", data)
    tape = rt.Tape(ws)
    y = rt.lp_norm(tape, [x], axis=1, end_axis=2, p=2, reduction="mean")
    norm = np.sqrt(np.square(data.astype(np.float64)).mean((1, 2), keepdims=True))
    assert_equal(ws.fetch(y), data / norm, 1e-5)
    with pytest.raises(rt.DragonError, match="Unsupported order"):
        ws.run_operator(rt.make_def("LpNorm", [x], ["y_bad"], p=3))


def test_softmax_cross_entropy_loss(rt, ws):
    g = GOLD["softmax_cross_entropy_loss"]
    for reduction in g["reductions"]:
        data1 = np.log(np.array(g["probs"], "float32"))
        data2 = np.array(g["target"], "int32")
        data3 = np.eye(3, dtype="float32")[data2]
        scale = (np.exp(data1) - data3) / (data1.shape[0] if reduction == "mean" else 1)
        picked = -data1[np.arange(2), data2]
        result = {"mean": picked.mean(), "sum": picked.sum(), "none": picked}[reduction]
        for target in (data2, data2.astype("int64"), data3):
            tape = rt.Tape(ws)
            x, y = ws.feed("x", data1), ws.feed("y", target)
            loss = rt.softmax_cross_entropy_loss(tape, [x, y], reduction=reduction)
            data4 = arange(np.shape(result), 2)
            dl = ws.feed("dl", data4)
            (dx,) = tape.gradient(loss, [x], output_gradient=dl)
            assert_equal(ws.fetch(loss), result, g["prec"])
            assert_equal(ws.fetch(dx), np.expand_dims(data4, -1) * scale, g["prec"])


def test_softmax_cross_entropy_loss_ignore_index_axis_and_valid(rt, ws):
    rng = np.random.default_rng(8)
    data = rng.standard_normal((4, 6, 5)).astype("float32")
    target = rng.integers(0, 6, (4, 5)).astype("int64")
    target[0, :] = 255
    for reduction in ("valid", "batch_mean", "mean", "sum", "none"):
        tape = rt.Tape(ws)
        x, y = ws.feed("x", data), ws.feed("y", target)
        loss = rt.softmax_cross_entropy_loss(tape, [x, y], axis=1, ignore_index=255,
                                             reduction=reduction)
        want, prob = R.op_softmax_cross_entropy_loss("float32", data, target, 1, 255, reduction)
        assert_equal(ws.fetch(loss), want, 1e-5)
        dl_np = (rng.standard_normal((4, 5)).astype("float32") if reduction == "none"
                 else np.array(0.7, "float32"))
        dl = ws.feed("dl", dl_np)
        (dx,) = tape.gradient(loss, [x], output_gradient=dl)
        want_dx = R.op_softmax_cross_entropy_loss_grad("float32", prob, target, dl_np, 1, 255,
                                                       reduction)
        assert_equal(ws.fetch(dx), want_dx, 1e-6)
        assert np.all(ws.fetch(dx)[0] == 0)
    with pytest.raises(rt.DragonError, match="Numel of X and Y"):
        ws.run_operator(rt.make_def("SoftmaxCrossEntropyLoss", [ws.feed("x", data),
                                                                ws.feed("y", target[:2])], ["l"], axis=1))


def test_layer_norm(rt, ws):
    g = GOLD["layer_norm"]
    x_shape, w_shape = tuple(g["x_shape"]), (g["x_shape"][-1],)
    data1 = arange(x_shape) * 0.1
    data2, data3 = arange(w_shape, 1) * 0.1, arange(w_shape) * 0.1
    data6 = arange(x_shape) * g["dy_scale"]
    tape = rt.Tape(ws)
    x, w, b = ws.feed("x", data1), ws.feed("w", data2), ws.feed("b", data3)
    y = rt.layer_norm(tape, [x, w, b], axis=g["axis"], epsilon=g["eps"])
    dy = ws.feed("dy", data6)
    dx, dw, db = tape.gradient(y, [x, w, b], output_gradient=dy)
    mean = data1.mean(1, keepdims=True)
    sig = np.sqrt(data1.var(1, keepdims=True) + g["eps"])
    result = (data1 - mean) / sig
    assert_equal(ws.fetch(y), result * data2 + data3, g["prec"])
    assert_equal(ws.fetch(dx), g["dx"], g["prec"])
    assert_equal(ws.fetch(dw), (data6 * result).sum(0), g["prec"])
    assert_equal(ws.fetch(db), data6.sum(0), g["prec"])


def _group_case(case, dy_scale, eps):
    x_shape, w_shape = tuple(case["x_shape"]), tuple(case["w_shape"])
    axis, group, axes = case["axis"], case["group"], tuple(case["axes"])
    data1 = arange(x_shape) * 0.1
    data2, data3 = arange(w_shape, 1) * 0.1, arange(w_shape) * 0.1
    data6 = arange(x_shape) * dy_scale
    new_shape = list(x_shape)
    new_shape[axis] //= group
    new_shape.insert(axis, group)
    r = data1.reshape(new_shape)
    result = ((r - r.mean(axes, keepdims=True)) / np.sqrt(r.var(axes, keepdims=True) + eps)).reshape(x_shape)
    ch_axis = axis % len(x_shape)
    red = tuple(i for i in range(len(x_shape)) if i != ch_axis)
    return (data1, data2.flatten(), data3.flatten(), data6, result * data2 + data3,
            (data6 * result).sum(red), data6.sum(red))


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_group_norm(rt, ws, idx):
    g = GOLD["group_norm"]
    case = g["cases"][idx]
    data1, data2, data3, data6, result, grad2, grad3 = _group_case(case, g["dy_scale"], g["eps"])
    tape = rt.Tape(ws)
    x, w, b = ws.feed("x", data1), ws.feed("w", data2), ws.feed("b", data3)
    y = rt.group_norm(tape, [x, w, b], axis=case["axis"], group=case["group"], epsilon=g["eps"])
    dy = ws.feed("dy", data6)
    dx, dw, db = tape.gradient(y, [x, w, b], output_gradient=dy)
    assert_equal(ws.fetch(y), result, g["prec"])
    assert_equal(ws.fetch(dx), case["dx"], g["prec"])
    assert_equal(ws.fetch(dw), grad2, g["prec"])
    assert_equal(ws.fetch(db), grad3, g["prec"])


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_instance_norm(rt, ws, idx):
    g = GOLD["instance_norm"]
    case = g["cases"][idx]
    data1, data2, data3, data6, result, grad2, grad3 = _group_case(case, g["dy_scale"], g["eps"])
    tape = rt.Tape(ws)
    x, w, b = ws.feed("x", data1), ws.feed("w", data2), ws.feed("b", data3)
    y = rt.instance_norm(tape, [x, w, b], axis=case["axis"], epsilon=g["eps"])
    dy = ws.feed("dy", data6)
    dx, dw, db = tape.gradient(y, [x, w, b], output_gradient=dy)
    assert_equal(ws.fetch(y), result, g["prec"])
    assert_equal(ws.fetch(dw), grad2, g["prec"])
    assert_equal(ws.fetch(db), grad3, g["prec"])


@pytest.mark.parametrize("op_type", ["BatchNorm", "SyncBatchNorm"])
@pytest.mark.parametrize("use_stats", [0, 1])
@pytest.mark.parametrize("idx", range(5))
def test_batch_norm(rt, ws, idx, use_stats, op_type):
    g = GOLD["batch_norm"]
    case, eps = g["cases"][idx], g["eps"]
    x_shape, w_shape, axis = tuple(case["x_shape"]), tuple(case["w_shape"]), case["axis"]
    np.random.seed(1337)
    data1 = arange(x_shape) * 0.1
    data2, data3 = arange(w_shape, 1) * 0.1, arange(w_shape) * 0.1
    data4, data5 = arange(w_shape) * 0.1, arange(w_shape, 1) * 0.1
    data6 = np.random.uniform(-1.0, 1.0, size=x_shape).astype("float32")
    axes = list(range(len(x_shape)))
    axes.pop(axis)
    axes = tuple(axes)
    bshape = [1] * len(x_shape)
    bshape[axis] = x_shape[axis]
    d2, d3, d4, d5 = (d.reshape(bshape) for d in (data2, data3, data4, data5))
    tape = rt.Tape(ws)
    x = ws.feed("x", data1)
    w, b = ws.feed("w", data2.flatten()), ws.feed("b", data3.flatten())
    rm, rv = ws.feed("rm", data4.flatten()), ws.feed("rv", data5.flatten())
    y = rt.batch_norm(tape, [x, w, b, rm, rv], axis=axis, use_stats=use_stats, epsilon=eps,
                      op_type=op_type)
    if use_stats == 0:
        mean = data1.mean(axes, keepdims=True)
        sig = np.sqrt(data1.var(axes, keepdims=True) + eps)
        result = (data1 - mean) / sig
    else:
        sig = np.sqrt(d5 + eps)
        result = (data1 - d4) / sig
    grad2 = (data6 * result).sum(axes, keepdims=True)
    grad3 = data6.sum(axes, keepdims=True)
    if use_stats == 0:
        scale = 1.0 / float(np.prod([x_shape[i] for i in axes]))
        grad1 = (data6 - (result * grad2 + grad3) * scale) * d2 / sig
    else:
        grad1 = data6 * d2 / sig
    dy = ws.feed("dy", data6)
    dx, dw, db = tape.gradient(y, [x, w, b], output_gradient=dy)
    assert_equal(ws.fetch(y), result * d2 + d3, g["prec"])
    assert_equal(ws.fetch(dx), grad1, g["prec"])
    assert_equal(ws.fetch(dw), grad2.flatten(), g["prec"])
    assert_equal(ws.fetch(db), grad3.flatten(), g["prec"])
    if use_stats == 0:  # running statistics: momentum * old + (1 - momentum) * batch (biased variance)
        m = np.float32(0.9)
        assert_equal(ws.fetch(rm), m * data4.flatten() + (1 - m) * data1.mean(axes), 1e-6)
        assert_equal(ws.fetch(rv), m * data5.flatten() + (1 - m) * data1.var(axes), 1e-5)
    else:
        assert np.array_equal(ws.fetch(rm), data4.flatten())
        assert np.array_equal(ws.fetch(rv), data5.flatten())


def test_softmax_in_place_and_middle_axis(rt, ws):
    rng = np.random.default_rng(0)
    data = rng.standard_normal((3, 6, 5)).astype("float32")
    x = ws.feed("x", data)
    ws.run_operator(rt.make_def("Softmax", [x], [x], name="sm_inplace", axis=1))  # Y over X
    e = np.exp(data.astype(np.float64) - data.max(1, keepdims=True))
    assert_equal(ws.fetch(x), e / e.sum(1, keepdims=True), 1e-6)
    dy = ws.feed("dy", rng.standard_normal((3, 6, 5)).astype("float32"))
    y = ws.fetch(x).astype(np.float64)
    g = ws.fetch(dy).astype(np.float64)
    ws.run_operator(rt.make_def("SoftmaxGradient", [x, dy], [dy], name="sm_inplace_grad", axis=1))
    assert_equal(ws.fetch(dy), (g - (g * y).sum(1, keepdims=True)) * y, 1e-6)


def test_operator_cache_and_error_paths(rt, ws):
    data = np.random.default_rng(1).standard_normal((4, 8)).astype("float32")
    ws.feed("w", np.ones(8, "float32"))
    ws.feed("b", np.zeros(8, "float32"))
    for i in range(3):  # same cache_key: one operator object, rebound per call
        ws.feed("x%d" % i, data + i)
        ws.run_operator(rt.make_def("LayerNorm", ["x%d" % i, "w", "b"], ["y%d" % i], name="ln%d" % i,
                                    axis=-1, cache_key="LayerNorm/hip:0"))
        want = (data + i - (data + i).mean(1, keepdims=True)) / np.sqrt((data + i).var(1, keepdims=True) + 1e-5)
        assert_equal(ws.fetch("y%d" % i), want, 1e-5)
        assert ws.info("ln%d/X_mu" % i) == ("float32", (4,))
    # gamma of the wrong shape / dtype, bad axis, bad grouping: fatal with the reference's wording
    ws.feed("w_bad", np.ones(7, "float32"))
    with pytest.raises(rt.DragonError, match="dimensions"):
        ws.run_operator(rt.make_def("LayerNorm", ["x0", "w_bad", "b"], ["y"], axis=-1))
    ws.feed("w64", np.ones(8, "float64"))
    with pytest.raises(rt.DragonError, match="type of Tensor"):
        ws.run_operator(rt.make_def("LayerNorm", ["x0", "w64", "b"], ["y"], axis=-1))
    with pytest.raises(rt.DragonError, match="axis"):
        ws.run_operator(rt.make_def("Softmax", ["x0"], ["y"], axis=5))
    with pytest.raises(rt.DragonError, match="can not be split"):
        ws.run_operator(rt.make_def("GroupNorm", ["x0", "w", "b"], ["y"], axis=-1, group=3))
    ws.feed("xi", np.zeros((2, 8), np.int64))
    with pytest.raises(rt.DragonError, match="Unsupported type"):
        ws.run_operator(rt.make_def("Softmax", ["xi"], ["y"]))
    ws.feed("rm", np.zeros(8, "float32"))
    ws.feed("rv", np.ones(8, "float32"))
    with pytest.raises(rt.DragonError, match="collective backend"):
        ws.run_operator(rt.make_def("SyncBatchNorm", ["x0", "w", "b", "rm", "rv"], ["y"], axis=-1, comm=1))


# ---------------------------------------------------------------- BASELINE configurations

# Parameter gradients are fp32 quantities: held to the 1e-5 of the parity bar against the
# fp64 closed form, and to the oracle within the oracle's own distance from fp64 (its column
# sums are strictly sequential fp32 sums over up to 200704 terms).
TOL_DGAMMA = 1e-5


def _three_way(got, oracle, exact, tol, what):
    ok, e_go, e_ge, e_oe = U.close3(got, oracle, exact, tol)
    print("three-way %s: gpu-vs-oracle %.3g, gpu-vs-fp64 %.3g, oracle-vs-fp64 %.3g (tol %.0e)"
          % (what, e_go, e_ge, e_oe, tol))
    assert ok, "%s: gpu-vs-oracle %.3g, gpu-vs-fp64 %.3g, oracle-vs-fp64 %.3g" % (what, e_go, e_ge, e_oe)


def test_config1_layer_norm_fp32_8192x1024(rt, ws):
    rng = np.random.default_rng(0)
    N, C = 8192, 1024
    x = rng.standard_normal((N, C), dtype=np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    ws.feed("x", x), ws.feed("w", g), ws.feed("b", b)
    ws.run_operator(rt.make_def("LayerNorm", ["x", "w", "b"], ["y"], name="cfg1", axis=-1, epsilon=1e-5))
    y_ref, mu_ref, rsig_ref = R.layer_norm("float32", x, g, b, 1e-5)
    assert U.normwise(ws.fetch("y"), y_ref) <= 1e-5
    assert U.normwise(ws.fetch("cfg1/X_mu"), mu_ref) <= 1e-5
    assert np.max(np.abs(ws.fetch("cfg1/X_rsig") / rsig_ref - 1)) <= 1e-5


def test_config2_softmax_fp16_16x32x512x512(rt, ws):
    rng = np.random.default_rng(1)
    shape = (16, 32, 512, 512)
    N, C = 16 * 32 * 512, 512
    x = rng.standard_normal((N, C), dtype=np.float32) * 3
    x[rng.random((N, C), dtype=np.float32) < 0.05] = -1e4
    xb = R.to_bits(x, "float16")
    del x
    dyb = R.to_bits(rng.standard_normal((N, C), dtype=np.float32), "float16")
    tape = rt.Tape(ws)
    xn = ws.feed("x", xb.reshape(shape), dtype="float16")
    y = rt.softmax(tape, [xn], axis=-1)
    dy = ws.feed("dy", dyb.reshape(shape), dtype="float16")
    (dx,) = tape.gradient(y, [xn], output_gradient=dy)
    yb = ws.fetch(y, raw=True).reshape(N, C)
    dxb = ws.fetch(dx, raw=True).reshape(N, C)
    # parity with the fp32 CPU kernels on the fp16-rounded inputs; backward uses the fp16 y
    # the forward produced. 59% of the outputs are fp16 subnormals: errors are per row,
    # relative to the row's largest value.
    y_ref = R.softmax("float32", N, 1, C, R.from_bits(xb, "float16"))
    yw = R.from_bits(yb, "float16")
    assert U.rowwise_normwise(yw, y_ref) <= 1e-2
    dx_ref = R.softmax_grad("float32", N, 1, C, R.from_bits(dyb, "float16"), yw)
    dxw = R.from_bits(dxb, "float16")
    assert U.rowwise_normwise(dxw, dx_ref) <= 1e-2
    # properties: masked logits give exact zeros, rows sum to one, gradients sum to zero
    assert np.all(yw[R.from_bits(xb, "float16") == -1e4] == 0)
    assert np.max(np.abs(yw.sum(1, dtype=np.float64) - 1)) < 5e-3
    assert np.max(np.abs(dxw.sum(1, dtype=np.float64))) < 2e-2


def test_config3_batch_norm_fp32_64x256x56x56(rt, ws):
    rng = np.random.default_rng(2)
    shape = (64, 256, 56, 56)
    C = 256
    x = 2 * rng.standard_normal(shape, dtype=np.float32) + 0.5
    dyv = rng.standard_normal(shape, dtype=np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    tape = rt.Tape(ws)
    xn, w, bb = ws.feed("x", x), ws.feed("w", g), ws.feed("b", b)
    rm, rv = ws.feed("rm", np.zeros(C, np.float32)), ws.feed("rv", np.ones(C, np.float32))
    y = rt.batch_norm(tape, [xn, w, bb, rm, rv], axis=1, momentum=0.9, epsilon=1e-5, use_stats=0)
    dy = ws.feed("dy", dyv)
    dx, dw, db = tape.gradient(y, [xn, w, bb], output_gradient=dy)
    # oracle (sequential fp32 sums over 200704 terms: itself ~5e-5 off fp64) and fp64 closed forms
    rm_ref, rv_ref = np.zeros(C, np.float32), np.ones(C, np.float32)
    y_ref, mu_ref, rsig_ref, _ = R.op_batch_norm_train("float32", x, g, b, rm_ref, rv_ref, 1, 0.9, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_train_grad("float32", x, g, dyv, mu_ref, rsig_ref, 1)
    x64 = x.astype(np.float64)
    mu64 = x64.mean((0, 2, 3))
    var64 = x64.var((0, 2, 3))
    rsig64 = 1 / np.sqrt(var64 + 1e-5)
    name = y.split("/")[0]
    _three_way(ws.fetch(name + "/X_mu"), mu_ref, mu64, 1e-5, "mu")
    _three_way(ws.fetch(name + "/X_rsig"), rsig_ref, rsig64, 1e-5, "rsig")
    _three_way(ws.fetch(rm), rm_ref, 0.1 * mu64, 1e-5, "running_mean")
    _three_way(ws.fetch(rv), rv_ref, 0.9 + 0.1 * var64, 1e-5, "running_var")
    xh64 = (x64 - mu64[None, :, None, None]) * rsig64[None, :, None, None]
    y64 = xh64 * g[None, :, None, None] + b[None, :, None, None]
    _three_way(ws.fetch(y), y_ref, y64, 1e-5, "y")
    dy64 = dyv.astype(np.float64)
    dg64 = (dy64 * xh64).sum((0, 2, 3))
    db64 = dy64.sum((0, 2, 3))
    _three_way(ws.fetch(dw), dg_ref, dg64, TOL_DGAMMA, "dgamma")
    _three_way(ws.fetch(db), db_ref, db64, TOL_DGAMMA, "dbeta")
    n = 64 * 56 * 56
    dx64 = (g * rsig64)[None, :, None, None] * (
        dy64 - (xh64 * dg64[None, :, None, None] + db64[None, :, None, None]) / n)
    dxg = ws.fetch(dx)
    _three_way(dxg, dx_ref, dx64, 1e-5, "dx")
    # property: the input gradient of a batch-normalised channel sums to zero
    assert np.max(np.abs(dxg.sum((0, 2, 3), dtype=np.float64))) < 5e-2


def test_config4_group_norm_bf16_32x512x64x64(rt, ws):
    rng = np.random.default_rng(3)
    shape, G = (32, 512, 64, 64), 32
    C = 512
    xb = R.to_bits(rng.standard_normal(shape, dtype=np.float32), "bfloat16")
    dyb = R.to_bits(rng.standard_normal(shape, dtype=np.float32), "bfloat16")
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    tape = rt.Tape(ws)
    xn, w, bb = ws.feed("x", xb, dtype="bfloat16"), ws.feed("w", g), ws.feed("b", b)
    y = rt.group_norm(tape, [xn, w, bb], axis=1, group=G, epsilon=1e-5)
    dy = ws.feed("dy", dyb, dtype="bfloat16")
    dx, dw, db = tape.gradient(y, [xn, w, bb], output_gradient=dy)
    y_ref, mu_ref, rsig_ref = R.op_group_norm("bfloat16", xb, g, b, 1, G, 1e-5)
    name = y.split("/")[0]
    x64 = U.widen(xb, "bfloat16").reshape(32, G, -1)
    _three_way(ws.fetch(name + "/X_mu").ravel(), mu_ref, x64.mean(2).ravel(), 1e-5, "mu")
    _three_way(ws.fetch(name + "/X_rsig").ravel(), rsig_ref, (1 / np.sqrt(x64.var(2) + 1e-5)).ravel(),
               1e-5, "rsig")
    assert U.normwise(U.widen(ws.fetch(y), "bfloat16"), U.widen(y_ref, "bfloat16")) <= 1e-2
    # the reference's CPU has no bf16 GroupNormGrad: fp32 kernel on the widened inputs
    dx_ref, dg_ref, db_ref = R.op_group_norm_grad(
        "float32", R.from_bits(xb, "bfloat16"), g, R.from_bits(dyb, "bfloat16"), mu_ref, rsig_ref, 1, G)
    assert U.normwise(U.widen(ws.fetch(dx), "bfloat16"), dx_ref) <= 1e-2
    # dgamma / dbeta are fp32 sums of 131072 terms per channel: three-way against fp64
    dy64 = U.widen(dyb, "bfloat16").reshape(32, G, -1)
    xh64 = (x64 - x64.mean(2, keepdims=True)) / np.sqrt(x64.var(2, keepdims=True) + 1e-5)
    dg64 = (dy64 * xh64).reshape(32, C, -1).sum((0, 2))
    db64 = dy64.reshape(32, C, -1).sum((0, 2))
    _three_way(ws.fetch(dw), dg_ref, dg64, TOL_DGAMMA, "dgamma")
    _three_way(ws.fetch(db), db_ref, db64, TOL_DGAMMA, "dbeta")


@pytest.mark.parametrize("shape", [(8192, 12288), (65536, 1000)])
def test_config5_layer_norm_bf16(rt, ws, shape):
    rng = np.random.default_rng(4)
    N, C = shape
    x = rng.standard_normal(shape, dtype=np.float32)
    x[rng.random(shape, dtype=np.float32) < 0.01] *= 50
    xb = R.to_bits(x, "bfloat16")
    del x
    dyb = R.to_bits(rng.standard_normal(shape, dtype=np.float32), "bfloat16")
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    tape = rt.Tape(ws)
    xn, w, bb = ws.feed("x", xb, dtype="bfloat16"), ws.feed("w", g), ws.feed("b", b)
    y = rt.layer_norm(tape, [xn, w, bb], axis=-1, epsilon=1e-5)
    dy = ws.feed("dy", dyb, dtype="bfloat16")
    dx, dw, db = tape.gradient(y, [xn, w, bb], output_gradient=dy)
    y_ref, mu_ref, rsig_ref = R.layer_norm("bfloat16", xb, g, b, 1e-5)
    name = y.split("/")[0]
    x64 = U.widen(xb, "bfloat16")
    _three_way(ws.fetch(name + "/X_mu"), mu_ref, x64.mean(1), 1e-5, "mu")
    _three_way(ws.fetch(name + "/X_rsig"), rsig_ref, 1 / np.sqrt(x64.var(1) + 1e-5), 1e-5, "rsig")
    del x64
    assert U.normwise(U.widen(ws.fetch(y), "bfloat16"), U.widen(y_ref, "bfloat16")) <= 1e-2
    dx_ref, dg_ref, db_ref, _, _ = R.group_norm_grad(
        "float32", N, 1, C, 1, "NHWC", R.from_bits(xb, "bfloat16"), mu_ref, rsig_ref, g,
        R.from_bits(dyb, "bfloat16"))
    dxw = U.widen(ws.fetch(dx), "bfloat16")
    assert U.normwise(dxw, dx_ref) <= 1e-2
    # dgamma / dbeta: sequential fp32 column sums over N rows in the oracle
    dy64 = U.widen(dyb, "bfloat16")
    _three_way(ws.fetch(db), db_ref, dy64.sum(0), TOL_DGAMMA, "dbeta")
    x64 = U.widen(xb, "bfloat16")
    xh64 = (x64 - x64.mean(1, keepdims=True)) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    _three_way(ws.fetch(dw), dg_ref, (dy64 * xh64).sum(0), TOL_DGAMMA, "dgamma")
    del x64, xh64
    # property: each row of dx is orthogonal to the all-ones vector (up to bf16 rounding of dx)
    assert np.max(np.abs(dxw.sum(1))) < 0.05 * np.sqrt(C)
