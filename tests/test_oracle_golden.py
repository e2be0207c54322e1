"""Pins the CPU oracle (oracle/ref_cpu.cc) without the reference being runnable.

Each check is one that a plausible restatement mistake would fail:
* the literal arrays the reference's own unit tests hold (tests/golden/),
* the numpy closed forms those tests spell out (BatchNorm, Moments),
* exhaustive 16-bit conversion checks against numpy / a bit-level model,
* fp64 brute force on small random inputs, and
* identities (GroupNorm with G=1,S=1 is LayerNorm; LogSoftmax = log(Softmax)).
"""

import json
import os

import numpy as np
import pytest

from oracle import ref_cpu as R

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_test_vectors.json")) as f:
    GOLD = json.load(f)


def arange(shape, start=0, dtype="float32"):
    return np.arange(start, start + int(np.prod(shape)), dtype=dtype).reshape(shape)


def maxabs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))))


# ---------------------------------------------------------------- conversions

def test_half_conversion_exhaustive_against_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    widened = R.from_bits(bits, "float16")
    expect = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(expect)
    assert np.array_equal(np.isnan(widened), nan)
    assert np.array_equal(widened[~nan], expect[~nan])
    # round trip of every finite value is the identity
    back = R.to_bits(widened[~nan], "float16")
    assert np.array_equal(back, bits[~nan])


def test_half_rounding_against_numpy_random():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 100,
        rng.standard_normal(200000).astype(np.float32) * 1e-5,  # subnormal range
        np.array([65504, 65519.99, 65520, 7e4, -7e4, 5.96e-8, 2.98e-8, 2.9802325e-8,
                  0.0, -0.0, np.inf, -np.inf], np.float32),
    ])
    got = R.to_bits(vals, "float16")
    with np.errstate(over="ignore"):
        expect = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, expect)


def test_bfloat16_rounding_bit_model():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        np.array([1.0, 1.00390625, 1.01171875, 3.3895314e38, -0.0, np.inf], np.float32),
    ])
    got = R.to_bits(vals, "bfloat16")
    u = vals.view(np.uint32).astype(np.uint64)
    expect = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(got, expect)
    # ties go to even: 1 + 2^-8 is exactly half-way between 1.0 and 1 + 2^-7
    assert R.to_bits(np.array([1.00390625], np.float32), "bfloat16")[0] == 0x3F80
    assert R.to_bits(np.array([1.01171875], np.float32), "bfloat16")[0] == 0x3F82
    assert R.to_bits(np.array([np.nan], np.float32), "bfloat16")[0] == 0x7FFF
    wid = R.from_bits(got, "bfloat16")
    assert np.array_equal(wid.view(np.uint32), got.astype(np.uint32) << 16)


# ---------------------------------------------------------------- softmax

@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_softmax_reference_literals(dtype):
    g = GOLD["softmax"]
    data = np.array(g["probs"], np.float32)
    x = np.log(data).astype(dtype)
    y = R.op_softmax(dtype, x)
    dx = R.op_softmax_grad(dtype, y, x)
    assert maxabs(y, data) <= g["prec"]
    assert maxabs(dx, g["dx_with_dy_eq_x"]) <= g["prec"]


@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_log_softmax_reference_literals(dtype):
    g = GOLD["log_softmax"]
    data = np.array(g["probs"], np.float32)
    x = np.log(data).astype(dtype)
    y = R.op_softmax(dtype, x, log=True)
    dx = R.op_softmax_grad(dtype, y, x, log=True)
    assert maxabs(y, x) <= g["prec"]
    assert maxabs(dx, g["dx_with_dy_eq_x"]) <= g["prec"]


@pytest.mark.parametrize("shape,axis", [((5, 7), -1), ((3, 6, 4), 1), ((2, 3, 4, 5), 2),
                                        ((4, 1), -1), ((1, 9, 1), 1)])
def test_softmax_strided_axis_vs_fp64_bruteforce(shape, axis):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis, keepdims=True))
    y64 = e / e.sum(axis, keepdims=True)
    y = R.op_softmax("float32", x, axis)
    ly = R.op_softmax("float32", x, axis, log=True)
    assert maxabs(y, y64) < 1e-6
    assert maxabs(ly, np.log(y64)) < 1e-5
    dx64 = (dy - (dy * y64).sum(axis, keepdims=True)) * y64
    assert maxabs(R.op_softmax_grad("float32", y, dy, axis), dx64) < 1e-6
    ldx64 = dy - y64 * dy.astype(np.float64).sum(axis, keepdims=True)
    assert maxabs(R.op_softmax_grad("float32", ly, dy, axis, log=True), ldx64) < 1e-5
    # invariants: rows sum to one, softmax gradients sum to zero
    assert maxabs(y.sum(axis), 1.0) < 1e-6
    assert maxabs(R.op_softmax_grad("float32", y, dy, axis).sum(axis), 0.0) < 1e-6


def test_softmax_in_place_and_masked():
    x = np.array([[0.0, -1e4, 1.0, -1e4]], np.float32)
    y = R.op_softmax("float32", x)
    assert y[0, 1] == 0.0 and y[0, 3] == 0.0
    assert abs(y[0, 0] + y[0, 2] - 1.0) < 1e-7


# ---------------------------------------------------------------- layer norm

def _ln_inputs(g):
    x_shape = tuple(g["x_shape"])
    w_shape = (x_shape[-1],)
    data1 = arange(x_shape) * 0.1
    data2, data3 = arange(w_shape, 1) * 0.1, arange(w_shape) * 0.1
    data6 = arange(x_shape) * g["dy_scale"]
    return data1, data2, data3, data6


def test_layer_norm_reference_literals():
    g = GOLD["layer_norm"]
    x, w, b, dy = _ln_inputs(g)
    y, mu, rsig = R.op_layer_norm("float32", x, w, b, g["axis"], g["eps"])
    dx, dw, db = R.op_layer_norm_grad("float32", x, w, dy, mu, rsig, g["axis"])
    mean = x.mean(1, keepdims=True)
    sig = np.sqrt(x.var(1, keepdims=True) + g["eps"])
    result = (x - mean) / sig
    assert maxabs(y, result * w + b) <= g["prec"]
    assert maxabs(dx, g["dx"]) <= g["prec"]
    assert maxabs(dw, (dy * result).sum(0)) <= g["prec"]
    assert maxabs(db, dy.sum(0)) <= g["prec"]


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_layer_norm_vs_fp64_bruteforce(dtype):
    rng = np.random.default_rng(7)
    N, C = 13, 257
    x = R.to_bits(rng.standard_normal((N, C)).astype(np.float32) * 2 + 0.3, dtype)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    y, mu, rsig = R.op_layer_norm(dtype, x, g, b, -1, 1e-5)
    xf = R.from_bits(x, dtype).astype(np.float64)
    m = xf.mean(1)
    r = 1 / np.sqrt(xf.var(1) + np.float64(np.float32(1e-5)))
    y64 = (xf - m[:, None]) * r[:, None] * g + b
    tol = {"float16": 2e-3, "bfloat16": 1.6e-2, "float32": 2e-6, "float64": 1e-12}[dtype]
    assert maxabs(mu, m) < 1e-5 and maxabs(rsig, r) < 1e-5
    assert maxabs(R.from_bits(y, dtype), y64) / np.abs(y64).max() < tol


def test_layer_norm_grad_is_group_norm_grad_identity_and_fp64():
    rng = np.random.default_rng(8)
    N, C = 9, 33
    x = rng.standard_normal((N, C)).astype(np.float32)
    dy = rng.standard_normal((N, C)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = np.zeros(C, np.float32)
    _, mu, rsig = R.op_layer_norm("float32", x, g, b)
    dx, dg, db = R.op_layer_norm_grad("float32", x, g, dy, mu, rsig)
    # autograd-free closed form in fp64
    x64, dy64, g64 = x.astype(np.float64), dy.astype(np.float64), g.astype(np.float64)
    m = x64.mean(1, keepdims=True)
    r = 1 / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
    xh = (x64 - m) * r
    gdy = dy64 * g64
    dx64 = r * (gdy - gdy.mean(1, keepdims=True) - xh * (gdy * xh).mean(1, keepdims=True))
    assert maxabs(dx, dx64) < 2e-5
    assert maxabs(dg, (dy64 * xh).sum(0)) < 2e-5
    assert maxabs(db, dy64.sum(0)) < 2e-5
    # invariants: dx is orthogonal to 1 and to x_hat within a row
    assert np.abs(dx.astype(np.float64).sum(1)).max() < 1e-4
    assert np.abs((dx * xh).sum(1)).max() < 5e-4


# ---------------------------------------------------------------- group / instance norm

def _gn_case(case, dy_scale, eps):
    x_shape, w_shape = tuple(case["x_shape"]), tuple(case["w_shape"])
    axis, group, axes = case["axis"], case["group"], tuple(case["axes"])
    data1 = arange(x_shape) * 0.1
    data2, data3 = arange(w_shape, 1) * 0.1, arange(w_shape) * 0.1
    data6 = arange(x_shape) * dy_scale
    new_shape = list(x_shape)
    new_shape[axis] //= group
    new_shape.insert(axis, group)
    r = data1.reshape(new_shape)
    mean = r.mean(axes, keepdims=True)
    sig = np.sqrt(r.var(axes, keepdims=True) + eps)
    result = ((r - mean) / sig).reshape(x_shape)
    red = tuple(i for i in range(len(x_shape)) if w_shape[i - len(x_shape) + len(w_shape)] == 1) \
        if len(w_shape) == len(x_shape) else tuple(range(len(x_shape) - 1))
    grad2 = (data6 * result).sum(red).flatten()
    grad3 = data6.sum(red).flatten()
    return data1, data2.flatten(), data3.flatten(), data6, result * data2 + data3, grad2, grad3


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_group_norm_reference_literals(idx):
    g = GOLD["group_norm"]
    case = g["cases"][idx]
    x, w, b, dy, y_exp, dw_exp, db_exp = _gn_case(case, g["dy_scale"], g["eps"])
    y, mu, rsig = R.op_group_norm("float32", x, w, b, case["axis"], case["group"], g["eps"])
    dx, dw, db = R.op_group_norm_grad("float32", x, w, dy, mu, rsig, case["axis"], case["group"])
    assert maxabs(y, y_exp) <= g["prec"]
    assert maxabs(dx, case["dx"]) <= g["prec"]
    assert maxabs(dw, dw_exp) <= g["prec"]
    assert maxabs(db, db_exp) <= g["prec"]


@pytest.mark.parametrize("idx", [0, 1, 2])
def test_instance_norm_reference_literals(idx):
    g = GOLD["instance_norm"]
    case = g["cases"][idx]
    x, w, b, dy, y_exp, dw_exp, db_exp = _gn_case(case, g["dy_scale"], g["eps"])
    y, mu, rsig = R.op_group_norm("float32", x, w, b, case["axis"], 0, g["eps"])
    dx, dw, db = R.op_group_norm_grad("float32", x, w, dy, mu, rsig, case["axis"], 0)
    assert maxabs(y, y_exp) <= g["prec"]
    assert maxabs(dw, dw_exp) <= g["prec"]
    assert maxabs(db, db_exp) <= g["prec"]
    if idx > 0:  # listed in the reference test (not asserted there); D*S=1 for idx 0
        assert maxabs(dx, case["dx"]) <= 2e-3


@pytest.mark.parametrize("layout_axis", [1, -1])
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_group_norm_vs_fp64_bruteforce(layout_axis, dtype):
    rng = np.random.default_rng(11)
    N, C, H, G = 3, 12, 5, 4
    shape = (N, C, H) if layout_axis == 1 else (N, H, C)
    x = rng.standard_normal(shape).astype(dtype)
    dy = rng.standard_normal(shape).astype(dtype)
    w = rng.uniform(0.5, 1.5, C).astype(dtype)
    b = rng.standard_normal(C).astype(dtype)
    y, mu, rsig = R.op_group_norm(dtype, x, w, b, layout_axis, G, 1e-5)
    dx, dw, db = R.op_group_norm_grad(dtype, x, w, dy, mu, rsig, layout_axis, G)
    # fp64 closed form on [N, G, D, S]
    x64 = x.astype(np.float64) if layout_axis == 1 else np.moveaxis(x.astype(np.float64), -1, 1)
    dy64 = dy.astype(np.float64) if layout_axis == 1 else np.moveaxis(dy.astype(np.float64), -1, 1)
    xg = x64.reshape(N, G, C // G, H)
    dg_ = dy64.reshape(N, G, C // G, H)
    wg = w.astype(np.float64).reshape(1, G, C // G, 1)
    m = xg.mean((2, 3), keepdims=True)
    r = 1 / np.sqrt(xg.var((2, 3), keepdims=True) + np.float64(np.float32(1e-5)))
    xh = (xg - m) * r
    gdy = dg_ * wg
    dx64 = r * (gdy - gdy.mean((2, 3), keepdims=True) - xh * (gdy * xh).mean((2, 3), keepdims=True))
    y64 = (xh * wg + b.astype(np.float64).reshape(1, G, C // G, 1)).reshape(N, C, H)
    dx64 = dx64.reshape(N, C, H)
    if layout_axis == -1:
        y64, dx64 = np.moveaxis(y64, 1, -1), np.moveaxis(dx64, 1, -1)
    tol = 3e-5 if dtype == "float32" else 1e-11
    assert maxabs(y, y64) < tol and maxabs(dx, dx64) < tol
    assert maxabs(dw, (dg_ * xh).sum((0, 3)).flatten()) < tol
    assert maxabs(db, dg_.sum((0, 3)).flatten()) < tol


# ---------------------------------------------------------------- batch norm

@pytest.mark.parametrize("idx", range(5))
@pytest.mark.parametrize("use_stats", [0, 1])
def test_batch_norm_reference_closed_forms(idx, use_stats):
    g = GOLD["batch_norm"]
    case = g["cases"][idx]
    eps = g["eps"]
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
    y_exp = result * d2 + d3
    w, b = data2.flatten(), data3.flatten()
    rm, rv = data4.flatten().copy(), data5.flatten().copy()
    if use_stats == 0:
        y, mu, rsig, _ = R.op_batch_norm_train("float32", data1, w, b, rm, rv, axis, 0.9, eps)
        dx, dw, db = R.op_batch_norm_train_grad("float32", data1, w, data6, mu, rsig, axis)
        # running statistics: closed form with the BIASED batch variance
        m = np.float32(0.9)
        assert maxabs(rm, m * data4.flatten() + (1 - m) * data1.mean(axes)) < 1e-6
        assert maxabs(rv, m * data5.flatten() + (1 - m) * data1.var(axes)) < 1e-5
    else:
        y = R.op_batch_norm_infer("float32", data1, w, b, rm, rv, axis, eps)
        dx, dw, db = R.op_batch_norm_infer_grad("float32", data1, w, rm, rv, data6, axis, eps)
        assert np.array_equal(rm, data4.flatten()) and np.array_equal(rv, data5.flatten())
    assert maxabs(y, y_exp) <= g["prec"]
    assert maxabs(dx, grad1) <= g["prec"]
    assert maxabs(dw, grad2.flatten()) <= g["prec"]
    assert maxabs(db, grad3.flatten()) <= g["prec"]


def test_batch_norm_aliasing_conventions():
    """scale==rsig selects the 3C inference buffer, dgamma==nullptr skips WGrad."""
    import ctypes
    rng = np.random.default_rng(3)
    N, C, S = 2, 3, 4
    x = rng.standard_normal((N, C, S)).astype(np.float32)
    mu = rng.standard_normal(C).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, C).astype(np.float32)
    beta = rng.standard_normal(C).astype(np.float32)
    params = np.zeros(3 * C, np.float32)
    params[:C] = rng.uniform(0.5, 2, C)
    rsig = params[:C].copy()
    y = np.empty_like(x)
    p = lambda a: ctypes.c_void_p(a.ctypes.data)
    st = R.lib().ref_batch_norm(2, ctypes.c_int64(N), ctypes.c_int64(C), ctypes.c_int64(S), 0,
                                p(x), p(mu), p(params), p(gamma), p(beta), p(params), p(params), p(y))
    assert st == 0
    assert np.array_equal(params[:C], rsig)
    assert np.allclose(params[C:2 * C], gamma * rsig, rtol=1e-6)
    assert np.allclose(params[2 * C:], beta - gamma * rsig * mu, rtol=1e-5, atol=1e-6)
    assert np.allclose(y, x * (gamma * rsig)[None, :, None] + (beta - gamma * rsig * mu)[None, :, None],
                       rtol=1e-5, atol=1e-6)
    dx, dg, db = R.batch_norm_inference_grad("float32", N, C, S, "NCHW", x, mu, rsig, gamma, x,
                                             want_wgrad=False)
    assert dg is None and np.allclose(dx, x * (gamma * rsig)[None, :, None], rtol=1e-6)


def test_batch_norm_expectation_closed_form():
    rng = np.random.default_rng(4)
    for layout, shape in (("NCHW", (3, 5, 7)), ("NHWC", (3, 7, 5))):
        x = rng.standard_normal(shape).astype(np.float32)
        N, C, S = (3, 5, 7)
        ex, ex2 = R.batch_norm_expectation("float32", N, C, S, float(N * S), layout, x)
        red = (0, 2) if layout == "NCHW" else (0, 1)
        assert maxabs(ex, x.astype(np.float64).mean(red)) < 1e-6
        assert maxabs(ex2, (x.astype(np.float64) ** 2).mean(red)) < 1e-6


def test_unsupported_dtypes_are_rejected_like_the_reference_cpu():
    x = np.zeros((2, 2), np.uint16)
    with pytest.raises(RuntimeError):
        R.batch_norm("float16", 2, 2, 1, "NCHW", x, [0, 0], [1, 1], [1, 1], [0, 0])
    with pytest.raises(RuntimeError):
        R.group_norm_grad("bfloat16", 2, 1, 2, 1, "NHWC", x, [0, 0], [1, 1], [1, 1], x)


# ---------------------------------------------------------------- moments

@pytest.mark.parametrize("axes", GOLD["moments"]["axes"])
def test_moments_reference_closed_form(axes):
    data = arange(tuple(GOLD["moments"]["x_shape"]))
    mean, var = R.moments("float32", data, axes)
    assert maxabs(mean, data.mean(tuple(axes)).flatten()) <= GOLD["moments"]["prec"]
    assert maxabs(var, data.var(tuple(axes)).flatten()) <= GOLD["moments"]["prec"]


@pytest.mark.parametrize("shape,axes", [
    ((4, 5, 6), (0, 2)),      # generic: BatchNorm NCHW
    ((20, 5), (0,)),          # row-wise: BatchNorm NHWC
    ((6, 35), (1,)),          # col-wise: GroupNorm NCHW
    ((3, 4, 2, 5), (1, 3)),   # generic: GroupNorm NHWC
    ((3, 1, 4, 1, 5), (2, 4)),
    ((2, 3, 4), (0, 1, 2)),
])
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32", "float64"])
def test_moments_layouts_vs_numpy(shape, axes, dtype):
    rng = np.random.default_rng(12)
    x = R.to_bits((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32), dtype)
    xf = R.from_bits(x, dtype).astype(np.float64)
    mean, var = R.moments(dtype, x, axes)
    assert maxabs(mean, xf.mean(axes).flatten()) < 1e-5
    assert maxabs(var, xf.var(axes).flatten()) < 2e-5


def test_inv_std_and_axpby_closed_forms():
    rng = np.random.default_rng(13)
    v = rng.uniform(0.1, 4, 257).astype(np.float32)
    r = R.inv_std(v, 1e-5)
    assert np.max(np.abs(r / (1 / np.sqrt(v.astype(np.float64) + 1e-5)) - 1)) < 2e-7
    x = rng.standard_normal(257).astype(np.float32)
    y0 = rng.standard_normal(257).astype(np.float32)
    y = y0.copy()
    R.axpby(0.1, x, 0.9, y)
    # exactly: round(round(0.9f*y) + round(0.1f*x))
    expect = (np.float32(0.9) * y0).astype(np.float32) + (np.float32(0.1) * x).astype(np.float32)
    assert np.array_equal(y, expect.astype(np.float32))


# ---------------------------------------------------------------- lp norm

@pytest.mark.parametrize("idx", range(4))
@pytest.mark.parametrize("dtype", ["float32", "float64"])
def test_lp_norm_reference_literals(idx, dtype):
    g = GOLD["lp_norm"]
    e = g["entries"][idx]
    data1 = arange(tuple(g["x_shape"])).astype(dtype)
    data2 = (arange(tuple(g["x_shape"])) / 10 + 1).astype(dtype)
    y = R.op_lp_norm(dtype, data1, e["axis"], None, e["p"], e["eps"], e["reduction"])
    dx = R.op_lp_norm_grad(dtype, data1, data2, e["axis"], None, e["p"], e["eps"], e["reduction"])
    norm = np.abs(data1) if e["p"] == 1 else np.square(data1)
    norm = norm.sum() if e["reduction"] == "sum" else norm.mean()
    norm = norm if e["p"] == 1 else np.sqrt(norm)
    assert maxabs(y, data1 / max(norm, e["eps"])) <= g["prec"]
    assert maxabs(dx, e["dx"]) <= g["prec"]


@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("reduction", ["sum", "mean"])
@pytest.mark.parametrize("shape,axis,end_axis", [((5, 7), -1, None), ((3, 6, 4), 1, None),
                                                 ((2, 3, 4, 5), 1, 2), ((4, 1), -1, None)])
def test_lp_norm_vs_fp64_bruteforce(p, reduction, shape, axis, end_axis):
    rng = np.random.default_rng(11)
    x = rng.standard_normal(shape).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    eps = 1e-12
    a = axis % len(shape)
    b = a if end_axis is None else end_axis
    red = tuple(range(a, b + 1))
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    n = float(np.prod([shape[i] for i in red])) if reduction == "mean" else 1.0
    if p == 1:
        norm = np.maximum(np.abs(x64).sum(red, keepdims=True) / n, eps)
        dx64 = dy64 / norm - np.sign(x64) * ((dy64 * x64).sum(red, keepdims=True) / n) / norm ** 2
    else:
        norm = np.maximum(np.sqrt(np.square(x64).sum(red, keepdims=True) / n), eps)
        dx64 = dy64 / norm - x64 * ((dy64 * x64).sum(red, keepdims=True) / n) / norm ** 3
    y = R.op_lp_norm("float32", x, axis, end_axis, p, eps, reduction)
    dx = R.op_lp_norm_grad("float32", x, dy, axis, end_axis, p, eps, reduction)
    scale = float(np.max(np.abs(dy64 / norm)))  # size of the terms that cancel in dx
    assert maxabs(y, x64 / norm) < 2e-6 * (float(np.max(np.abs(x64 / norm))) + 1e-30)
    assert maxabs(dx, dx64) < 5e-6 * scale


def test_lp_norm_epsilon_clamp_and_zero_rows():
    x = np.zeros((2, 4), np.float32)
    x[1] = [3.0, -4.0, 0.0, 0.0]
    dy = np.ones((2, 4), np.float32)
    y = R.op_lp_norm("float32", x, -1, None, 2, 0.5, "sum")
    assert np.all(y[0] == 0.0)                       # 0 / max(0, eps)
    assert maxabs(y[1], x[1] / 5.0) < 1e-7
    dx = R.op_lp_norm_grad("float32", x, dy, -1, None, 2, 0.5, "sum")
    assert maxabs(dx[0], dy[0] / 0.5) < 1e-7          # sum == 0: second term vanishes
    # d/dx of x/|x| is orthogonal to x when dy is parallel to x
    dxp = R.op_lp_norm_grad("float32", x[1:], x[1:].copy(), -1, None, 2, 1e-12, "sum")
    assert maxabs(dxp, 0.0) < 1e-6


# ---------------------------------------------------------------- reduce sums

REDUCE_CASES = [((2, 3, 3), (0,)), ((2, 3, 3), (1,)), ((2, 3, 3), (1, 2)), ((2, 3, 3), (0, 1, 2)),
                ((4, 5, 6, 7), (1, 3)), ((4, 5, 6, 7), (0, 2)), ((3, 1, 5), (1,)), ((7,), (0,)),
                ((6, 5), (0,)), ((2, 3, 4, 5), (0, 3))]


@pytest.mark.parametrize("kind", ["sum", "sum_sqr", "l1"])
@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("shape,axes", REDUCE_CASES)
def test_reduce_sum_against_numpy(shape, axes, dtype, kind):
    # the reference's own reduce tests compare with numpy (test_ops.py:4047-4073 for sum)
    if shape == (2, 3, 3):
        data = arange(shape).astype(dtype) - 4
    else:
        data = np.random.default_rng(21).standard_normal(shape).astype(dtype)
    f = {"sum": lambda v: v, "sum_sqr": np.square, "l1": np.abs}[kind]
    for scale in (1.0, 0.25):
        want = f(data.astype(np.float64)).sum(axes) * scale
        got = R.reduce_sum(dtype, data, list(axes), scale, kind)
        assert got.shape == (want.size,)
        tol = 1e-12 if dtype == "float64" else 2e-6
        assert maxabs(got, want.ravel()) <= tol * max(1.0, float(np.max(np.abs(want))))


def test_reduce_sum_rejects_16_bit_like_the_reference_cpu():
    x = np.zeros(4, np.uint16)
    with pytest.raises(RuntimeError):
        R.reduce_sum("float16", x, [0])


# ---------------------------------------------------------------- softmax cross-entropy loss

def _sce_numpy(x, target, dl, axis, ignore_index, reduction):
    """fp64 closed form of the operator pair for class-index targets."""
    x64 = np.moveaxis(np.asarray(x, np.float64), axis, -1)
    e = np.exp(x64 - x64.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    tgt = np.asarray(target)
    valid = tgt != ignore_index if ignore_index is not None else np.ones(tgt.shape, bool)
    safe = np.where(valid, tgt, 0)
    picked = np.take_along_axis(p, safe[..., None], -1)[..., 0]
    loss = np.where(valid, -np.log(np.maximum(picked, np.finfo(np.float32).tiny)), 0.0)
    onehot = np.zeros_like(p)
    np.put_along_axis(onehot, safe[..., None], 1.0, -1)
    g = (p - onehot) * valid[..., None]
    r = reduction.lower()
    if r == "none":
        return loss, np.moveaxis(g * np.asarray(dl, np.float64)[..., None], -1, axis)
    n = {"sum": 1.0, "mean": float(tgt.size), "batch_mean": float(x.shape[0]),
         "valid": float(valid.sum())}[r]
    return loss.sum() / max(n, 1.0), np.moveaxis(g * float(dl) / max(n, 0.5), -1, axis)


@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("target_kind", ["int32", "int64", "dense"])
def test_softmax_cross_entropy_loss_reference_closed_form(dtype, target_kind):
    g = GOLD["softmax_cross_entropy_loss"]
    data1 = np.log(np.array(g["probs"], "float32")).astype(dtype)
    data2 = np.array(g["target"], "int32")
    data3 = np.eye(3, dtype=dtype)[data2]
    tgt = data3 if target_kind == "dense" else data2.astype(target_kind)
    for reduction in g["reductions"]:
        scale = (np.exp(data1) - data3) / (data1.shape[0] if reduction == "mean" else 1)
        picked = -data1[np.arange(2), data2]
        result = {"mean": picked.mean(), "sum": picked.sum(), "none": picked}[reduction]
        loss, prob = R.op_softmax_cross_entropy_loss(dtype, data1, tgt, reduction=reduction)
        data4 = arange(loss.shape, 2).astype(dtype)
        dx = R.op_softmax_cross_entropy_loss_grad(dtype, prob, tgt, data4, reduction=reduction)
        assert maxabs(loss, result) <= g["prec"]
        assert maxabs(dx, np.expand_dims(data4, -1) * scale) <= g["prec"]


@pytest.mark.parametrize("reduction", ["none", "sum", "mean", "batch_mean", "valid"])
@pytest.mark.parametrize("shape,axis", [((6, 7), -1), ((3, 5, 4), 1), ((2, 4, 3, 3), 1)])
def test_softmax_cross_entropy_loss_ignore_index_vs_fp64(shape, axis, reduction):
    rng = np.random.default_rng(31)
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    C = shape[axis]
    tshape = tuple(d for i, d in enumerate(shape) if i != axis % len(shape))
    target = rng.integers(0, C, tshape).astype(np.int64)
    target.ravel()[::3] = 255                                  # ignored positions
    loss, prob = R.op_softmax_cross_entropy_loss("float32", x, target, axis, 255, reduction)
    dl = rng.standard_normal(tshape).astype(np.float32) if reduction == "none" else np.float32(1.7)
    dx = R.op_softmax_cross_entropy_loss_grad("float32", prob, target, np.asarray(dl, np.float32),
                                              axis, 255, reduction)
    want_loss, want_dx = _sce_numpy(x, target, dl, axis % len(shape), 255, reduction)
    assert maxabs(loss, want_loss) <= 2e-6 * max(1.0, float(np.max(np.abs(want_loss))))
    assert maxabs(dx, want_dx) <= 2e-6 * max(1.0, float(np.max(np.abs(want_dx))))


def test_softmax_cross_entropy_loss_all_ignored_is_zero():
    x = np.zeros((3, 4), np.float32)
    target = np.full(3, 9, np.int32)
    loss, prob = R.op_softmax_cross_entropy_loss("float32", x, target, -1, 9, "valid")
    assert float(loss) == 0.0                                   # sum 0 / max(0, 1)
    dx = R.op_softmax_cross_entropy_loss_grad("float32", prob, target, np.float32(1), -1, 9, "valid")
    assert np.all(dx == 0)
