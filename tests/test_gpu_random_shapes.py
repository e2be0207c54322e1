"""Seeded random shapes around the widths at which the launchers switch kernels (rows of one
packet per lane, the LDS-staged short rows, 256- and 1024-thread tiles, raw-packet tiles,
the looped and the sliced kernels; channel rows that are or are not whole packets), with
odd row counts, every I/O type and tensors that start a few elements past a 16-byte
boundary. The checker is the defining formula in fp64 (numpy), which the oracle itself is
pinned against; tolerances as in tests/util.py. Every output lies in a poisoned buffer whose
surroundings must come back untouched."""

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests import util as U

pytestmark = pytest.mark.gpu

DTYPES = ("float32", "bfloat16", "float16")
EDGES = (8, 32, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 65536, 131072)
GUARD = 16
POISON = -7.0


@pytest.fixture(scope="module")
def K():
    import torch
    assert torch.cuda.is_available()
    from dragon_amd import kernels
    return kernels


def _row_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        edge = int(rng.choice(EDGES))
        C = max(1, edge + int(rng.integers(-9, 10)) * int(rng.choice((1, 1, 8))))
        N = int(rng.integers(1, max(2, min(48, 1_500_000 // C))))
        dtype = DTYPES[int(rng.integers(0, 3))]
        sx = int(rng.choice((0, 0, 0, 1, 3, 4)))
        sy = sx if rng.random() < 0.7 else int(rng.choice((0, 2, 5)))
        cases.append((N, C, dtype, sx, sy, 1000 + i))
    return cases


def _held(n, dtype, shift, bits=None):
    """A poisoned buffer and the view of n elements that starts `shift` elements into it."""
    import torch
    buf = torch.full((n + shift + GUARD,), POISON, dtype=U.torch_dtype(dtype), device="cuda")
    view = buf[shift:shift + n]
    if bits is not None:
        view.copy_(U.to_device(np.ascontiguousarray(bits).ravel(), dtype))
    return buf, view


def _untouched(buf, dtype, shift, n):
    flat = U.widen(U.to_host(buf), dtype).ravel()
    return bool(np.all(flat[:shift] == POISON) and np.all(flat[shift + n:] == POISON))


def _mean_ok(got, want, x):
    """A mean of values that nearly cancel is held to the scale of the values, not of the mean."""
    err = np.max(np.abs(np.asarray(got, np.float64).ravel() - np.asarray(want).ravel()))
    return err <= 2e-5 * (np.max(np.abs(want)) + np.sqrt(np.mean(np.asarray(x) ** 2)))


def _values(rng, shape, dtype, scale=1.0):
    bits = R.to_bits((rng.standard_normal(shape) * scale).astype(np.float32), dtype)
    return bits, U.widen(bits, dtype).reshape(shape)


@pytest.mark.parametrize("N,C,dtype,sx,sy,seed", _row_cases(60, 1))
def test_softmax_rows(K, N, C, dtype, sx, sy, seed):
    rng = np.random.default_rng(seed)
    log = bool(seed & 1)
    xb, x = _values(rng, (N, C), dtype, 3.0)
    dyb, dy = _values(rng, (N, C), dtype)
    e = np.exp(x - x.max(1, keepdims=True))
    p = e / e.sum(1, keepdims=True)
    y_ref = np.log(p) if log else p
    _, xd = _held(N * C, dtype, sx, xb)
    ybuf, yd = _held(N * C, dtype, sy)
    (K.log_softmax if log else K.softmax)(N, 1, C, xd, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, C)
    if log:
        assert np.max(np.abs(y - y_ref) / (1 + np.abs(y_ref))) <= U.TIGHT[dtype]
    else:
        assert U.rowwise_normwise(y, y_ref) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, sy, N * C)
    # backward from the forward's own (rounded) output, as the operator graph does
    _, dyd = _held(N * C, dtype, sx, dyb)
    _, yin = _held(N * C, dtype, sx, U.to_host(yd.contiguous()))
    dxbuf, dxd = _held(N * C, dtype, sy)
    (K.log_softmax_grad if log else K.softmax_grad)(N, 1, C, dyd, yin, dxd)
    dx = U.widen(U.to_host(dxd.contiguous()), dtype).reshape(N, C)
    dx_ref = (dy - np.exp(y) * dy.sum(1, keepdims=True)) if log else \
        (dy - (dy * y).sum(1, keepdims=True)) * y
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert _untouched(dxbuf, dtype, sy, N * C)


@pytest.mark.parametrize("N,C,dtype,sx,sy,seed", _row_cases(60, 2))
def test_layer_norm_rows(K, N, C, dtype, sx, sy, seed):
    import torch
    rng = np.random.default_rng(seed)
    xb, x = _values(rng, (N, C), dtype, 2.0)
    dyb, dy = _values(rng, (N, C), dtype)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    eps = 1e-5
    mean = x.mean(1, keepdims=True)
    var = ((x - mean) ** 2).mean(1, keepdims=True)
    rs = 1 / np.sqrt(var + np.float64(np.float32(eps)))
    xh = (x - mean) * rs
    y_ref = xh * g + b
    _, xd = _held(N * C, dtype, sx, xb)
    ybuf, yd = _held(N * C, dtype, sy)
    gd, bd = torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda()
    mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    K.layer_norm(N, C, eps, xd, gd, bd, mu, rsig, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, C)
    assert _mean_ok(mu.cpu().numpy(), mean, x)
    assert np.max(np.abs(rsig.cpu().numpy().astype(np.float64) / rs.ravel() - 1)) <= 2e-5
    assert U.normwise(y, y_ref) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, sy, N * C)
    # backward = GroupNormGrad with one group and S = 1, from the kernel's own statistics
    m32 = mu.cpu().numpy().astype(np.float64)[:, None]
    r32 = rsig.cpu().numpy().astype(np.float64)[:, None]
    _, dyd = _held(N * C, dtype, sx, dyb)
    dxbuf, dxd = _held(N * C, dtype, sy)
    params = torch.empty(2 * N, device="cuda")
    dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    K.group_norm_grad(N, 1, C, 1, "NHWC", xd, mu, rsig, gd, dyd, params, params, dg, db, dxd)
    ds_ref = (g * dy * x).sum(1)
    db_ref = (g * dy).sum(1)
    u = (db_ref[:, None] * m32 - ds_ref[:, None]) * (x - m32) * r32 ** 3
    dx_ref = g * dy * r32 + (u - db_ref[:, None] * r32) / C
    dx = U.widen(U.to_host(dxd.contiguous()), dtype).reshape(N, C)
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(dg.cpu().numpy(), (dy * (x - m32) * r32).sum(0)) <= 2e-5
    assert U.normwise(db.cpu().numpy(), dy.sum(0)) <= 2e-5
    assert U.normwise(params[:N].cpu().numpy(), ds_ref) <= 2e-5
    assert U.normwise(params[N:].cpu().numpy(), db_ref) <= 2e-5
    assert _untouched(dxbuf, dtype, sy, N * C)


@pytest.mark.parametrize("N,C,dtype,sx,sy,seed", _row_cases(40, 3))
def test_l2_norm_rows(K, N, C, dtype, sx, sy, seed):
    rng = np.random.default_rng(seed)
    xb, x = _values(rng, (N, C), dtype)
    dyb, dy = _values(rng, (N, C), dtype)
    eps = 1e-12
    nrm = np.sqrt((x * x).sum(1, keepdims=True))
    nrm = np.maximum(nrm, eps)
    _, xd = _held(N * C, dtype, sx, xb)
    ybuf, yd = _held(N * C, dtype, sy)
    K.l2_norm(N, 1, C, 1.0, eps, xd, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, C)
    assert U.normwise(y, x / nrm) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, sy, N * C)
    _, dyd = _held(N * C, dtype, sx, dyb)
    dxbuf, dxd = _held(N * C, dtype, sy)
    K.l2_norm_grad(N, 1, C, 1.0, eps, dyd, xd, dxd)
    dx = U.widen(U.to_host(dxd.contiguous()), dtype).reshape(N, C)
    dx_ref = dy / nrm - x * (dy * x).sum(1, keepdims=True) / nrm ** 3
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert _untouched(dxbuf, dtype, sy, N * C)


def _channel_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        N = int(rng.integers(1, 7))
        G = int(rng.choice((1, 2, 4, 8)))
        D = int(rng.choice((1, 2, 3, 4, 16)))
        S = int(rng.choice((1, 7, 49, 64, 196, 200, 1024, 1030, 3136, 4099)))
        fmt = "NCHW" if rng.random() < 0.6 else "NHWC"
        dtype = DTYPES[int(rng.integers(0, 3))]
        cases.append((N, G, D, S, fmt, dtype, 2000 + i))
    return cases


def _as_ncs(a, N, C, S, fmt):
    """fp64 view [N, C, S] of a tensor stored in `fmt`."""
    return a.reshape(N, C, S) if fmt == "NCHW" else a.reshape(N, S, C).transpose(0, 2, 1)


@pytest.mark.parametrize("N,G,D,S,fmt,dtype,seed", _channel_cases(40, 4))
def test_group_norm_shapes(K, N, G, D, S, fmt, dtype, seed):
    import torch
    rng = np.random.default_rng(seed)
    C = G * D
    n = N * C * S
    xb, xs = _values(rng, (n,), dtype, 2.0)
    dyb, dys = _values(rng, (n,), dtype)
    x, dy = _as_ncs(xs, N, C, S, fmt), _as_ncs(dys, N, C, S, fmt)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    eps = 1e-5
    xg = x.reshape(N, G, D * S)
    mean = xg.mean(2)
    rs = 1 / np.sqrt(((xg - mean[..., None]) ** 2).mean(2) + np.float64(np.float32(eps)))
    mc, rc = np.repeat(mean, D, 1)[..., None], np.repeat(rs, D, 1)[..., None]
    y_ref = (x - mc) * rc * g[None, :, None] + b[None, :, None]
    _, xd = _held(n, dtype, 0, xb)
    ybuf, yd = _held(n, dtype, 0)
    gd, bd = torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda()
    mu, rsig = torch.empty(N * G, device="cuda"), torch.empty(N * G, device="cuda")
    K.group_norm_forward(N, G, D, S, fmt, eps, xd, gd, bd, mu, rsig, yd)
    y = _as_ncs(U.widen(U.to_host(yd.contiguous()), dtype), N, C, S, fmt)
    assert _mean_ok(mu.cpu().numpy(), mean, x)
    assert np.max(np.abs(rsig.cpu().numpy().astype(np.float64) / rs.ravel() - 1)) <= 5e-5
    assert U.normwise(y, y_ref) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, 0, n)
    m32 = np.repeat(mu.cpu().numpy().astype(np.float64).reshape(N, G), D, 1)[..., None]
    r32 = np.repeat(rsig.cpu().numpy().astype(np.float64).reshape(N, G), D, 1)[..., None]
    _, dyd = _held(n, dtype, 0, dyb)
    dxbuf, dxd = _held(n, dtype, 0)
    params = torch.empty(2 * N * G, device="cuda")
    dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    K.group_norm_grad(N, G, D, S, fmt, xd, mu, rsig, gd, dyd, params, params, dg, db, dxd)
    gc = g[None, :, None]
    ds_ref = (gc * dy * x).reshape(N, G, D * S).sum(2)
    db_ref = (gc * dy).reshape(N, G, D * S).sum(2)
    dsc, dbc = np.repeat(ds_ref, D, 1)[..., None], np.repeat(db_ref, D, 1)[..., None]
    dx_ref = gc * dy * r32 + ((dbc * m32 - dsc) * (x - m32) * r32 ** 3 - dbc * r32) / (D * S)
    dx = _as_ncs(U.widen(U.to_host(dxd.contiguous()), dtype), N, C, S, fmt)
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(dg.cpu().numpy(), (dy * (x - m32) * r32).sum((0, 2))) <= 5e-5
    assert U.normwise(db.cpu().numpy(), dy.sum((0, 2))) <= 5e-5
    assert _untouched(dxbuf, dtype, 0, n)


# NHWC samples cut into slices of whole rows: one row at a time per workgroup and many, idle
# threads (C / packet does not divide 256), a last slice of fewer rows than a workgroup holds at
# a time, fewer and more slices than groups, more items than resident workgroups, one group,
# x at an address that is not 16-byte aligned (another path, same answer), in place.
NHWC_SLICE_CASES = [
    (1, 1, 8, 70001, "bfloat16", 0), (2, 4, 48, 1537, "float32", 0), (1, 200, 8, 301, "bfloat16", 0),
    (3, 25, 8, 2049, "float16", 0), (1, 256, 8, 700, "bfloat16", 0), (40, 8, 16, 2304, "float32", 0),
    (2, 32, 16, 4097, "bfloat16", 0), (2, 32, 16, 4097, "bfloat16", 3), (5, 3, 8, 6000, "float16", 0),
    (2, 2, 256, 1030, "float32", 0), (1, 64, 4, 3000, "float32", 0), (2, 16, 24, 999, "bfloat16", 0),
    # groups of 10, 12 and 20 channels: a packet may lie in two groups (one slice and several)
    (2, 32, 10, 1030, "bfloat16", 0), (3, 32, 20, 300, "float16", 0), (2, 16, 10, 2000, "float32", 0),
    (40, 32, 10, 64, "bfloat16", 0), (3, 8, 12, 5000, "bfloat16", 0),
    # groups of 1-6 channels, narrower than a packet: every channel of a packet finds its own
    # group (one slice and several, a group count that is not a power of two)
    (3, 32, 3, 196, "bfloat16", 0), (2, 8, 4, 256, "bfloat16", 0), (2, 32, 6, 64, "float16", 0),
    (2, 32, 2, 3136, "bfloat16", 0), (2, 16, 2, 1000, "float32", 0), (40, 32, 1, 64, "bfloat16", 0),
    (2, 24, 3, 3000, "float32", 0), (5000, 8, 4, 16, "bfloat16", 0),
    # rows of 160, 320 and 384 packets: not sliced (too many idle threads), same answer
    (3, 32, 40, 777, "bfloat16", 0), (2, 32, 40, 600, "float32", 0), (2, 48, 64, 500, "float16", 0),
]


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("N,G,D,S,dtype,shift", NHWC_SLICE_CASES)
def test_group_norm_forward_nhwc_slice_shapes(K, N, G, D, S, dtype, shift, in_place):
    import torch
    rng = np.random.default_rng(7000 + G * D + S)
    C = G * D
    n = N * C * S
    xb, xs = _values(rng, (n,), dtype, 2.0)
    xs = xs + 0.0
    x = xs.reshape(N, S, G, D)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    eps = 1e-5
    mean = x.mean((1, 3))
    rs = 1 / np.sqrt(((x - mean[:, None, :, None]) ** 2).mean((1, 3)) + np.float64(np.float32(eps)))
    y_ref = ((x - mean[:, None, :, None]) * rs[:, None, :, None]).reshape(N, S, C) * g + b
    xbuf, xd = _held(n, dtype, shift, xb)
    ybuf, yd = (xbuf, xd) if in_place else _held(n, dtype, shift)
    gd, bd = torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda()
    mu, rsig = torch.empty(N * G, device="cuda"), torch.empty(N * G, device="cuda")
    K.group_norm_forward(N, G, D, S, "NHWC", eps, xd, gd, bd, mu, rsig, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, S, C)
    assert _mean_ok(mu.cpu().numpy(), mean, x)
    assert np.max(np.abs(rsig.cpu().numpy().astype(np.float64) / rs.ravel() - 1)) <= 5e-5
    assert U.normwise(y, y_ref) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, shift, n)
    assert K.exchange_timed_out() == 0


# NCHW groups that one 256- or 512-thread workgroup holds whole (2048 packets and more, sixteen
# per thread at most): 9-16 packets per thread, a last slot that few threads fill, channels of
# fewer packets than the workgroup has threads (several channels per slot, a boundary inside the
# workgroup) and of more, one channel per group, more groups than resident workgroups, a group
# count that does not divide the grid, x at an address that is not 16-byte aligned (another
# path, same answer), in place.
NCHW_ITEM_CASES = [
    (2, 3, 6, 3136, "bfloat16", 0), (1, 2, 40, 784, "bfloat16", 0), (2, 2, 20, 784, "float32", 0),
    (3, 2, 1, 65536, "float16", 0), (1, 5, 16, 4096, "bfloat16", 0), (2, 4, 8, 4096, "float32", 0),
    (700, 3, 4, 2048, "float32", 0), (2, 2, 256, 128, "bfloat16", 0), (2, 2, 300, 64, "float16", 0),
    (1, 3, 16, 4096, "bfloat16", 3), (2, 7, 3, 5464, "bfloat16", 0), (1100, 2, 8, 2048, "bfloat16", 0),
    # every flavour: eight and ten packets on 256 threads, eight to sixteen on 512
    (2, 2, 20, 1024, "bfloat16", 0), (3, 3, 10, 4096, "bfloat16", 0), (2, 2, 12, 4096, "float16", 0),
    (2, 5, 10, 1000, "float32", 0), (2, 3, 11, 2048, "float32", 0), (40, 2, 5, 4096, "float32", 0),
    # groups of 128-256 KB on 1024 threads (ten, twelve and sixteen packets; more channels than
    # 512 threads; more groups than compute units)
    (1, 2, 32, 3136, "bfloat16", 0), (1, 3, 24, 3136, "bfloat16", 0), (2, 2, 20, 4096, "float16", 0),
    (1, 2, 45, 2048, "bfloat16", 0), (1, 2, 12, 4096, "float32", 0), (1, 2, 600, 64, "bfloat16", 0),
    (6, 16, 16, 4096, "float32", 0),
]


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("N,G,D,S,dtype,shift", NCHW_ITEM_CASES)
def test_group_norm_forward_nchw_whole_group_shapes(K, N, G, D, S, dtype, shift, in_place):
    import torch
    rng = np.random.default_rng(7100 + G * D + S)
    C = G * D
    n = N * C * S
    xb, xs = _values(rng, (n,), dtype, 2.0)
    xs = xs + 0.0
    x = xs.reshape(N, G, D, S)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    eps = 1e-5
    mean = x.mean((2, 3))
    rs = 1 / np.sqrt(((x - mean[:, :, None, None]) ** 2).mean((2, 3)) + np.float64(np.float32(eps)))
    y_ref = ((x - mean[:, :, None, None]) * rs[:, :, None, None]).reshape(N, C, S) * g[None, :, None] \
        + b[None, :, None]
    xbuf, xd = _held(n, dtype, shift, xb)
    ybuf, yd = (xbuf, xd) if in_place else _held(n, dtype, shift)
    gd, bd = torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda()
    mu, rsig = torch.empty(N * G, device="cuda"), torch.empty(N * G, device="cuda")
    K.group_norm_forward(N, G, D, S, "NCHW", eps, xd, gd, bd, mu, rsig, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, C, S)
    assert _mean_ok(mu.cpu().numpy(), mean, x)
    assert np.max(np.abs(rsig.cpu().numpy().astype(np.float64) / rs.ravel() - 1)) <= 5e-5
    assert U.normwise(y, y_ref) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, shift, n)


@pytest.mark.parametrize("N,G,D,S,fmt,dtype,seed", _channel_cases(40, 5))
def test_batch_norm_training_shapes(K, N, G, D, S, fmt, dtype, seed):
    import torch
    rng = np.random.default_rng(seed)
    C = G * D * int(rng.choice((1, 5, 16)))
    if N * S < 2:
        S = 2
    n = N * C * S
    xb, xs = _values(rng, (n,), dtype, 2.0)
    dyb, dys = _values(rng, (n,), dtype)
    x, dy = _as_ncs(xs, N, C, S, fmt), _as_ncs(dys, N, C, S, fmt)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    eps, momentum = 1e-5, 0.9
    mean = x.mean((0, 2))
    var = ((x - mean[None, :, None]) ** 2).mean((0, 2))
    rs = 1 / np.sqrt(var + np.float64(np.float32(eps)))
    y_ref = (x - mean[None, :, None]) * (rs * g)[None, :, None] + b[None, :, None]
    _, xd = _held(n, dtype, 0, xb)
    ybuf, yd = _held(n, dtype, 0)
    gd, bd = torch.from_numpy(g).cuda(), torch.from_numpy(b).cuda()
    rm0 = rng.standard_normal(C).astype(np.float32)
    rv0 = rng.uniform(0.5, 2.0, C).astype(np.float32)
    rm, rv = torch.from_numpy(rm0.copy()).cuda(), torch.from_numpy(rv0.copy()).cuda()
    mu, rsig = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    params = torch.empty(2 * C, device="cuda")
    K.batch_norm_training_forward(N, C, S, fmt, momentum, eps, xd, gd, bd, rm, rv, mu, rsig, params, yd)
    y = _as_ncs(U.widen(U.to_host(yd.contiguous()), dtype), N, C, S, fmt)
    assert _mean_ok(mu.cpu().numpy(), mean, x)
    assert np.max(np.abs(rsig.cpu().numpy().astype(np.float64) / rs - 1)) <= 5e-5
    assert U.normwise(y, y_ref) <= U.TIGHT[dtype]
    assert U.normwise(rm.cpu().numpy(), momentum * rm0 + (1 - momentum) * mean) <= 2e-5
    assert U.normwise(rv.cpu().numpy(), momentum * rv0 + (1 - momentum) * var) <= 5e-5
    assert _untouched(ybuf, dtype, 0, n)
    m32 = mu.cpu().numpy().astype(np.float64)[None, :, None]
    r32 = rsig.cpu().numpy().astype(np.float64)[None, :, None]
    _, dyd = _held(n, dtype, 0, dyb)
    dxbuf, dxd = _held(n, dtype, 0)
    wg = torch.empty(2 * C, device="cuda")
    K.batch_norm_training_backward(N, C, S, float(N * S), fmt, xd, mu, rsig, gd, dyd, wg, wg, dxd)
    xh = (x - m32) * r32
    dg_ref, db_ref = (dy * xh).sum((0, 2)), dy.sum((0, 2))
    dx_ref = (g[None, :, None] * r32) * (dy - (xh * dg_ref[None, :, None] + db_ref[None, :, None]) / (N * S))
    dx = _as_ncs(U.widen(U.to_host(dxd.contiguous()), dtype), N, C, S, fmt)
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(wg[:C].cpu().numpy(), dg_ref) <= 5e-5
    assert U.normwise(wg[C:].cpu().numpy(), db_ref) <= 5e-5
    assert _untouched(dxbuf, dtype, 0, n)


def _strided_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        C = max(1, int(rng.choice((1, 2, 7, 21, 64, 150, 1024, 1030, 2051))) + int(rng.integers(-1, 2)))
        S = max(2, int(rng.choice((2, 3, 8, 24, 70, 530, 4096))) + int(rng.integers(-1, 2)))
        N = int(rng.integers(1, max(2, min(9, 1_200_000 // (C * S)))))
        cases.append((N, C, S, DTYPES[int(rng.integers(0, 3))], 3000 + i))
    return cases


@pytest.mark.parametrize("N,C,S,dtype,seed", _strided_cases(40, 6))
def test_softmax_along_a_strided_axis(K, N, C, S, dtype, seed):
    rng = np.random.default_rng(seed)
    log = bool(seed & 1)
    xb, x = _values(rng, (N, C, S), dtype, 3.0)
    dyb, dy = _values(rng, (N, C, S), dtype)
    e = np.exp(x - x.max(1, keepdims=True))
    p = e / e.sum(1, keepdims=True)
    n = N * C * S
    _, xd = _held(n, dtype, 0, xb)
    ybuf, yd = _held(n, dtype, 0)
    (K.log_softmax if log else K.softmax)(N, S, C, xd, yd)
    y = U.widen(U.to_host(yd.contiguous()), dtype).reshape(N, C, S)
    if log:
        assert np.max(np.abs(y - np.log(p)) / (1 + np.abs(np.log(p)))) <= U.TIGHT[dtype]
    else:
        assert U.rowwise_normwise(y, p, axis=1) <= U.TIGHT[dtype]
    assert _untouched(ybuf, dtype, 0, n)
    _, dyd = _held(n, dtype, 0, dyb)
    dxbuf, dxd = _held(n, dtype, 0)
    (K.log_softmax_grad if log else K.softmax_grad)(N, S, C, dyd, yd, dxd)
    dx = U.widen(U.to_host(dxd.contiguous()), dtype).reshape(N, C, S)
    dx_ref = (dy - np.exp(y) * dy.sum(1, keepdims=True)) if log else \
        (dy - (dy * y).sum(1, keepdims=True)) * y
    assert U.normwise(dx, dx_ref) <= U.TIGHT[dtype]
    assert _untouched(dxbuf, dtype, 0, n)


def _moment_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        nd = int(rng.integers(1, 5))
        dims = [int(rng.choice((1, 2, 3, 7, 16, 33, 64, 200, 1031))) for _ in range(nd)]
        while int(np.prod(dims)) > 1_500_000:
            dims[int(np.argmax(dims))] = max(1, max(dims) // 4)
        k = int(rng.integers(1, nd + 1))
        axes = sorted(int(a) for a in rng.choice(nd, size=k, replace=False))
        cases.append((tuple(dims), tuple(axes), DTYPES[int(rng.integers(0, 3))], 4000 + i))
    return cases


@pytest.mark.parametrize("dims,axes,dtype,seed", _moment_cases(50, 7))
def test_moments_over_random_axes(K, dims, axes, dtype, seed):
    import torch
    rng = np.random.default_rng(seed)
    xb = R.to_bits((rng.standard_normal(dims) * 2 + 0.5).astype(np.float32), dtype)
    x = U.widen(xb, dtype).reshape(dims)
    want_m, want_v = x.mean(axes), x.var(axes)
    out = int(np.prod(want_m.shape)) if want_m.shape else 1
    mean, var = torch.empty(out, device="cuda"), torch.empty(out, device="cuda")
    K.moments(list(dims), list(axes), U.to_device(xb, dtype), mean, var)
    scale = np.sqrt(np.mean(x ** 2)) + 1e-30
    assert np.max(np.abs(mean.cpu().numpy() - want_m.ravel())) <= 2e-5 * scale
    assert np.max(np.abs(var.cpu().numpy() - want_v.ravel())) <= 4e-5 * scale ** 2


def _loss_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        C = max(2, int(rng.choice((2, 10, 21, 100, 1000, 4096, 20001, 30522, 32000))) + int(rng.integers(-1, 2)))
        S = int(rng.choice((1, 1, 1, 5, 64)))
        N = int(rng.integers(1, max(2, min(300, 600_000 // (C * S)))))
        cases.append((N, C, S, ("none", "sum", "mean", "valid")[int(rng.integers(0, 4))],
                      ("int64", "int32")[int(rng.integers(0, 2))], 5000 + i))
    return cases


@pytest.mark.parametrize("N,C,S,reduction,tdtype,seed", _loss_cases(40, 8))
def test_fused_softmax_cross_entropy_loss_shapes(K, N, C, S, reduction, tdtype, seed):
    import torch
    rng = np.random.default_rng(seed)
    dtype = "float32"
    x = (rng.standard_normal((N, C, S)) * 3).astype(np.float32)
    target = rng.integers(0, C, (N, S)).astype(tdtype)
    target[rng.random((N, S)) < 0.1] = 255 if C <= 255 else -1
    ignore = 255 if C <= 255 else -1
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(1, keepdims=True))
    p = e / e.sum(1, keepdims=True)
    valid = target != ignore
    safe = np.where(valid, target, 0).astype(np.int64)
    picked = np.take_along_axis(p, safe[:, None, :], 1)[:, 0, :]
    losses = np.where(valid, -np.log(np.maximum(picked, np.finfo(np.float32).tiny)), 0.0)
    nvalid = max(int(valid.sum()), 1)
    want = {"none": losses, "sum": losses.sum(), "mean": losses.sum() / (N * S),
            "valid": losses.sum() / nvalid}[reduction]
    xd, td = torch.from_numpy(x).cuda(), torch.from_numpy(target).cuda()
    prob = torch.empty((N, C, S), device="cuda")
    loss = torch.empty((N, S) if reduction == "none" else (1,), device="cuda")
    K.softmax_cross_entropy_loss_forward(N, S, C, ignore, reduction, xd, td, prob, loss)
    assert U.rowwise_normwise(prob.cpu().numpy(), p, axis=1) <= 1e-5
    got = loss.cpu().numpy().reshape(np.shape(want))
    assert np.max(np.abs(got - want)) <= 4e-5 * max(1.0, float(np.max(np.abs(want))))
    dl = rng.standard_normal((N, S)).astype(np.float32) if reduction == "none" else np.float32(1.7)
    dx = torch.empty((N, C, S), device="cuda")
    K.softmax_cross_entropy_loss_backward(N, S, C, ignore, reduction, prob, td,
                                          torch.from_numpy(np.atleast_1d(dl)).cuda(), dx)
    ph = prob.cpu().numpy().astype(np.float64)
    onehot = np.zeros((N, C, S))
    np.put_along_axis(onehot, safe[:, None, :], 1.0, 1)
    g = (ph - onehot) * valid[:, None, :]
    w = {"none": np.asarray(dl, np.float64)[:, None, :] if reduction == "none" else 0,
         "sum": 1.7, "mean": 1.7 / (N * S), "valid": 1.7 / nvalid}[reduction]
    assert U.normwise(dx.cpu().numpy(), g * w) <= 1e-5
    assert np.all(dx.cpu().numpy()[np.broadcast_to(~valid[:, None, :], (N, C, S))] == 0)


@pytest.mark.parametrize("C", [20001, 30522, 32002])
@pytest.mark.parametrize("shift", [0, 1, 3])
def test_fused_loss_on_wide_rows_at_shifted_bases(K, C, shift):
    """Vocabulary-sized fp32 rows that are not whole packets, logits and probabilities starting
    `shift` elements past a 16-byte boundary: the rows go through the aligned packets that cover
    them, the target's column moves with the window, and what surrounds the logits (a huge
    value) must not reach a row."""
    import torch
    N = 6
    rng = np.random.default_rng(C + shift)
    x = (rng.standard_normal((N, C)) * 3).astype(np.float32)
    target = rng.integers(0, C, N).astype(np.int64)
    target[1] = -1
    target[2], target[3] = 0, C - 1  # the row's first and last class: the window's edge packets
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(1, keepdims=True))
    p = e / e.sum(1, keepdims=True)
    valid = target != -1
    picked = p[np.arange(N), np.where(valid, target, 0)]
    want = np.where(valid, -np.log(picked), 0.0)
    xbuf = torch.full((N * C + shift + GUARD,), 3e4, device="cuda")
    xd = xbuf[shift:shift + N * C]
    xd.copy_(torch.from_numpy(x.ravel()).cuda())
    pbuf, pd = _held(N * C, "float32", shift)
    loss = torch.empty(N, device="cuda")
    K.softmax_cross_entropy_loss_forward(N, 1, C, -1, "none", xd, torch.from_numpy(target).cuda(),
                                         pd, loss)
    got = pd.contiguous().cpu().numpy().reshape(N, C)
    assert U.rowwise_normwise(got, p) <= 1e-5
    assert np.max(np.abs(loss.cpu().numpy() - want)) <= 4e-5 * max(1.0, float(want.max()))
    assert _untouched(pbuf, "float32", shift, N * C)
