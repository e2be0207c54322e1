"""Parity at the shapes bench.py measures, at full size: every workload of the sweep whose
kernel instantiation the small parity cases do not drive through more than one iteration per
workgroup (persistent workgroups with a prefetch ring, many rounds of the slice exchange,
more chunks of short rows than the grid holds).

Where the CPU oracle finishes in seconds it checks the whole tensor; for the larger ones it
checks sampled rows (first, last, and rows that only later rounds of a persistent grid reach)
and every row goes through a size-independent property and through the same formula evaluated
by torch on the device in a wider type (a library routine, not the code under test)."""

import numpy as np
import pytest

from oracle import ref_cpu as R
from tests import util as U

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    import torch
    assert torch.cuda.is_available()
    from dragon_amd import kernels
    return kernels


def _rows(t, rows):
    import torch
    return U.to_host(t[torch.as_tensor(rows, device=t.device)].contiguous())


def _widen_rows(t, rows, dtype):
    return R.from_bits(_rows(t, rows), dtype) if dtype in ("float16", "bfloat16") else _rows(t, rows)


def _sample_rows(N, count=48, seed=0):
    rng = np.random.default_rng(seed)
    rows = {0, 1, N // 2, N - 2, N - 1}
    rows.update(int(r) for r in rng.integers(0, N, count))
    return sorted(rows)


def _layer_norm_inputs(N, C, dtype, seed, outliers=False):
    import torch
    gen = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.empty((N, C), device="cuda").normal_(generator=gen)
    if outliers:
        x[torch.empty((N, C), device="cuda").uniform_(generator=gen) < 0.01] *= 50
    x = x.to(U.torch_dtype(dtype))
    dy = torch.empty((N, C), device="cuda").normal_(generator=gen).to(U.torch_dtype(dtype))
    g = torch.empty(C, device="cuda").uniform_(0.5, 1.5, generator=gen)
    b = torch.empty(C, device="cuda").normal_(generator=gen).mul_(0.1)
    return x, dy, g, b


def _layer_norm_run(K, N, C, x, dy, g, b):
    import torch
    y, dx = torch.empty_like(x), torch.empty_like(x)
    mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    K.layer_norm(N, C, 1e-5, x, g, b, mu, rsig, y)
    params = torch.empty(2 * N, device="cuda")
    dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    K.group_norm_grad(N, 1, C, 1, "NHWC", x, mu, rsig, g, dy, params, params, dg, db, dx)
    return y, mu, rsig, dx, dg, db, params


def _column_sums_fp64(x, dy, mu, rsig, step=1 << 15):
    """dgamma, dbeta as fp64 sums of the same products, in row chunks."""
    import torch
    C = x.shape[1]
    dg = torch.zeros(C, dtype=torch.float64, device="cuda")
    db = torch.zeros(C, dtype=torch.float64, device="cuda")
    for r0 in range(0, x.shape[0], step):
        xc, dc = x[r0:r0 + step].double(), dy[r0:r0 + step].double()
        m, r = mu[r0:r0 + step].double()[:, None], rsig[r0:r0 + step].double()[:, None]
        dg += (dc * (xc - m) * r).sum(0)
        db += dc.sum(0)
    return dg.cpu().numpy(), db.cpu().numpy()


@pytest.mark.parametrize("dtype", ["bfloat16", "float16", "float32"])
def test_layer_norm_8192x4096_whole_tensor_against_the_oracle(K, dtype):
    """bench workloads layer_norm_{bf16,f32}_8192x4096: eight iterations per persistent
    workgroup of the forward tiles and of the backward's 1024-thread ring kernel."""
    N, C = 8192, 4096
    x, dy, g, b = _layer_norm_inputs(N, C, dtype, 41)
    y, mu, rsig, dx, dg, db, params = _layer_norm_run(K, N, C, x, dy, g, b)
    gh, bh = U.to_host(g), U.to_host(b)
    y_ref, mu_ref, rsig_ref = R.layer_norm(dtype, U.to_host(x), gh, bh, 1e-5)
    assert U.normwise(U.to_host(mu), mu_ref) <= 1e-5
    assert np.max(np.abs(U.to_host(rsig) / rsig_ref - 1)) <= 1e-5
    assert U.normwise(U.widen(U.to_host(y), dtype), U.widen(y_ref, dtype)) <= U.TIGHT[dtype]
    xo = R.from_bits(U.to_host(x), dtype) if dtype != "float32" else U.to_host(x)
    dyo = R.from_bits(U.to_host(dy), dtype) if dtype != "float32" else U.to_host(dy)
    dx_ref, dg_ref, db_ref, ds_ref, dbb_ref = R.group_norm_grad(
        "float32", N, 1, C, 1, "NHWC", xo, U.to_host(mu), U.to_host(rsig), gh, dyo)
    assert U.normwise(U.widen(U.to_host(dx), dtype), dx_ref) <= U.TIGHT[dtype]
    p = U.to_host(params)
    assert U.normwise(p[:N], ds_ref) <= 2e-5 and U.normwise(p[N:], dbb_ref) <= 2e-5
    # 8192-term column sums: the oracle's sequential fp32 sums are themselves off, so three-way
    dg64, db64 = _column_sums_fp64(x, dy, mu, rsig)
    for got, ref, exact in ((dg, dg_ref, dg64), (db, db_ref, db64)):
        ok, *errs = U.close3(U.to_host(got), ref, exact, 2e-5)
        assert ok, errs


@pytest.mark.parametrize("shape,dtype,outliers", [((8192, 12288), "bfloat16", True),
                                                  ((1048576, 64), "bfloat16", False),
                                                  ((65536, 1000), "bfloat16", True),
                                                  ((32768, 4096), "bfloat16", False),
                                                  ((32768, 12288), "bfloat16", False)])
def test_layer_norm_bench_shapes_sampled_rows_and_column_sums(K, shape, dtype, outliers):
    """bench workloads layer_norm_bf16_8192x12288 (32 rows per workgroup of the 768-thread
    backward tile), layer_norm_bf16_1048576x64 (more chunks of staged short rows than the grid
    holds), layer_norm_bf16_65536x1000 (ragged rows), and layer_norm_bf16_32768x4096 /
    32768x12288 (32 and 128 iterations per persistent workgroup)."""
    N, C = shape
    x, dy, g, b = _layer_norm_inputs(N, C, dtype, 42, outliers)
    y, mu, rsig, dx, dg, db, params = _layer_norm_run(K, N, C, x, dy, g, b)
    rows = _sample_rows(N, 64, seed=C)
    gh, bh = U.to_host(g), U.to_host(b)
    y_ref, mu_ref, rsig_ref = R.layer_norm(dtype, _rows(x, rows), gh, bh, 1e-5)
    assert U.normwise(_rows(mu, rows), mu_ref) <= 1e-5
    assert np.max(np.abs(_rows(rsig, rows) / rsig_ref - 1)) <= 1e-5
    assert U.normwise(U.widen(_rows(y, rows), dtype), U.widen(y_ref, dtype)) <= U.TIGHT[dtype]
    dx_ref, _, _, ds_ref, db_ref = R.group_norm_grad(
        "float32", len(rows), 1, C, 1, "NHWC", _widen_rows(x, rows, dtype), _rows(mu, rows),
        _rows(rsig, rows), gh, _widen_rows(dy, rows, dtype))
    assert U.normwise(U.widen(_rows(dx, rows), dtype), dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(_rows(params[:N], rows), ds_ref) <= 2e-5
    assert U.normwise(_rows(params[N:], rows), db_ref) <= 2e-5
    # every row: the statistics against torch in fp64, the output through its own moments
    xf = x.double()
    assert float((mu.double() - xf.mean(1)).abs().max()) <= 1e-5 * float(xf.mean(1).abs().max() + 1)
    var = xf.var(1, unbiased=False)
    assert float((rsig.double() * (var + 1e-5).sqrt() - 1).abs().max()) <= 2e-5
    del xf, var
    # dx is orthogonal to the ones vector and to x-hat in the gamma-weighted sense:
    # sum_c dx = 0 holds for every row whatever gamma is
    assert float(dx.float().sum(1).abs().max()) <= 0.08 * np.sqrt(C)
    dg64, db64 = _column_sums_fp64(x, dy, mu, rsig)
    assert U.normwise(U.to_host(dg), dg64) <= 2e-5
    assert U.normwise(U.to_host(db), db64) <= 2e-5


def _softmax_inputs(N, C, dtype, seed):
    import torch
    gen = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.empty((N, C), device="cuda").normal_(generator=gen).mul_(3)
    x[torch.empty((N, C), device="cuda").uniform_(generator=gen) < 0.05] = -1e4
    x = x.to(U.torch_dtype(dtype))
    dy = torch.empty((N, C), device="cuda").normal_(generator=gen).to(U.torch_dtype(dtype))
    return x, dy


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float32"])
def test_softmax_8192x4096_whole_tensor_against_the_oracle(K, dtype):
    """bench workloads softmax_{f16,f32}_8192x4096: rows of 512 / 1024 packets."""
    import torch
    N, C = 8192, 4096
    x, dy = _softmax_inputs(N, C, dtype, 43)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    K.softmax(N, 1, C, x, y)
    K.softmax_grad(N, 1, C, dy, y, dx)
    xo = R.from_bits(U.to_host(x), dtype) if dtype != "float32" else U.to_host(x)
    y_ref = R.softmax("float32", N, 1, C, xo)
    # the oracle's sequential fp32 sum of 4096 exponentials is itself ~1e-5 off: three-way
    y64 = torch.softmax(x.double(), 1).cpu().numpy()
    yw = U.widen(U.to_host(y), dtype)
    e_go, e_ge, e_oe = (U.rowwise_normwise(yw, y_ref), U.rowwise_normwise(yw, y64),
                        U.rowwise_normwise(y_ref, y64))
    assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)
    yo = R.from_bits(U.to_host(y), dtype) if dtype != "float32" else U.to_host(y)
    dyo = R.from_bits(U.to_host(dy), dtype) if dtype != "float32" else U.to_host(dy)
    dx_ref = R.softmax_grad("float32", N, 1, C, dyo, yo)
    yd, dd = y.double(), dy.double()
    dx64 = ((dd - (dd * yd).sum(1, keepdim=True)) * yd).cpu().numpy()
    dxw = U.widen(U.to_host(dx), dtype)
    e_go, e_ge, e_oe = (U.rowwise_normwise(dxw, dx_ref), U.rowwise_normwise(dxw, dx64),
                        U.rowwise_normwise(dx_ref, dx64))
    assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)


@pytest.mark.parametrize("shape,dtype", [((2048, 128256), "float32"), ((2048, 128256), "bfloat16"),
                                         ((605184, 197), "bfloat16"), ((4096, 50257), "bfloat16"),
                                         ((4096, 30522), "float16")])
@pytest.mark.parametrize("log", [False, True])
def test_softmax_bench_shapes_sampled_rows_and_every_row(K, shape, dtype, log):
    """bench workloads softmax_f32_2048x128256 (vocabulary-sized rows cut into slices that
    several workgroups hold: tens of thousands of work items over many rounds of the resident
    grid, each round's packets requested into the registers the round before has just
    rewritten), softmax_bf16_605184x197 (rows that are not whole packets, far more chunks
    of staged rows than the grid holds) and softmax_bf16_4096x50257 (rows that are not whole
    packets through the aligned packets that cover them, many rows per persistent workgroup;
    [4096, 30522] for the flavour that holds the converted row)."""
    import torch
    N, C = shape
    x, dy = _softmax_inputs(N, C, dtype, 44)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    (K.log_softmax if log else K.softmax)(N, 1, C, x, y)
    (K.log_softmax_grad if log else K.softmax_grad)(N, 1, C, dy, y, dx)
    # every row against torch in fp32 / fp64 on the device
    step = max(1, (1 << 25) // C)
    tol = U.TIGHT[dtype]
    for r0 in range(0, N, step):
        xs = x[r0:r0 + step].double()
        ref = torch.log_softmax(xs, 1) if log else torch.softmax(xs, 1)
        got = y[r0:r0 + step].double()
        if log:
            keep = ref > -5e3
            err = ((got - ref).abs() / ref.abs().clamp_min(1.0))[keep].max()
        else:
            err = ((got - ref).abs().amax(1) / ref.amax(1)).max()
        assert float(err) <= tol, (r0, float(err))
        yy, dd = y[r0:r0 + step].double(), dy[r0:r0 + step].double()
        if log:
            dref = dd - yy.exp() * dd.sum(1, keepdim=True)
        else:
            dref = (dd - (dd * yy).sum(1, keepdim=True)) * yy
        gd = dx[r0:r0 + step].double()
        err = (gd - dref).abs().amax(1) / dref.abs().amax(1).clamp_min(1e-30)
        assert float(err.max()) <= tol, (r0, float(err.max()))
    del xs, ref, got, yy, dd, dref, gd
    # sampled rows against the oracle (backward on the y the forward produced). Rows of
    # 128256 put the oracle's sequential fp32 sums ~3e-4 off, so the check is three-way:
    # within the bar of fp64, and of the oracle up to the oracle's own distance from fp64
    rows = _sample_rows(N, 24, seed=C)
    xo = _widen_rows(x, rows, dtype)
    y_ref = np.asarray((R.log_softmax if log else R.softmax)("float32", len(rows), 1, C, xo), np.float64)
    x64 = np.asarray(xo, np.float64)
    s64 = x64 - x64.max(1, keepdims=True)
    ly64 = s64 - np.log(np.exp(s64).sum(1, keepdims=True))
    y64 = ly64 if log else np.exp(ly64)
    yw = U.widen(_rows(y, rows), dtype)
    if log:
        keep = y64 > -5e3

        def dist(a, b):
            return float((np.abs(a - b)[keep] / np.maximum(np.abs(b)[keep], 1.0)).max())
    else:
        dist = U.rowwise_normwise
    e_go, e_ge, e_oe = dist(yw, y_ref), dist(yw, y64), dist(y_ref, y64)
    assert e_ge <= tol and e_go <= tol + e_oe, (e_go, e_ge, e_oe)
    yo, dyo = _widen_rows(y, rows, dtype), _widen_rows(dy, rows, dtype)
    dx_ref = (R.log_softmax_grad if log else R.softmax_grad)("float32", len(rows), 1, C, dyo, yo)
    y6, d6 = np.asarray(yo, np.float64), np.asarray(dyo, np.float64)
    dx64 = (d6 - np.exp(y6) * d6.sum(1, keepdims=True)) if log else (
        (d6 - (d6 * y6).sum(1, keepdims=True)) * y6)
    dxw = U.widen(_rows(dx, rows), dtype)
    e_go, e_ge, e_oe = (U.rowwise_normwise(dxw, dx_ref), U.rowwise_normwise(dxw, dx64),
                        U.rowwise_normwise(dx_ref, dx64))
    assert e_ge <= tol and e_go <= tol + e_oe, (e_go, e_ge, e_oe)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batch_norm_64x256x57x57_sampled_channels_and_every_channel(K, dtype):
    """bench workload batch_norm_f32_64x256x57x57: feature maps that are not whole packets
    through the single-read kernels, four rounds of work items over the resident grid. The
    oracle's operator checks sampled channels (channels are independent); every channel goes
    through the closed forms in fp64 on the device and through the property that a
    batch-normalised channel's input gradient sums to zero."""
    import torch
    N, C, H, W = 64, 256, 57, 57
    S = H * W
    gen = torch.Generator(device="cuda").manual_seed(21)
    td = U.torch_dtype(dtype)
    x = torch.empty((N, C, S), device="cuda").normal_(generator=gen).mul_(2).add_(0.5).to(td)
    dy = torch.empty((N, C, S), device="cuda").normal_(generator=gen).to(td)
    g = torch.empty(C, device="cuda").uniform_(0.5, 1.5, generator=gen)
    b = torch.empty(C, device="cuda").normal_(generator=gen).mul_(0.1)
    rm, rv = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
    mu, rsig, params = (torch.empty(n, device="cuda") for n in (C, C, 2 * C))
    y, dx = torch.empty_like(x), torch.empty_like(x)
    wg = torch.empty(2 * C, device="cuda")
    K.batch_norm_training_forward(N, C, S, "NCHW", 0.9, 1e-5, x, g, b, rm, rv, mu, rsig, params, y)
    K.batch_norm_training_backward(N, C, S, float(N * S), "NCHW", x, mu, rsig, g, dy, wg, wg, dx)
    torch.cuda.synchronize()
    tol = U.TIGHT[dtype]
    # every channel: fp64 closed forms on the device
    x64, dy64 = x.double(), dy.double()
    mu64 = x64.mean((0, 2))
    var64 = x64.var((0, 2), unbiased=False)
    rsig64 = torch.rsqrt(var64 + 1e-5)
    assert float((mu.double() - mu64).abs().max()) <= 1e-5 * float(mu64.abs().max())
    assert float((rsig.double() / rsig64 - 1).abs().max()) <= 1e-5
    assert float((rm.double() - 0.1 * mu64).abs().max()) <= 1e-5
    assert float((rv.double() - (0.9 + 0.1 * var64)).abs().max()) <= 1e-4
    xh = (x64 - mu.double()[None, :, None]) * rsig.double()[None, :, None]
    y64 = xh * g.double()[None, :, None] + b.double()[None, :, None]
    assert float((y.double() - y64).norm() / y64.norm()) <= tol
    dg64, db64 = (dy64 * xh).sum((0, 2)), dy64.sum((0, 2))
    assert float((wg[:C].double() - dg64).norm() / dg64.norm()) <= 2e-5
    assert float((wg[C:].double() - db64).norm() / db64.norm()) <= 2e-5
    dx64 = (g.double() * rsig.double())[None, :, None] * (
        dy64 - (xh * dg64[None, :, None] + db64[None, :, None]) / (N * S))
    assert float((dx.double() - dx64).norm() / dx64.norm()) <= tol
    # (16-bit outputs: 207936 roundings per channel, bounded relative to the sum of magnitudes)
    sums, mags = dx.double().sum((0, 2)).abs(), dx.double().abs().sum((0, 2))
    assert float(sums.max()) < 5e-2 if dtype == "float32" else bool((sums <= 1e-3 * mags).all())
    del x64, dy64, xh, y64, dx64
    # sampled channels against the oracle's operator (first, last, and ones that later
    # rounds of the grid reach)
    chans = [0, 1, 100, 191, 254, 255]
    idx = torch.as_tensor(chans, device="cuda")
    xs = U.to_host(x[:, idx].contiguous()).reshape(N, len(chans), H, W)
    dys = U.to_host(dy[:, idx].contiguous()).reshape(N, len(chans), H, W)
    gs, bs = U.to_host(g[idx]), U.to_host(b[idx])
    xo, od = (R.from_bits(xs, dtype), "float32") if dtype != "float32" else (xs, "float32")
    dyo = R.from_bits(dys, dtype) if dtype != "float32" else dys
    rm_ref, rv_ref = np.zeros(len(chans), np.float32), np.ones(len(chans), np.float32)
    y_ref, mu_ref, rsig_ref, _ = R.op_batch_norm_train(od, xo, gs, bs, rm_ref, rv_ref, 1, 0.9, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_train_grad(od, xo, gs, dyo, mu_ref, rsig_ref, 1)
    # the oracle's sequential fp32 sums over 207936 terms are themselves ~5e-5 off fp64
    assert U.normwise(U.to_host(mu[idx]), mu_ref) <= 1e-4
    assert np.max(np.abs(U.to_host(rsig[idx]) / rsig_ref - 1)) <= 1e-4
    yg = U.to_host(y[:, idx].contiguous()).reshape(xs.shape)
    dxg = U.to_host(dx[:, idx].contiguous()).reshape(xs.shape)
    assert U.normwise(U.widen(yg, dtype), y_ref) <= max(tol, 1e-4)
    assert U.normwise(U.widen(dxg, dtype), dx_ref) <= max(tol, 1e-4)
    assert U.normwise(U.to_host(wg[:C][idx]), dg_ref) <= 1e-4
    assert U.normwise(U.to_host(wg[C:][idx]), db_ref) <= 1e-4


def test_group_norm_nhwc_32x64x64x512_sampled_samples_and_every_group(K):
    """The channels-last GroupNorm tensor of the sweep: 32 samples of 4 MB, 64 slices of rows
    each, more work items than resident workgroups. Two samples against the oracle; every
    group's statistics against fp64 on the device; every element of y against the defining
    formula in fp32 on the device."""
    import torch
    N, S, G, D = 32, 64 * 64, 32, 16
    C = G * D
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.empty((N, S, C), device="cuda").normal_(generator=gen) + 0.3).to(torch.bfloat16)
    g = torch.empty(C, device="cuda").uniform_(0.5, 1.5, generator=gen)
    b = torch.empty(C, device="cuda").normal_(generator=gen).mul_(0.1)
    mu, rsig = torch.empty(N * G, device="cuda"), torch.empty(N * G, device="cuda")
    y = torch.empty_like(x)
    K.group_norm_forward(N, G, D, S, "NHWC", 1e-5, x, g, b, mu, rsig, y)
    torch.cuda.synchronize()
    assert K.exchange_timed_out() == 0
    xg = x.double().reshape(N, S, G, D)
    mean64 = xg.mean((1, 3))
    rs64 = torch.rsqrt(xg.var((1, 3), unbiased=False) + float(np.float32(1e-5)))
    assert float((mu.reshape(N, G).double() - mean64).abs().max()) <= 1e-5
    assert float((rsig.reshape(N, G).double() / rs64 - 1).abs().max()) <= 1e-5
    want = ((x.float().reshape(N, S, G, D) - mu.reshape(N, 1, G, 1)) * rsig.reshape(N, 1, G, 1)
            ).reshape(N, S, C) * g + b
    err = (y.float() - want).abs().max()
    assert float(err) <= 2 ** -7 * float(want.abs().max())  # one bf16 rounding of the result
    for n in (0, N - 1):
        xb = U.to_host(x[n].contiguous())
        y_ref, mu_ref, rsig_ref = R.op_group_norm("bfloat16", xb.reshape(1, S, C), U.to_host(g),
                                                  U.to_host(b), -1, G, 1e-5)
        # the oracle's sequential fp32 sums over 65536 elements are themselves a few 1e-5 off
        # fp64: three-way, as for the other long reductions
        rs_n = rs64[n].cpu().numpy()
        oracle_off = np.max(np.abs(rsig_ref / rs_n - 1))
        assert U.normwise(U.to_host(mu[n * G:(n + 1) * G]), mu_ref) <= 1e-5 + oracle_off
        assert np.max(np.abs(U.to_host(rsig[n * G:(n + 1) * G]) / rsig_ref - 1)) <= 1e-5 + oracle_off
        assert U.normwise(U.widen(U.to_host(y[n].contiguous()), "bfloat16").ravel(),
                          np.asarray(U.widen(y_ref, "bfloat16")).ravel()) <= U.TIGHT["bfloat16"]

