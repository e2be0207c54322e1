"""GPU parity: every C-ABI kernel entry point against the CPU oracle on the same
seeded inputs, at sizes the oracle finishes in seconds.

Bar: normwise 1e-5 for fp32 I/O and 1e-2 for fp16 / bf16 I/O against the fp32
oracle run on the 16-bit-rounded inputs (tests/util.py: TOL); fp64 to 1e-12.
Where the reference's CPU kernel supports the 16-bit type itself (LayerNorm,
GroupNorm forward, Moments) the oracle runs in that type.
"""

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


def empty(shape, dtype):
    import torch
    return torch.empty(shape, dtype=U.torch_dtype(dtype), device="cuda")


def acc_name(dtype):
    return "float64" if dtype == "float64" else "float32"


def oracle_dtype_inputs(bits, dtype):
    """Inputs for an oracle kernel that only exists in fp32/fp64: widen 16-bit storage."""
    if dtype in ("float16", "bfloat16"):
        return R.from_bits(bits, dtype), "float32"
    return bits, dtype


# ---------------------------------------------------------------- LayerNorm forward

LN_SHAPES = [(64, 1024), (33, 1000), (7, 12288), (5, 4096), (300, 48), (3, 37), (9, 8),
             (2, 70000), (3, 40000), (1, 1), (513, 256),
             # short and odd rows staged through LDS (several ranges per workgroup)
             (5000, 64), (700, 197), (130, 577), (9000, 16)]


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape", LN_SHAPES)
def test_layer_norm_forward(K, dtype, shape):
    N, C = shape
    rng = U.rng_for(100 + C)
    x = R.to_bits((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    y_ref, mu_ref, rsig_ref = R.layer_norm(dtype, x, g, b, 1e-5)
    xd, gd, bd = U.to_device(x, dtype), U.to_device(g, acc_name(dtype)), U.to_device(b, acc_name(dtype))
    y, mu, rsig = empty(shape, dtype), empty((N,), acc_name(dtype)), empty((N,), acc_name(dtype))
    K.layer_norm(N, C, 1e-5, xd, gd, bd, mu, rsig, y)
    stat_tol = 1e-12 if dtype == "float64" else 1e-5
    # fp64 statistics of the same (rounded) inputs: rows longer than a few
    # thousand elements put the oracle's sequential fp32 sums above 1e-5
    x64 = U.widen(x, dtype)
    mu64 = x64.mean(1)
    rsig64 = 1 / np.sqrt(x64.var(1) + np.float64(np.float32(1e-5)))
    ok, *errs = U.close3(U.to_host(mu), mu_ref, mu64, stat_tol)
    assert ok, errs
    ok, *errs = U.close3(U.to_host(rsig), rsig_ref, rsig64, stat_tol)
    assert ok, errs
    assert U.normwise(U.widen(U.to_host(y), dtype), U.widen(y_ref, dtype)) <= U.TIGHT[dtype]


def test_layer_norm_empty_and_errors(K):
    import torch
    from dragon_amd._lib import DragonHipError
    z = torch.empty(0, device="cuda")
    K.layer_norm(0, 16, 1e-5, z, z, z, z, z, z)  # no rows: nothing enqueued, no error
    with pytest.raises(DragonHipError):
        K.layer_norm(4, 0, 1e-5, z, z, z, z, z, z)
    with pytest.raises(TypeError):
        K.layer_norm(1, 1, 1e-5, z.to(torch.int32), z, z, z, z, z)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("C", [37, 64, 1000, 4096, 12288, 40000, 70000])
def test_layer_norm_special_values_follow_the_reference(K, C, dtype):
    """A row holding one nan or one inf comes out all nan, statistics included, as the CPU
    kernel's sums make it (layer_norm_kernel.cc:10-39); its neighbours are untouched."""
    N = 6
    rng = U.rng_for(C)
    xf = rng.standard_normal((N, C)).astype(np.float32)
    xf[1, C // 3] = np.nan
    xf[3, C - 1] = np.inf
    xf[4, 0] = -np.inf
    x = R.to_bits(xf, dtype)
    g, b = U.affine_params(rng, C, dtype)
    y_ref, mu_ref, rsig_ref = R.layer_norm(dtype, x, g, b, 1e-5)
    y, mu, rsig = empty((N, C), dtype), empty((N,), "float32"), empty((N,), "float32")
    K.layer_norm(N, C, 1e-5, U.to_device(x, dtype), U.to_device(g, "float32"),
                 U.to_device(b, "float32"), mu, rsig, y)
    yw, yr = U.widen(U.to_host(y), dtype), U.widen(y_ref, dtype)
    assert np.array_equal(np.isnan(yw), np.isnan(yr))
    assert np.array_equal(np.isnan(U.to_host(rsig)), np.isnan(rsig_ref))
    assert np.array_equal(np.isnan(U.to_host(mu)), np.isnan(mu_ref))
    assert np.array_equal(U.to_host(mu)[np.isinf(mu_ref)], mu_ref[np.isinf(mu_ref)])
    clean = [0, 2, 5]
    assert U.normwise(yw[clean], yr[clean]) <= U.TIGHT[dtype]


def test_layer_norm_large_mean_stays_accurate(K):
    """|mean| >> stddev: the centred variance must not cancel (fp64 is the judge)."""
    rng = U.rng_for(7)
    N, C = 16, 4096
    x = (rng.standard_normal((N, C)) + 1000.0).astype(np.float32)
    g, b = np.ones(C, np.float32), np.zeros(C, np.float32)
    y, mu, rsig = empty((N, C), "float32"), empty((N,), "float32"), empty((N,), "float32")
    K.layer_norm(N, C, 1e-5, U.to_device(x, "float32"), U.to_device(g, "float32"),
                 U.to_device(b, "float32"), mu, rsig, y)
    x64 = x.astype(np.float64)
    r64 = 1 / np.sqrt(x64.var(1) + 1e-5)
    assert np.max(np.abs(U.to_host(rsig) / r64 - 1)) < 1e-5


# ---------------------------------------------------------------- Softmax family

SM_SHAPES = [((256, 512), -1), ((10, 1000), -1), ((4, 4096), -1), ((3, 100000), -1), ((5, 37), -1),
             ((6, 300), -1), ((3, 7, 5), 1), ((2, 3, 4, 6), 2), ((4, 1), -1), ((2, 16, 8, 8), -1),
             ((3, 8200), -1),
             # a wavefront takes two rows at a time: odd row counts, a single row
             ((7, 512), -1), ((1, 512), -1), ((33, 1000), -1), ((9, 1024), -1),
             # rows beyond the one-workgroup tiles: several workgroups per row (with the
             # scratch the wrapper passes); (3, 100000) above takes the same path
             ((5, 131072), -1),
             # short rows staged through LDS, several rows per wavefront
             ((64, 64), -1), ((33, 197), -1), ((9, 577), -1), ((100, 128), -1), ((300, 8), -1),
             # a strided axis beyond the register tiles (more than 1024 classes): panels of
             # columns walked in chunks of rows, twice; wide, medium and narrow panels, a
             # partial last chunk, columns that are not whole packets
             ((2, 1500, 40), 1), ((3, 4096, 24), 1), ((1, 1100, 530), 1), ((300, 1030, 70), 1),
             ((2, 2051, 3), 1)]


def _softmax_inputs(shape, dtype, seed):
    rng = U.rng_for(seed)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    x[rng.random(shape) < 0.05] = -1e4
    # keep one finite logit per reduced slice
    dy = rng.standard_normal(shape).astype(np.float32)
    return R.to_bits(x, dtype), R.to_bits(dy, dtype)


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape,axis", SM_SHAPES)
def test_softmax_forward_backward(K, shape, axis, dtype, log):
    x, dy = _softmax_inputs(shape, dtype, 200 + len(shape))
    ax = axis % len(shape)
    N = int(np.prod(shape[:ax] or (1,)))
    C = shape[ax]
    S = int(np.prod(shape[ax + 1:] or (1,)))
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    y_ref = R.op_softmax(od, xo, axis, log=log)
    xd, dyd = U.to_device(x, dtype), U.to_device(dy, dtype)
    y = empty(shape, dtype)
    (K.log_softmax if log else K.softmax)(N, S, C, xd, y)
    y_host = U.to_host(y)
    yw = U.widen(y_host, dtype).reshape(shape)
    if log:
        finite = np.isfinite(y_ref) & (np.asarray(y_ref) > -5e3)
        x64 = np.asarray(xo, np.float64)
        s64 = x64 - x64.max(ax, keepdims=True)
        ly64 = s64 - np.log(np.exp(s64).sum(ax, keepdims=True))

        def rel(a, b):
            return np.max(np.abs(a[finite] - b[finite]) / np.maximum(np.abs(b[finite]), 1.0))

        yr = np.asarray(y_ref, np.float64)
        e_go, e_ge, e_oe = rel(yw, yr), rel(yw, ly64), rel(yr, ly64)
        assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)
    else:
        # fp64 softmax of the same inputs; a 100000-term sequential fp32 sum puts
        # the oracle itself ~1e-4 off, which the three-way check allows for
        x64 = np.asarray(xo, np.float64)
        e64 = np.exp(x64 - x64.max(ax, keepdims=True))
        y64 = e64 / e64.sum(ax, keepdims=True)
        e_go = U.rowwise_normwise(np.moveaxis(yw, ax, -1), np.moveaxis(np.asarray(y_ref), ax, -1))
        e_ge = U.rowwise_normwise(np.moveaxis(yw, ax, -1), np.moveaxis(y64, ax, -1))
        e_oe = U.rowwise_normwise(np.moveaxis(np.asarray(y_ref), ax, -1), np.moveaxis(y64, ax, -1))
        assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)
        sums = yw.sum(ax)
        assert np.max(np.abs(sums - 1)) <= {"float16": 2e-3, "bfloat16": 2e-2}.get(dtype, 1e-5)
    # backward consumes the y the forward produced, as the operator graph does
    yo, _ = oracle_dtype_inputs(y_host.reshape(shape), dtype)
    dx_ref = R.op_softmax_grad(od, yo, dyo, axis, log=log)
    dx = empty(shape, dtype)
    (K.log_softmax_grad if log else K.softmax_grad)(N, S, C, dyd, y, dx)
    dxw = U.widen(U.to_host(dx), dtype).reshape(shape)
    ok = np.isfinite(np.asarray(dx_ref))
    assert U.normwise(dxw[ok], np.asarray(dx_ref)[ok]) <= U.TIGHT[dtype]


@pytest.mark.parametrize("shape", [(64, 512), (7, 197), (2, 66001), (2, 66000), (3, 10, 33),
                                   (2, 1300, 20), (3, 30522), (2, 50257)])
@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_softmax_in_place(K, dtype, shape):
    x, dy = _softmax_inputs(shape, dtype, 5)
    xo, od = oracle_dtype_inputs(x, dtype)
    axis = 1  # the last axis of the 2-d shapes, the strided middle axis of the 3-d one
    N, C = shape[0], shape[1]
    S = int(np.prod(shape[2:] or (1,)))
    y_ref = R.op_softmax(od, xo, axis)
    buf = U.to_device(x, dtype)
    K.softmax(N, S, C, buf, buf)  # Y aliases X (AllowInplace {0,0})
    got = np.moveaxis(U.widen(U.to_host(buf), dtype).reshape(shape), axis, -1)
    x64 = np.moveaxis(np.asarray(xo, np.float64), axis, -1)
    e64 = np.exp(x64 - x64.max(-1, keepdims=True))
    y64 = e64 / e64.sum(-1, keepdims=True)
    yr = np.moveaxis(np.asarray(y_ref), axis, -1)
    # rows of 66001 put the oracle's sequential fp32 sum itself off: three-way check
    e_ge, e_go, e_oe = (U.rowwise_normwise(got, y64), U.rowwise_normwise(got, yr),
                        U.rowwise_normwise(yr, y64))
    assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)
    g = U.to_device(dy, dtype)
    yo, _ = oracle_dtype_inputs(U.to_host(buf).reshape(shape), dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    dx_ref = R.op_softmax_grad(od, yo, dyo, axis)
    K.softmax_grad(N, S, C, g, buf, g)  # dX aliases dY (AllowInplace {1,0})
    assert U.normwise(U.widen(U.to_host(g), dtype).reshape(shape), dx_ref) <= U.TIGHT[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_softmax_wide_rows_with_and_without_scratch(K, dtype):
    """Scratch is optional: without it wide rows take the one-workgroup-per-row kernels,
    with it the slice kernel; both must agree with the oracle."""
    import ctypes
    import torch
    from dragon_amd import _lib
    shape = (4, 81920)
    N, C = shape
    x, dy = _softmax_inputs(shape, dtype, 11)
    # fp64 is the judge: the oracle's sequential fp32 sum over 81920 terms is itself ~1e-4 off
    x64 = np.asarray(U.widen(x, dtype), np.float64).reshape(shape)
    e64 = np.exp(x64 - x64.max(1, keepdims=True))
    y_ref = e64 / e64.sum(1, keepdims=True)
    xd = U.to_device(x, dtype)
    lib, tag = _lib.lib(), K.dtype_tag(xd)
    need = lib.dragon_hip_softmax_scratch_bytes(tag, N, 1, C)
    assert need > 0
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for scratch in (None, torch.empty(need, dtype=torch.uint8, device="cuda")):
        y = empty(shape, dtype)
        ptr = ctypes.c_void_p(scratch.data_ptr()) if scratch is not None else None
        st = lib.dragon_hip_softmax(tag, N, 1, C, ctypes.c_void_p(xd.data_ptr()),
                                    ctypes.c_void_p(y.data_ptr()), ptr,
                                    need if scratch is not None else 0, stream)
        assert st == 0
        yw = U.widen(U.to_host(y), dtype).reshape(shape)
        assert U.rowwise_normwise(yw, y_ref) <= U.TIGHT[dtype]
        outs.append(yw)
    # too little scratch is the same as none
    y = empty(shape, dtype)
    small = torch.empty(16, dtype=torch.uint8, device="cuda")
    assert lib.dragon_hip_softmax(tag, N, 1, C, ctypes.c_void_p(xd.data_ptr()),
                                  ctypes.c_void_p(y.data_ptr()), ctypes.c_void_p(small.data_ptr()),
                                  16, stream) == 0
    assert np.array_equal(U.widen(U.to_host(y), dtype).reshape(shape), outs[0])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shift_x,shift_y", [(1, 1), (3, 3), (1, 0), (0, 5)])
def test_softmax_short_rows_at_shifted_bases(K, dtype, shift_x, shift_y):
    """Input and output that start a few elements past a 16-byte boundary: equal shifts take the
    staged short-row kernels (whose first and last packet reach outside the tensors), unequal
    shifts the register tiles."""
    shape = (37, 197)
    N, C = shape
    x, dy = _softmax_inputs(shape, dtype, 21)
    x64 = np.asarray(U.widen(x, dtype), np.float64).reshape(shape)
    e64 = np.exp(x64 - x64.max(1, keepdims=True))
    y_ref = e64 / e64.sum(1, keepdims=True)
    guard = 8

    def shifted(shift, bits=None):
        buf = empty((N * C + shift + guard,), dtype)
        buf.zero_()
        view = buf[shift:shift + N * C].view(N, C)
        if bits is not None:
            view.copy_(U.to_device(bits, dtype))
        return buf, view

    _, xd = shifted(shift_x, x)
    ybuf, y = shifted(shift_y)
    K.softmax(N, 1, C, xd, y)
    yw = U.widen(U.to_host(y.contiguous()), dtype).reshape(shape)
    assert U.rowwise_normwise(yw, y_ref) <= U.TIGHT[dtype]
    # nothing outside the output was written
    flat = U.widen(U.to_host(ybuf), dtype).ravel()
    assert np.all(flat[:shift_y] == 0) and np.all(flat[shift_y + N * C:] == 0)
    _, dyd = shifted(shift_x, dy)
    dxbuf, dx = shifted(shift_x)
    _, yin = shifted(shift_x, U.to_host(y.contiguous()).reshape(shape))
    K.softmax_grad(N, 1, C, dyd, yin, dx)
    dy64 = np.asarray(U.widen(dy, dtype), np.float64).reshape(shape)
    y64 = np.asarray(yw, np.float64)
    dx_ref = (dy64 - (dy64 * y64).sum(1, keepdims=True)) * y64
    assert U.normwise(U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape), dx_ref) <= U.TIGHT[dtype]
    flat = U.widen(U.to_host(dxbuf), dtype).ravel()
    assert np.all(flat[:shift_x] == 0) and np.all(flat[shift_x + N * C:] == 0)


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("C", [16411, 20001, 30522, 50257])
@pytest.mark.parametrize("shift_x,shift_y", [(0, 0), (3, 3), (1, 0)])
def test_softmax_wide_rows_that_are_not_whole_packets(K, C, dtype, shift_x, shift_y, log):
    """Vocabulary-sized rows whose width or base address is not a multiple of 16 bytes (the
    ragged register tiles, 1024 threads per row and up to sixteen packets per thread; in the
    backward pass, with congruent tensors, the aligned packets that cover a row), with equal
    and unequal shifts of input and output. What surrounds the inputs is poisoned (a huge
    logit, NaN for the backward) and must not leak into a row; against fp64, and nothing
    outside the outputs may be written."""
    N = 5
    shape = (N, C)
    x, _ = _softmax_inputs(shape, dtype, 31)
    x64 = np.asarray(U.widen(x, dtype), np.float64).reshape(shape)
    e64 = np.exp(x64 - x64.max(1, keepdims=True))
    y_ref = e64 / e64.sum(1, keepdims=True)
    if log:
        y_ref = (x64 - x64.max(1, keepdims=True)) - np.log(e64.sum(1, keepdims=True))
    guard = 24

    def shifted(shift, bits=None, fill=0.0):
        buf = empty((N * C + shift + guard,), dtype)
        buf.fill_(fill)
        view = buf[shift:shift + N * C].view(N, C)
        if bits is not None:
            view.copy_(U.to_device(bits, dtype))
        return buf, view

    # what lies around the input must not leak into the rows: poison it with a huge logit
    _, xd = shifted(shift_x, x, fill=6e4)
    ybuf, y = shifted(shift_y, fill=-7.0)
    (K.log_softmax if log else K.softmax)(N, 1, C, xd, y)
    yw = U.widen(U.to_host(y.contiguous()), dtype).reshape(shape)
    if log:
        keep = y_ref > -1e3
        assert np.max(np.abs(yw[keep] - y_ref[keep]) / (1 + np.abs(y_ref[keep]))) <= U.TIGHT[dtype]
    else:
        assert U.rowwise_normwise(yw, y_ref) <= U.TIGHT[dtype]
    flat = U.widen(U.to_host(ybuf), dtype).ravel()
    assert np.all(flat[:shift_y] == -7.0) and np.all(flat[shift_y + N * C:] == -7.0)
    # backward from the forward's own output; what surrounds dy and y is NaN and must not
    # reach a row's sum
    _, dyb = _softmax_inputs(shape, dtype, 32)
    dy64 = np.asarray(U.widen(dyb, dtype), np.float64).reshape(shape)
    _, dyd = shifted(shift_x, dyb, fill=float("nan"))
    _, yin = shifted(shift_x, U.to_host(y.contiguous()).reshape(shape), fill=float("nan"))
    dxbuf, dx = shifted(shift_y, fill=-7.0)
    (K.log_softmax_grad if log else K.softmax_grad)(N, 1, C, dyd, yin, dx)
    dxw = U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape)
    dx_ref = (dy64 - np.exp(yw) * dy64.sum(1, keepdims=True)) if log else \
        (dy64 - (dy64 * yw).sum(1, keepdims=True)) * yw
    assert np.all(np.isfinite(dxw))
    assert U.normwise(dxw, dx_ref) <= U.TIGHT[dtype]
    flat = U.widen(U.to_host(dxbuf), dtype).ravel()
    assert np.all(flat[:shift_y] == -7.0) and np.all(flat[shift_y + N * C:] == -7.0)


def test_softmax_masked_logits_are_exact_zero(K):
    x = np.zeros((4, 512), np.float32)
    x[:, ::2] = -1e4
    xd = U.to_device(R.to_bits(x, "float16"), "float16")
    y = empty((4, 512), "float16")
    K.softmax(4, 1, 512, xd, y)
    yw = U.widen(U.to_host(y), "float16")
    assert np.all(yw[:, ::2] == 0)
    assert np.allclose(yw[:, 1::2], 1 / 256, rtol=1e-3)


# one shape per kernel family: short rows in LDS, one wavefront, a workgroup, 1024-thread
# rows, several workgroups per row, column tiles and long columns (S > 1)
SPECIAL_SHAPES = [(8, 1, 37), (8, 1, 64), (8, 1, 512), (8, 1, 1000), (8, 1, 4096), (8, 1, 8200),
                  (8, 1, 40000), (8, 1, 131072), (8, 5, 21), (8, 3, 2000)]


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("N,S,C", SPECIAL_SHAPES)
def test_softmax_special_values_follow_the_reference(K, N, S, C, dtype, log):
    """Rows holding -inf everywhere, one +inf, one nan, a finite mask everywhere, -inf in one
    half, and one huge logit: nan and inf must appear exactly where the CPU kernels put them
    (max-subtraction turns inf - inf into nan: softmax_kernel.cc's row maximum then exp), in
    the forward and in the backward that consumes such an output."""
    rng = U.rng_for(C)
    x = (rng.standard_normal((N, C, S)) * 3).astype(np.float32)
    x[0, :, 0] = -np.inf
    x[1, C // 2, 0] = np.inf
    x[2, C - 1, 0] = np.nan
    x[3, :, 0] = -1e4
    x[4, : C // 2, 0] = -np.inf
    x[5, 0, 0] = 6e4
    xb = R.to_bits(x, dtype)
    xo, od = oracle_dtype_inputs(xb, dtype)

    def stored(a):
        """An fp32 oracle result as the I/O type stores it."""
        a = np.asarray(a, np.float32).reshape(N, C, S)
        return U.widen(R.to_bits(a, dtype), dtype) if dtype != "float32" else a.astype(np.float64)

    def same_specials(got, want):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.isinf(got), np.isinf(want))
        assert np.array_equal(got[np.isinf(got)], want[np.isinf(want)])

    want = stored((R.log_softmax if log else R.softmax)(od, N, S, C, np.asarray(xo, np.float32)))
    y = empty((N, C, S), dtype)
    (K.log_softmax if log else K.softmax)(N, S, C, U.to_device(xb, dtype), y)
    got = U.widen(U.to_host(y), dtype)
    same_specials(got, want)
    # finite values to the usual bar, per slice relative to its maximum, against fp64 and
    # against the oracle (whose sequential fp32 sum of a long row is itself 1e-5 to 1e-4 off)
    x64 = np.asarray(xo, np.float64).reshape(N, C, S)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        z = x64 - x64.max(1, keepdims=True)
        y64 = z - np.log(np.exp(z).sum(1, keepdims=True)) if log else \
            np.exp(z) / np.exp(z).sum(1, keepdims=True)
    for n in range(N):
        for s in range(S):
            w, g, e = want[n, :, s], got[n, :, s], y64[n, :, s]
            fin = np.isfinite(w) & np.isfinite(e)
            if fin.any():
                scale = max(np.max(np.abs(w[fin])), 1e-30)
                e_go = np.max(np.abs(g[fin] - w[fin])) / scale
                e_ge = np.max(np.abs(g[fin] - e[fin])) / scale
                e_oe = np.max(np.abs(w[fin] - e[fin])) / scale
                assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (n, s)

    yb = R.to_bits(want.astype(np.float32), dtype)
    dyb = R.to_bits(rng.standard_normal((N, C, S)).astype(np.float32), dtype)
    yo, _ = oracle_dtype_inputs(yb, dtype)
    dyo, _ = oracle_dtype_inputs(dyb, dtype)
    want_dx = stored((R.log_softmax_grad if log else R.softmax_grad)(
        od, N, S, C, np.asarray(dyo, np.float32), np.asarray(yo, np.float32)))
    dx = empty((N, C, S), dtype)
    (K.log_softmax_grad if log else K.softmax_grad)(N, S, C, U.to_device(dyb, dtype),
                                                   U.to_device(yb, dtype), dx)
    same_specials(U.widen(U.to_host(dx), dtype), want_dx)


# ---------------------------------------------------------------- LayerNorm backward

LNB_SHAPES = [(64, 1024), (33, 1000), (16, 12288), (300, 48), (5, 37), (1100, 256), (40, 4096),
              (3, 20000), (2, 8),
              # short and odd rows staged through LDS: several ranges per workgroup, 8 to 64
              # lanes per row, a last range that is not full
              (5000, 64), (700, 197), (130, 577), (9000, 16),
              # wider rows that are not whole packets: the ragged flavour of the fused kernel
              (70, 1030), (300, 4097), (33, 12289),
              # rows beyond the register tiles: row sums, then dx with column partials
              # (packets; elements for the odd width; a row cut over several workgroups)
              (40, 33000), (19, 40001), (2, 300000)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16", "float64"])
@pytest.mark.parametrize("shape", LNB_SHAPES)
def test_layer_norm_backward(K, dtype, shape):
    N, C = shape
    rng = U.rng_for(300 + C)
    x = (rng.standard_normal(shape)).astype(np.float32)
    x[rng.random(shape) < 0.01] *= 50
    x = R.to_bits(x, dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    an = acc_name(dtype)
    _, mu, rsig = R.layer_norm(dtype, x, g, b, 1e-5)
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    dx_ref, dg_ref, db_ref, ds_ref, dbb_ref = R.group_norm_grad(od, N, 1, C, 1, "NHWC", xo, mu, rsig, g, dyo)
    params = empty((2 * N,), an)
    dg, db, dx = empty((C,), an), empty((C,), an), empty(shape, dtype)
    K.group_norm_grad(N, 1, C, 1, "NHWC", U.to_device(x, dtype), U.to_device(mu, an),
                      U.to_device(rsig, an), U.to_device(g, an), U.to_device(dy, dtype),
                      params, params, dg, db, dx)
    tol = U.TIGHT[dtype]
    assert U.normwise(U.widen(U.to_host(dx), dtype), dx_ref) <= tol
    ptol = 1e-12 if dtype == "float64" else 2e-5
    assert U.normwise(U.to_host(dg), dg_ref) <= ptol
    assert U.normwise(U.to_host(db), db_ref) <= ptol
    p = U.to_host(params)
    assert U.normwise(p[:N], ds_ref) <= ptol and U.normwise(p[N:], dbb_ref) <= ptol


# ---------------------------------------------------------------- GroupNorm

GN_CASES = [((2, 32, 8, 8), 1, 4), ((3, 12, 5), 1, 3), ((2, 6, 6, 16), -1, 4), ((3, 5, 12), -1, 3),
            ((2, 64, 16, 16), 1, 32), ((4, 8), -1, 2), ((2, 16, 4, 4), 1, 0), ((1, 4, 2), 1, 2),
            # groups that take the register-resident fused kernels
            ((2, 32, 32, 32), 1, 4), ((2, 16, 64, 64), 1, 2), ((3, 6, 32, 16), 1, 3),
            ((2, 8, 64, 128), 1, 8), ((1, 4, 128, 128), 1, 2),
            # spatial sizes that are not whole packets: ragged fused forward, per-(n, c) sums
            ((4, 32, 7, 7), 1, 4), ((2, 24, 14, 14), 1, 3), ((2, 3, 70, 70), 1, 0),
            # rows beyond the register tiles: the looped per-(n, c) sums
            ((1, 2, 300, 301), 1, 2),
            # groups beyond one workgroup's registers: slices of a group held by several
            # workgroups that exchange their partial sums (12 and 16+ slices per group)
            ((2, 6, 128, 128), 1, 2), ((2, 8, 256, 256), 1, 2),
            # channels of 64 or more packets that are not whole wavefronts of packets: the
            # fused backward splits a wavefront's packets between two channels
            ((2, 16, 28, 28), 1, 4), ((2, 64, 56, 56), 1, 8), ((1, 6, 24, 24), 1, 2),
            # channels of a few packets: several channels per wavefront in the fused backward
            ((2, 64, 16, 16), 1, 4), ((3, 48, 8, 8), 1, 2),
            # odd feature maps of more than 1024 elements in every dtype: one wavefront per
            # (n, c) row in the backward and the map; per group row in the forward statistics
            # of groups beyond the register tiles
            ((2, 6, 33, 35), 1, 2), ((1, 2, 301, 303), 1, 2),
            # 14x14 and 7x7 maps in groups of whole packets: the fused backward with one LDS
            # entry per packet (up to 100 KB of dynamic LDS in fp64)
            ((2, 64, 14, 14), 1, 2), ((3, 128, 7, 7), 1, 4),
            # channels of 64 packets' worth or more that are not whole packets, in groups that
            # are: a wavefront's packets split between two channels inside one packet (or, for
            # (2, 8, 4, 257) in 16-bit types, inside one and between two by turns)
            ((2, 32, 35, 35), 1, 4), ((2, 16, 23, 23), 1, 2), ((1, 32, 63, 63), 1, 4),
            ((2, 8, 4, 257), 1, 2),
            # NHWC samples that fit one workgroup's registers (fused forward: 1, 7-8 and 13
            # packets per thread; 12 of every 1024 threads idle; more samples than workgroups,
            # so that the backward's per-channel shares accumulate over several samples)
            ((2, 14, 14, 64), -1, 4), ((3, 5, 7, 96), -1, 4), ((2, 28, 28, 64), -1, 2),
            ((700, 4, 4, 32), -1, 2),
            # the same with groups of 10 and 12 channels: a packet of the fused NHWC forward
            # and backward lies in two groups (and more samples than workgroups)
            ((2, 7, 7, 320), -1, 32), ((3, 6, 5, 96), -1, 8), ((5, 9, 9, 160), -1, 16),
            ((1100, 3, 3, 40), -1, 4),
            # NHWC samples beyond one workgroup's registers: slices of whole rows that exchange
            # their groups' sums (8 to 32 slices per sample; a ragged last slice and idle
            # threads; fewer slices than groups and more; more items than workgroups)
            ((2, 64, 64, 64), -1, 8), ((3, 40, 41, 96), -1, 4), ((1, 48, 48, 256), -1, 32),
            ((70, 48, 48, 64), -1, 8),
            # rows of 160 / 320 packets leave too many of a slice workgroup's threads without a
            # row: the column reductions
            ((2, 40, 41, 1280), -1, 32),
            # groups narrower than a packet: a share per channel of the packet (and more samples
            # than workgroups)
            ((2, 14, 14, 128), -1, 32), ((3, 6, 6, 64), -1, 32), ((600, 4, 4, 96), -1, 32),
            ((1100, 3, 3, 32), -1, 8),
            # more narrow groups than the team sums take (512): the column reductions
            ((2, 4, 4, 1024), -1, 512),
            # small groups, a wavefront each in the fused backward: more channels per group
            # than lanes, three channels per group, more groups than the grid's wavefronts hold
            ((2, 160, 3, 3), 1, 2), ((5, 96, 8, 8), 1, 32), ((40, 64, 14, 14), 1, 32),
            # thousands of groups of at most 32 packets: several groups per wavefront in the
            # forward (staged through LDS), channels that are and are not whole packets
            ((140, 64, 8, 8), 1, 32), ((130, 96, 5, 5), 1, 32)]


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16", "float64"])
@pytest.mark.parametrize("shape,axis,group", GN_CASES)
def test_group_norm_forward_backward(K, shape, axis, group, dtype, fused):
    rng = U.rng_for(400 + len(shape) + group)
    ax = axis % len(shape)
    N, C = shape[0], shape[ax]
    S = int(np.prod(shape)) // N // C
    G = group if group > 0 else C
    D = C // G
    layout = "NHWC" if ax + 1 == len(shape) else "NCHW"
    an = acc_name(dtype)
    x = R.to_bits((rng.standard_normal(shape) + 0.3).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    y_ref, mu_ref, rsig_ref = R.op_group_norm(dtype, x, g, b, axis, group, 1e-5)
    xd, gd, bd = U.to_device(x, dtype), U.to_device(g, an), U.to_device(b, an)
    mu, rsig, y = empty((N * G,), an), empty((N * G,), an), empty(shape, dtype)
    if fused:
        K.group_norm_forward(N, G, D, S, layout, 1e-5, xd, gd, bd, mu, rsig, y)
    else:  # the operator's own sequence: Moments -> InvStd -> GroupNorm
        if layout == "NCHW":
            K.moments([N * G, D * S], [1], xd, mu, rsig)
        else:
            K.moments([N, S, G, D], [1, 3], xd, mu, rsig)
        K.inv_std(N * G, 1e-5, rsig, rsig)
        K.group_norm(N, G, D, S, layout, xd, mu, rsig, gd, bd, y)
    stat_tol = 1e-12 if dtype == "float64" else 1e-5
    # groups of ~1e5 elements put the oracle's sequential fp32 sums themselves off: three-way
    x64 = np.asarray(U.widen(x, dtype), np.float64)
    xg = (x64.reshape(N, G, D * S) if layout == "NCHW"
          else x64.reshape(N, S, G, D).transpose(0, 2, 1, 3).reshape(N, G, S * D))
    mu64 = xg.mean(-1).ravel()
    rsig64 = 1.0 / np.sqrt(xg.var(-1).ravel() + np.float64(np.float32(1e-5)))
    ok, *errs = U.close3(U.to_host(mu), mu_ref, mu64, stat_tol)
    assert ok, errs
    e_go = np.max(np.abs(U.to_host(rsig) / rsig_ref - 1))
    e_ge = np.max(np.abs(U.to_host(rsig) / rsig64 - 1))
    e_oe = np.max(np.abs(rsig_ref / rsig64 - 1))
    assert e_ge <= stat_tol and e_go <= stat_tol + e_oe, (e_go, e_ge, e_oe)
    # y inherits the statistics' error: three-way as well
    g64, b64 = np.asarray(g, np.float64), np.asarray(b, np.float64)
    xh = (xg - mu64.reshape(N, G, 1)) * rsig64.reshape(N, G, 1)
    if layout == "NCHW":
        y64 = xh.reshape(N, C, S) * g64[None, :, None] + b64[None, :, None]
    else:
        y64 = xh.reshape(N, G, S, D).transpose(0, 2, 1, 3).reshape(N, S, C) * g64 + b64
    ok, *errs = U.close3(U.widen(U.to_host(y), dtype).reshape(y64.shape),
                         np.asarray(U.widen(y_ref, dtype)).reshape(y64.shape), y64, U.TIGHT[dtype])
    assert ok, errs
    if fused:
        return
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    dx_ref, dg_ref, db_ref, ds_ref, dbb_ref = R.group_norm_grad(
        od, N, G, D, S, layout, xo, mu_ref, rsig_ref, g, dyo)
    params = empty((2 * N * G,), an)
    dg, db, dx = empty((C,), an), empty((C,), an), empty(shape, dtype)
    K.group_norm_grad(N, G, D, S, layout, xd, U.to_device(mu_ref, an), U.to_device(rsig_ref, an), gd,
                      U.to_device(dy, dtype), params, params, dg, db, dx)
    ptol = 1e-12 if dtype == "float64" else 2e-5
    assert U.normwise(U.widen(U.to_host(dx), dtype), dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(U.to_host(dg), dg_ref) <= ptol
    assert U.normwise(U.to_host(db), db_ref) <= ptol
    p = U.to_host(params)
    assert U.normwise(p[:N * G], ds_ref) <= ptol and U.normwise(p[N * G:], dbb_ref) <= ptol


# ---------------------------------------------------------------- BatchNorm

# The NCHW shapes from (8, 40, 56, 56) on take the single-read path: channels of 100 KB in
# fp32, which one 512- or 1024-thread workgroup holds whole (a single slice of the 256-thread
# kernel in 16-bit types) where there are at least as many channels as compute units, else
# slices; 1100 single-slice channels over two rounds; 260 channels of 135 KB (whole on 1024
# threads forward, slices that exchange their sums backward) and 40 of 300 KB (slices either way).
BN_CASES = [((8, 16, 7, 7), 1), ((4, 3, 2), 1), ((16, 32), -1), ((4, 5, 5, 24), -1),
            ((6, 64, 28, 28), 1), ((4, 2, 3), -1), ((3, 130, 4), 1), ((50, 70), -1),
            ((8, 40, 56, 56), 1), ((2, 1100, 16, 16), 1), ((32, 350, 28, 28), 1),
            ((11, 260, 56, 56), 1), ((24, 40, 56, 56), 1),
            # feature maps that are not whole packets: (n, c) rows staged through LDS, several
            # ranges per workgroup ((8, 16, 7, 7) and (4, 3, 2) above take the same path)
            ((16, 96, 14, 14), 1), ((12, 200, 7, 7), 1), ((3, 33, 30, 30), 1),
            # longer rows of that kind: one wavefront per (n, c) row, leading and trailing
            # elements of a row moved one by one around its aligned packets
            ((5, 24, 35, 35), 1), ((3, 10, 71, 71), 1)]


@pytest.mark.parametrize("dtype", ["float32", "float64", "bfloat16", "float16"])
@pytest.mark.parametrize("shape,axis", BN_CASES)
def test_batch_norm_training(K, shape, axis, dtype):
    rng = U.rng_for(500 + len(shape))
    ax = axis % len(shape)
    N, C = shape[0], shape[ax]
    S = int(np.prod(shape)) // N // C
    layout = "NHWC" if ax + 1 == len(shape) else "NCHW"
    an = acc_name(dtype)
    x = R.to_bits((2 * rng.standard_normal(shape) + 0.5).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    rm0 = (rng.standard_normal(C) * 0.1).astype(U.acc_np(dtype))
    rv0 = rng.uniform(0.5, 1.5, C).astype(U.acc_np(dtype))
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    rm_ref, rv_ref = rm0.copy(), rv0.copy()
    y_ref, mu_ref, rsig_ref, params_ref = R.op_batch_norm_train(
        od, np.asarray(xo).reshape(shape), g, b, rm_ref, rv_ref, axis, 0.9, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_train_grad(
        od, np.asarray(xo).reshape(shape), g, np.asarray(dyo).reshape(shape), mu_ref, rsig_ref, axis)

    xd, gd, bd = U.to_device(x, dtype), U.to_device(g, an), U.to_device(b, an)
    stat_tol = 1e-12 if dtype == "float64" else 1e-5

    # Channels of tens of thousands of elements put the oracle's sequential fp32 sums
    # themselves off: the distance to the oracle may exceed the tolerance by the oracle's own
    # distance to the fp64 statistics, no more.
    x64 = np.moveaxis(np.asarray(U.widen(x, dtype), np.float64).reshape(shape), ax, 1).reshape(N, C, S)
    mean64 = x64.mean((0, 2))
    rsig64 = 1 / np.sqrt(((x64 - mean64[None, :, None]) ** 2).mean((0, 2)) + np.float64(np.float32(1e-5)))
    slack_mu = U.normwise(mu_ref, mean64)
    slack_rs = float(np.max(np.abs(np.asarray(rsig_ref, np.float64) / rsig64 - 1)))

    def check_forward(mu, rsig, params, rm, rv, y):
        assert U.normwise(U.to_host(mu), mu_ref) <= stat_tol + slack_mu
        assert np.max(np.abs(U.to_host(rsig) / rsig_ref - 1)) <= stat_tol + slack_rs
        assert U.normwise(U.to_host(params), params_ref) <= stat_tol + slack_mu + slack_rs
        assert U.normwise(U.to_host(rm), rm_ref) <= stat_tol + slack_mu
        assert U.normwise(U.to_host(rv), rv_ref) <= stat_tol + 2 * slack_rs
        # 16-bit y is compared with the fp32 reference result (the CPU has no 16-bit BatchNorm)
        assert U.normwise(U.widen(U.to_host(y), dtype), y_ref) <= U.TIGHT[dtype]

    # (a) the operator's own sequence: Moments, Axpby x2, InvStd, BatchNorm
    mu, rsig, params = empty((C,), an), empty((C,), an), empty((2 * C,), an)
    rm, rv, y = U.to_device(rm0, an), U.to_device(rv0, an), empty(shape, dtype)
    if layout == "NCHW":
        K.moments([N, C, S], [0, 2], xd, mu, rsig)
    else:
        K.moments([N * S, C], [0], xd, mu, rsig)
    one_minus = float(np.float32(1.0) - np.float32(0.9))  # `1.f - decay`, batch_norm_op.cc:60-63
    K.axpby(C, one_minus, mu, 0.9, rm)
    K.axpby(C, one_minus, rsig, 0.9, rv)
    K.inv_std(C, 1e-5, rsig, rsig)
    K.batch_norm(N, C, S, layout, xd, mu, rsig, gd, bd, params, params, y)
    check_forward(mu, rsig, params, rm, rv, y)

    # (b) the fused training forward
    mu2, rsig2, params2 = empty((C,), an), empty((C,), an), empty((2 * C,), an)
    rm2, rv2, y2 = U.to_device(rm0, an), U.to_device(rv0, an), empty(shape, dtype)
    K.batch_norm_training_forward(N, C, S, layout, 0.9, 1e-5, xd, gd, bd, rm2, rv2, mu2, rsig2,
                                  params2, y2)
    check_forward(mu2, rsig2, params2, rm2, rv2, y2)

    # backward: WGrad into the packed params buffer, then TrainingGrad
    dyd = U.to_device(dy, dtype)
    mud, rsd = U.to_device(mu_ref, an), U.to_device(rsig_ref, an)
    wg, dx = empty((2 * C,), an), empty(shape, dtype)
    K.batch_norm_wgrad(N, C, S, layout, xd, mud, rsd, dyd, wg, wg)
    ptol = 1e-12 if dtype == "float64" else 2e-5
    w = U.to_host(wg)
    assert U.normwise(w[:C], dg_ref) <= ptol and U.normwise(w[C:], db_ref) <= ptol
    wref = U.to_device(np.concatenate([dg_ref, db_ref]).astype(U.acc_np(dtype)), an)
    K.batch_norm_training_grad(N, C, S, float(N * S), layout, xd, mud, rsd, gd, wref, wref, dyd, dx)
    assert U.normwise(U.widen(U.to_host(dx), dtype), dx_ref) <= U.TIGHT[dtype]

    # the two as one call (x and dy read once where a channel slice fits the registers)
    wg2, dx2 = empty((2 * C,), an), empty(shape, dtype)
    K.batch_norm_training_backward(N, C, S, float(N * S), layout, xd, mud, rsd, gd, dyd, wg2, wg2, dx2)
    w2 = U.to_host(wg2)
    assert U.normwise(w2[:C], dg_ref) <= ptol and U.normwise(w2[C:], db_ref) <= ptol
    assert U.normwise(U.widen(U.to_host(dx2), dtype), dx_ref) <= U.TIGHT[dtype]


# (N, C, H, W): slices per channel and rounds of work items as in BN_CASES above, on maps
# that are not whole packets
BN_WINDOW_CASES = [(8, 40, 57, 57), (2, 1100, 15, 15), (32, 350, 27, 27), (4, 24, 35, 35),
                   (3, 10, 71, 71), (16, 96, 14, 14), (11, 260, 57, 57), (24, 40, 57, 57)]


@pytest.mark.parametrize("shift,shift_out", [(0, 0), (1, 1), (3, 3), (5, 5), (2, 0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("N,C,H,W", BN_WINDOW_CASES)
def test_batch_norm_training_on_maps_that_are_not_whole_packets(K, N, C, H, W, dtype, shift,
                                                                shift_out):
    """NCHW feature maps whose (n, c) runs are not whole 16-byte packets, at bases shifted by
    whole elements: the single-read kernels take the aligned packets that cover each run
    (inputs and outputs shifted alike), or the call goes the split way (shifted differently).
    What surrounds the inputs is NaN and must not reach a channel's sums; nothing outside the
    outputs may be written; the backward may overwrite dy."""
    shape, S = (N, C, H, W), H * W
    rng = U.rng_for(540 + N + H)
    an = acc_name(dtype)
    x = R.to_bits((2 * rng.standard_normal(shape) + 0.5).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    rm0 = (rng.standard_normal(C) * 0.1).astype(np.float32)
    rv0 = rng.uniform(0.5, 1.5, C).astype(np.float32)
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    rm_ref, rv_ref = rm0.copy(), rv0.copy()
    y_ref, mu_ref, rsig_ref, params_ref = R.op_batch_norm_train(
        od, np.asarray(xo).reshape(shape), g, b, rm_ref, rv_ref, 1, 0.9, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_train_grad(
        od, np.asarray(xo).reshape(shape), g, np.asarray(dyo).reshape(shape), mu_ref, rsig_ref, 1)
    n, guard = N * C * S, 24

    def shifted(shift, bits=None, fill=0.0):
        buf = empty((n + shift + guard,), dtype)
        buf.fill_(fill)
        view = buf[shift:shift + n].view(shape)
        if bits is not None:
            view.copy_(U.to_device(bits, dtype).view(shape))
        return buf, view

    def untouched(buf, shift):
        flat = U.widen(U.to_host(buf), dtype).ravel()
        return np.all(flat[:shift] == -7.0) and np.all(flat[shift + n:] == -7.0)

    _, xd = shifted(shift, x, fill=float("nan"))
    _, dyd = shifted(shift, dy, fill=float("nan"))
    gd, bd = U.to_device(g, an), U.to_device(b, an)
    mu, rsig, params = empty((C,), an), empty((C,), an), empty((2 * C,), an)
    rm, rv = U.to_device(rm0, an), U.to_device(rv0, an)
    ybuf, y = shifted(shift_out, fill=-7.0)
    K.batch_norm_training_forward(N, C, S, "NCHW", 0.9, 1e-5, xd, gd, bd, rm, rv, mu, rsig, params, y)
    # (channels of tens of thousands of elements: the oracle's own distance to the fp64
    # statistics is allowed on top of the tolerance, as in test_batch_norm_training)
    x64 = np.asarray(U.widen(x, dtype), np.float64).reshape(N, C, S)
    mean64 = x64.mean((0, 2))
    rsig64 = 1 / np.sqrt(((x64 - mean64[None, :, None]) ** 2).mean((0, 2)) + np.float64(np.float32(1e-5)))
    slack_mu = U.normwise(mu_ref, mean64)
    slack_rs = float(np.max(np.abs(np.asarray(rsig_ref, np.float64) / rsig64 - 1)))
    assert U.normwise(U.to_host(mu), mu_ref) <= 1e-5 + slack_mu
    assert np.max(np.abs(U.to_host(rsig) / rsig_ref - 1)) <= 1e-5 + slack_rs
    assert U.normwise(U.to_host(params), params_ref) <= 1e-5 + slack_mu + slack_rs
    assert U.normwise(U.to_host(rm), rm_ref) <= 1e-5 + slack_mu
    assert U.normwise(U.to_host(rv), rv_ref) <= 1e-5 + 2 * slack_rs
    assert U.normwise(U.widen(U.to_host(y.contiguous()), dtype), y_ref) <= U.TIGHT[dtype]
    assert untouched(ybuf, shift_out)

    mud, rsd = U.to_device(mu_ref, an), U.to_device(rsig_ref, an)
    wg = empty((2 * C,), an)
    dxbuf, dx = shifted(shift_out, fill=-7.0)
    K.batch_norm_training_backward(N, C, S, float(N * S), "NCHW", xd, mud, rsd, gd, dyd, wg, wg, dx)
    w = U.to_host(wg)
    assert U.normwise(w[:C], dg_ref) <= 2e-5 and U.normwise(w[C:], db_ref) <= 2e-5
    got = U.to_host(dx.contiguous())
    assert U.normwise(U.widen(got, dtype), dx_ref) <= U.TIGHT[dtype]
    assert untouched(dxbuf, shift_out)
    # the separate entry points (the operator's own sequence): element-wise maps over the
    # aligned packets that cover the tensor
    y2buf, y2 = shifted(shift_out, fill=-7.0)
    K.batch_norm(N, C, S, "NCHW", xd, mud, rsd, gd, bd, params, params, y2)
    assert U.normwise(U.widen(U.to_host(y2.contiguous()), dtype), y_ref) <= U.TIGHT[dtype]
    assert untouched(y2buf, shift_out)
    wref = U.to_device(np.concatenate([dg_ref, db_ref]).astype(np.float32), an)
    dx2buf, dx2 = shifted(shift_out, fill=-7.0)
    K.batch_norm_training_grad(N, C, S, float(N * S), "NCHW", xd, mud, rsd, gd, wref, wref, dyd, dx2)
    assert U.normwise(U.widen(U.to_host(dx2.contiguous()), dtype), dx_ref) <= U.TIGHT[dtype]
    assert untouched(dx2buf, shift_out)
    dx3buf, dx3 = shifted(shift_out, fill=-7.0)
    K.batch_norm_inference_grad(N, C, S, "NCHW", xd, mud, rsd, gd, dyd, None, None, dx3)
    want = np.asarray(dyo, np.float64).reshape(shape) * (
        np.asarray(g, np.float64) * np.asarray(rsig_ref, np.float64))[None, :, None, None]
    assert U.normwise(U.widen(U.to_host(dx3.contiguous()), dtype), want) <= U.TIGHT[dtype]
    assert untouched(dx3buf, shift_out)
    if shift == shift_out:
        # dx over dy: the same bits, and the guards around dy still as they were
        inbuf, dyin = shifted(shift, dy, fill=-7.0)
        wg2 = empty((2 * C,), an)
        K.batch_norm_training_backward(N, C, S, float(N * S), "NCHW", xd, mud, rsd, gd, dyin, wg2, wg2,
                                       dyin)
        assert np.array_equal(U.to_host(dyin.contiguous()), got)
        assert np.array_equal(U.to_host(wg2), w)
        assert untouched(inbuf, shift)


def _same_specials(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(np.isinf(got), np.isinf(want))
    assert np.array_equal(got[np.isinf(got)], want[np.isinf(want)])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,axis", [((4, 6, 8, 8), 1), ((3, 5, 7, 7), 1), ((2, 4, 150, 150), 1),
                                        ((4, 8, 8, 6), -1), ((64, 6, 56, 56), 1), ((9, 40), 1)])
def test_batch_norm_special_values_follow_the_reference(K, shape, axis, dtype):
    """A channel whose first sample is -inf, one holding +inf and one holding nan: batch and
    running statistics, fused parameters and y carry inf / nan exactly where the CPU operator's
    do (batch_norm_op.cc:49-82); the clean channels stay within the usual bar."""
    rng = U.rng_for(520 + len(shape))
    ax = axis % len(shape)
    N, C = shape[0], shape[ax]
    S = int(np.prod(shape)) // N // C
    layout = "NHWC" if ax + 1 == len(shape) and len(shape) > 2 else "NCHW"
    xf = (2 * rng.standard_normal(shape) + 0.5).astype(np.float32)
    xc = np.moveaxis(xf, ax, 0)           # [C, ...] view
    xc[0].reshape(-1)[0] = -np.inf         # the sample the shifted sums start from
    xc[2].reshape(-1)[xc[2].size // 2] = np.inf
    xc[3].reshape(-1)[-1] = np.nan
    x = R.to_bits(xf, dtype)
    g, b = U.affine_params(rng, C, dtype)
    rm0 = (rng.standard_normal(C) * 0.1).astype(np.float32)
    rv0 = rng.uniform(0.5, 1.5, C).astype(np.float32)
    xo, od = oracle_dtype_inputs(x, dtype)
    rm_ref, rv_ref = rm0.copy(), rv0.copy()
    y_ref, mu_ref, rsig_ref, params_ref = R.op_batch_norm_train(
        od, np.asarray(xo).reshape(shape), g, b, rm_ref, rv_ref, axis, 0.9, 1e-5)
    mu, rsig, params = empty((C,), "float32"), empty((C,), "float32"), empty((2 * C,), "float32")
    rm, rv, y = U.to_device(rm0, "float32"), U.to_device(rv0, "float32"), empty(shape, dtype)
    K.batch_norm_training_forward(N, C, S, layout, 0.9, 1e-5, U.to_device(x, dtype),
                                  U.to_device(g, "float32"), U.to_device(b, "float32"), rm, rv, mu,
                                  rsig, params, y)
    _same_specials(U.to_host(mu), mu_ref)
    _same_specials(U.to_host(rsig), rsig_ref)
    _same_specials(U.to_host(rm), rm_ref)
    _same_specials(U.to_host(rv), rv_ref)
    _same_specials(U.to_host(params), params_ref)
    yw = U.widen(U.to_host(y), dtype).reshape(shape)
    yr = np.asarray(R.to_bits(np.asarray(y_ref, np.float32), dtype) if dtype != "float32" else y_ref)
    yr = U.widen(yr, dtype).reshape(shape) if dtype != "float32" else np.asarray(y_ref, np.float64).reshape(shape)
    _same_specials(yw, yr)
    clean = [c for c in range(C) if c not in (0, 2, 3)]
    # the oracle's sequential fp32 sum over a 200704-element channel is itself 2-6e-5 off
    assert U.normwise(np.moveaxis(yw, ax, 0)[clean], np.moveaxis(yr, ax, 0)[clean]) <= max(
        U.TIGHT[dtype], 6e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,axis,group", [((4, 8, 8, 8), 1, 4), ((3, 6, 7, 7), 1, 3),
                                              ((5, 4, 150, 150), 1, 2), ((4, 8, 8, 8), -1, 4),
                                              ((5, 32, 64, 64), 1, 4), ((5, 6, 14, 14), 1, 0),
                                              # channels-last samples cut into slices of rows
                                              ((5, 48, 48, 64), -1, 8)])
def test_group_norm_special_values_follow_the_reference(K, shape, axis, group, dtype):
    """Groups that start with -inf, hold +inf or hold nan (group_norm_op.cc's Moments -> InvStd
    -> GroupNorm sequence on the CPU): mu, rsig and y carry inf / nan in the same places."""
    rng = U.rng_for(530 + len(shape) + group)
    ax = axis % len(shape)
    N, C = shape[0], shape[ax]
    S = int(np.prod(shape)) // N // C
    G = group if group > 0 else C
    D = C // G
    layout = "NHWC" if ax + 1 == len(shape) else "NCHW"
    xf = (rng.standard_normal(shape) + 0.3).astype(np.float32)
    xf[0].reshape(-1)[0] = -np.inf         # first element of sample 0, group 0
    xf[1].reshape(-1)[xf[1].size // 2] = np.inf
    xf[2].reshape(-1)[-1] = np.nan
    x = R.to_bits(xf, dtype)
    g, b = U.affine_params(rng, C, dtype)
    y_ref, mu_ref, rsig_ref = R.op_group_norm(dtype, x, g, b, axis, group, 1e-5)
    mu, rsig, y = empty((N * G,), "float32"), empty((N * G,), "float32"), empty(shape, dtype)
    K.group_norm_forward(N, G, D, S, layout, 1e-5, U.to_device(x, dtype), U.to_device(g, "float32"),
                         U.to_device(b, "float32"), mu, rsig, y)
    _same_specials(U.to_host(mu), mu_ref)
    _same_specials(U.to_host(rsig), rsig_ref)
    yw, yr = U.widen(U.to_host(y), dtype).reshape(shape), U.widen(y_ref, dtype).reshape(shape)
    _same_specials(yw, yr)
    assert U.normwise(yw[3:], yr[3:]) <= U.TIGHT[dtype]


@pytest.mark.parametrize("dtype", ["float32", "float64", "bfloat16"])
@pytest.mark.parametrize("shape,axis", BN_CASES[:5])
def test_batch_norm_inference_and_expectation(K, shape, axis, dtype):
    rng = U.rng_for(600 + len(shape))
    ax = axis % len(shape)
    N, C = shape[0], shape[ax]
    S = int(np.prod(shape)) // N // C
    layout = "NHWC" if ax + 1 == len(shape) else "NCHW"
    an = acc_name(dtype)
    x = R.to_bits((2 * rng.standard_normal(shape) + 0.5).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    rm = (rng.standard_normal(C) * 0.1).astype(U.acc_np(dtype))
    rv = rng.uniform(0.5, 1.5, C).astype(U.acc_np(dtype))
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    xo, dyo = np.asarray(xo).reshape(shape), np.asarray(dyo).reshape(shape)
    y_ref = R.op_batch_norm_infer(od, xo, g, b, rm, rv, axis, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_infer_grad(od, xo, g, rm, rv, dyo, axis, 1e-5)
    xd, gd, bd = U.to_device(x, dtype), U.to_device(g, an), U.to_device(b, an)
    rmd, rvd = U.to_device(rm, an), U.to_device(rv, an)
    # RunInference: InvStd into params[0:C], BatchNorm with scale == bias == rsig (3C buffer)
    params, y = empty((3 * C,), an), empty(shape, dtype)
    K.inv_std(C, 1e-5, rvd, params)
    K.batch_norm(N, C, S, layout, xd, rmd, params, gd, bd, params, params, y)
    assert U.normwise(U.widen(U.to_host(y), dtype), y_ref) <= U.TIGHT[dtype]
    p = U.to_host(params)
    rs = 1 / np.sqrt(rv.astype(np.float64) + 1e-5)
    assert np.max(np.abs(p[:C] / rs - 1)) < 1e-5 and np.max(np.abs(p[C:2 * C] / (g * rs) - 1)) < 1e-5
    # RunInference gradient
    dyd = U.to_device(dy, dtype)
    rsd, dg, db, dx = empty((C,), an), empty((C,), an), empty((C,), an), empty(shape, dtype)
    K.inv_std(C, 1e-5, rvd, rsd)
    K.batch_norm_inference_grad(N, C, S, layout, xd, rmd, rsd, gd, dyd, dg, db, dx)
    ptol = 1e-12 if dtype == "float64" else 2e-5
    assert U.normwise(U.widen(U.to_host(dx), dtype), dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(U.to_host(dg), dg_ref) <= ptol and U.normwise(U.to_host(db), db_ref) <= ptol
    dx2 = empty(shape, dtype)
    K.batch_norm_inference_grad(N, C, S, layout, xd, rmd, rsd, gd, dyd, None, None, dx2)
    assert np.array_equal(U.to_host(dx2), U.to_host(dx))
    # SyncBN statistics kernel against E[x], E[x^2] with a doubled ("two rank") normaliser
    ex, ex2 = empty((C,), an), empty((C,), an)
    K.batch_norm_expectation(N, C, S, float(2 * N * S), layout, xd, ex, ex2)
    ex_ref, ex2_ref = R.batch_norm_expectation(od, N, C, S, float(2 * N * S), layout, xo)
    assert U.normwise(U.to_host(ex), ex_ref) <= ptol and U.normwise(U.to_host(ex2), ex2_ref) <= ptol


# ---------------------------------------------------------------- Moments / math helpers

MOMENT_CASES = [((4, 5, 6), (0, 2)), ((20, 5), (0,)), ((6, 35), (1,)), ((3, 4, 2, 5), (1, 3)),
                ((3, 1, 4, 1, 5), (2, 4)), ((2, 3, 4), (0, 1, 2)), ((2, 3, 4), (1,)),
                ((5, 4, 3, 2, 2), (0, 2, 4)), ((7,), ()), ((64, 40, 49), (0, 2)),
                ((1000, 72), (0,)), ((16, 8192), (1,)), ((2, 3), (0,)), ((2, 3), (1,)),
                ((2, 3), (0, 1)),
                # thousands of short rows: staged through LDS, several rows per wavefront
                ((5000, 7), (1,)), ((4100, 300), (1,)), ((70, 64, 2), (2,)),
                # a reduced axis between kept ones, a thread per output
                ((70, 9, 300), (1,)), ((4200, 33, 4), (1,)),
                # fewer than 64 columns: the lanes a row leaves idle take adjacent rows
                ((20000, 2), (0,)), ((3000, 24), (0,)),
                # thousands of rows of a few KB: a wavefront per row through the aligned packets
                # that cover it
                ((2100, 1025), (1,)), ((2048, 4099), (1,)), ((2500, 2048), (1,)),
                # segments that are not whole packets, a workgroup or several per output
                ((40, 4097), (1,)), ((6, 10, 3137), (0, 2)), ((3, 20001), (1,))]


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape,axes", MOMENT_CASES)
def test_moments(K, shape, axes, dtype):
    rng = U.rng_for(700 + len(shape))
    x = R.to_bits((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32), dtype)
    mean_ref, var_ref = R.moments(dtype, x, list(axes))
    an = acc_name(dtype)
    mean, var = empty(mean_ref.shape, an), empty(var_ref.shape, an)
    K.moments(list(shape), list(axes), U.to_device(x, dtype), mean, var)
    tol = 1e-12 if dtype == "float64" else 1e-5
    # fp64 moments of the same (rounded) inputs: over 100000 elements the oracle's
    # sequential fp32 sums are themselves several 1e-5 off
    x64 = np.asarray(U.widen(x, dtype), np.float64).reshape(shape)
    ok, *errs = U.close3(U.to_host(mean), mean_ref, x64.mean(tuple(axes)).reshape(mean_ref.shape), tol)
    assert ok, errs
    ok, *errs = U.close3(U.to_host(var), var_ref, x64.var(tuple(axes)).reshape(var_ref.shape), tol * 2)
    assert ok, errs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape,axes", [((6, 35), (1,)), ((16, 8192), (1,)), ((6, 70000), (1,)),
                                        ((1000, 72), (0,)), ((64, 40, 49), (0, 2)),
                                        ((5000, 7), (1,)), ((70, 9, 300), (1,)),
                                        ((20000, 2), (0,)), ((2, 3, 4), (0, 1, 2)),
                                        ((2100, 1025), (1,)), ((40, 4097), (1,))])
def test_moments_special_values_follow_the_reference(K, shape, axes, dtype):
    """inf and nan among the reduced elements, the first one included (the sample the
    shifted sums are taken from): the mean is the infinity or nan that the CPU kernel's
    plain sums give, the variance nan (moments.cc:10-120: E[x^2] - E[x]^2)."""
    rng = U.rng_for(720 + len(shape))
    xf = (rng.standard_normal(shape) + 0.5).astype(np.float32)
    flat = xf.reshape(-1)
    flat[0] = -np.inf                      # first sample of the first output
    flat[flat.size // 2] = np.inf
    flat[flat.size - 1] = np.nan
    x = R.to_bits(xf, dtype)
    mean_ref, var_ref = R.moments(dtype, x, list(axes))
    an = acc_name(dtype)
    mean, var = empty(mean_ref.shape, an), empty(var_ref.shape, an)
    K.moments(list(shape), list(axes), U.to_device(x, dtype), mean, var)
    m, v = U.to_host(mean), U.to_host(var)
    assert np.array_equal(np.isnan(m), np.isnan(mean_ref))
    assert np.array_equal(np.isinf(m), np.isinf(mean_ref))
    assert np.array_equal(m[np.isinf(m)], mean_ref[np.isinf(mean_ref)])
    assert np.array_equal(np.isnan(v), np.isnan(var_ref))
    ok = np.isfinite(mean_ref)
    with np.errstate(invalid="ignore"):
        m64 = np.asarray(U.widen(x, dtype), np.float64).reshape(shape).mean(tuple(axes))
    good, *errs = U.close3(m[ok], mean_ref[ok], m64.reshape(mean_ref.shape)[ok], 1e-5)
    assert good, errs


def test_math_helpers_bitwise(K):
    rng = U.rng_for(9)
    n = 1000
    x = rng.uniform(0.1, 4, n).astype(np.float32)
    y0 = rng.standard_normal(n).astype(np.float32)
    xd, yd = U.to_device(x, "float32"), U.to_device(y0, "float32")
    out = empty((n,), "float32")
    K.inv_std(n, 1e-5, xd, out)
    assert np.max(np.abs(U.to_host(out) / R.inv_std(x, 1e-5) - 1)) <= 1.2e-7
    K.axpby(n, 0.1, xd, 0.9, yd)
    y_ref = y0.copy()
    R.axpby(0.1, x, 0.9, y_ref)
    assert np.array_equal(U.to_host(yd), y_ref)  # two roundings, no fused multiply-add
    K.copy(n, xd, out)
    assert np.array_equal(U.to_host(out), x)
    K.square(n, xd, out)
    assert np.array_equal(U.to_host(out), x * x)
    K.sub(n, xd, yd, out)
    assert np.array_equal(U.to_host(out), x - U.to_host(yd))
    K.set(n, 2.5, out)
    assert np.all(U.to_host(out) == 2.5)


# ---------------------------------------------------------------- L1Norm / L2Norm

LP_SHAPES = [((256, 512), -1), ((10, 1000), -1), ((4, 4096), -1), ((3, 70000), -1), ((5, 37), -1),
             ((6, 300), -1), ((3, 7, 5), 1), ((2, 3, 4, 16), 2), ((4, 1), -1), ((2, 16, 8, 8), 1),
             ((3, 8200), -1), ((2, 40, 24), 1),
             # short and odd rows staged through LDS
             ((5000, 64), -1), ((700, 197), -1), ((130, 577), -1)]


def _lp_fp64(x, dy, ax, p, normalizer, eps):
    x64, dy64 = np.asarray(x, np.float64), np.asarray(dy, np.float64)
    if p == 1:
        norm = np.maximum(np.abs(x64).sum(ax, keepdims=True) / normalizer, eps)
        g = np.sign(x64)
    else:
        norm = np.maximum(np.sqrt(np.square(x64).sum(ax, keepdims=True) / normalizer), eps)
        g = x64
    dot = (dy64 * x64).sum(ax, keepdims=True) / normalizer
    # third value: size of the two terms that cancel in dx
    return x64 / norm, dy64 / norm - g * dot / norm ** (p + 1), float(np.max(np.abs(dy64 / norm)))


@pytest.mark.parametrize("reduction", ["sum", "mean"])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape,axis", LP_SHAPES)
def test_lp_norm_forward_backward(K, shape, axis, dtype, p, reduction):
    rng = U.rng_for(900 + len(shape) + p)
    x = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    ax = axis % len(shape)
    N = int(np.prod(shape[:ax] or (1,)))
    C = shape[ax]
    S = int(np.prod(shape[ax + 1:] or (1,)))
    normalizer = float(C) if reduction == "mean" else 1.0
    eps = 1e-12
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    y_ref = R.op_lp_norm(od, xo, axis, None, p, eps, reduction)
    dx_ref = R.op_lp_norm_grad(od, xo, dyo, axis, None, p, eps, reduction)
    y64, dx64, term = _lp_fp64(xo, dyo, ax, p, normalizer, eps)
    xd, dyd = U.to_device(x, dtype), U.to_device(dy, dtype)
    y, dx = empty(shape, dtype), empty(shape, dtype)
    fwd = K.l1_norm if p == 1 else K.l2_norm
    bwd = K.l1_norm_grad if p == 1 else K.l2_norm_grad
    fwd(N, S, C, normalizer, eps, xd, y)
    bwd(N, S, C, normalizer, eps, dyd, xd, dx)
    yw = U.widen(U.to_host(y), dtype).reshape(shape)
    dxw = U.widen(U.to_host(dx), dtype).reshape(shape)
    # rows of 70000 put the oracle's sequential fp32 sums themselves off: three-way check
    ok, *errs = U.close3(yw, y_ref, y64, U.TIGHT[dtype])
    assert ok, errs
    # dx is a difference of two terms of size `term` (it vanishes for C == 1):
    # errors are measured against that size
    e_go = np.max(np.abs(dxw - np.asarray(dx_ref, np.float64))) / term
    e_ge = np.max(np.abs(dxw - dx64)) / term
    e_oe = np.max(np.abs(np.asarray(dx_ref, np.float64) - dx64)) / term
    assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)


@pytest.mark.parametrize("p", [1, 2])
def test_lp_norm_reference_literals_on_device(K, p):
    # test/dragon/test_ops.py:4480-4512
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_test_vectors.json")) as f:
        g = json.load(f)["lp_norm"]
    data1 = np.arange(6, dtype=np.float32)
    data2 = (np.arange(6, dtype=np.float32) / 10 + 1).astype(np.float32)
    for e in g["entries"]:
        if e["p"] != p:
            continue
        normalizer = 6.0 if e["reduction"] == "mean" else 1.0
        xd, dyd = U.to_device(data1, "float32"), U.to_device(data2, "float32")
        y, dx = empty((6,), "float32"), empty((6,), "float32")
        (K.l1_norm if p == 1 else K.l2_norm)(1, 1, 6, normalizer, e["eps"], xd, y)
        (K.l1_norm_grad if p == 1 else K.l2_norm_grad)(1, 1, 6, normalizer, e["eps"], dyd, xd, dx)
        norm = np.abs(data1) if p == 1 else np.square(data1)
        norm = norm.sum() if e["reduction"] == "sum" else norm.mean()
        norm = norm if p == 1 else np.sqrt(norm)
        assert np.max(np.abs(U.to_host(y) - data1 / max(norm, e["eps"]))) <= g["prec"]
        assert np.max(np.abs(U.to_host(dx) - np.array(e["dx"], np.float32))) <= g["prec"]


def test_lp_norm_in_place_epsilon_clamp_and_empty(K):
    x = np.zeros((4, 512), np.float32)
    x[1] = np.linspace(-1, 1, 512)
    x[2, 7] = 3.0
    dy = np.ones((4, 512), np.float32)
    y_ref = R.op_lp_norm("float32", x, -1, None, 2, 0.5, "sum")
    dx_ref = R.op_lp_norm_grad("float32", x, dy, -1, None, 2, 0.5, "sum")
    buf, g = U.to_device(x, "float32"), U.to_device(dy, "float32")
    K.l2_norm_grad(4, 1, 512, 1.0, 0.5, g, buf, g)   # dX aliases dY
    K.l2_norm(4, 1, 512, 1.0, 0.5, buf, buf)         # Y aliases X
    assert U.normwise(U.to_host(buf), y_ref) <= 1e-6
    assert U.normwise(U.to_host(g), dx_ref) <= 1e-6
    assert np.all(U.to_host(buf)[0] == 0)            # 0 / max(0, eps)
    e = empty((0, 8), "float32")
    K.l1_norm(0, 1, 8, 1.0, 1e-12, e, e)             # no rows: nothing to do, no error


# ---------------------------------------------------------------- ReduceSum / ReduceSumSqr / ReduceL1

@pytest.mark.parametrize("kind", ["sum", "sum_sqr", "l1"])
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape,axes", MOMENT_CASES)
def test_reduce_sums(K, shape, axes, dtype, kind):
    rng = U.rng_for(1100 + len(shape))
    x = R.to_bits((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32), dtype)
    xo, od = oracle_dtype_inputs(x, dtype)   # the reference's CPU has these for fp32/fp64 only
    scale = 0.5
    y_ref = R.reduce_sum(od, xo, list(axes), scale, kind)
    f = {"sum": lambda v: v, "sum_sqr": np.square, "l1": np.abs}[kind]
    y64 = (f(np.asarray(xo, np.float64)).sum(tuple(axes)) * scale).ravel()
    y = empty(y_ref.shape, dtype)
    fn = {"sum": K.reduce_sum, "sum_sqr": K.reduce_sum_sqr, "l1": K.reduce_l1}[kind]
    fn(list(shape), list(axes), scale, U.to_device(x, dtype), y)
    yw = U.widen(U.to_host(y), dtype)
    # plain sums cancel: errors are measured against the sum of magnitudes
    mag = (np.abs(f(np.asarray(xo, np.float64))).sum(tuple(axes)) * scale).ravel()
    mag = float(np.max(mag)) if mag.size else 1.0
    e_go = np.max(np.abs(yw - np.asarray(y_ref, np.float64))) / mag if yw.size else 0.0
    e_ge = np.max(np.abs(yw - y64)) / mag if yw.size else 0.0
    e_oe = np.max(np.abs(np.asarray(y_ref, np.float64) - y64)) / mag if yw.size else 0.0
    assert e_ge <= U.TIGHT[dtype] and e_go <= U.TIGHT[dtype] + e_oe, (e_go, e_ge, e_oe)


def test_sum_of_a_large_vector_and_empty_reduction(K):
    rng = U.rng_for(12)
    n = 3_000_001
    x = rng.standard_normal(n).astype(np.float32)
    y = empty((1,), "float32")
    K.sum(n, 1.0, U.to_device(x, "float32"), y)
    want = float(x.astype(np.float64).sum())
    assert abs(float(U.to_host(y)[0]) - want) <= 1e-5 * float(np.abs(x).sum())
    # a reduced extent of zero yields the sum's identity
    out = U.to_device(np.full(3, 7.0, np.float32), "float32")
    K.reduce_sum([3, 0], [1], 1.0, empty((3, 0), "float32"), out)
    assert np.all(U.to_host(out) == 0)


# ---------------------------------------------------------------- softmax cross-entropy loss

SCE_SHAPES = [((64, 512), -1), ((10, 1000), -1), ((5, 37), -1), ((6, 4096), -1), ((3, 7, 5), 1),
              ((2, 19, 8, 8), 1), ((4, 1), -1), ((3, 40000), -1), ((2, 6, 16), 1),
              # 1024-thread rows (prefetching forward); packets that straddle rows in the backward
              ((4, 20000), -1), ((3, 6000), -1), ((8, 1001), -1),
              # more than 16384 positions: the two-stage loss reductions
              ((70000, 8), -1), ((2, 5, 40000), 1)]


def _sce_case(shape, axis, dtype, tdtype, seed):
    rng = U.rng_for(seed)
    ax = axis % len(shape)
    x = (rng.standard_normal(shape) * 2).astype(dtype)
    C = shape[ax]
    tshape = tuple(d for i, d in enumerate(shape) if i != ax)
    target = rng.integers(0, C, tshape).astype(tdtype)
    target.ravel()[::4] = 255
    N = int(np.prod(shape[:ax] or (1,)))
    S = int(np.prod(shape[ax + 1:] or (1,)))
    return x, target, tshape, N, C, S


@pytest.mark.parametrize("dtype,tdtype", [("float32", "int64"), ("float32", "int32"),
                                          ("float64", "int64")])
@pytest.mark.parametrize("shape,axis", SCE_SHAPES)
def test_loss_kernels_one_by_one(K, shape, axis, dtype, tdtype):
    import torch
    x, target, tshape, N, C, S = _sce_case(shape, axis, dtype, tdtype, 1300 + len(shape))
    tol = U.TIGHT[dtype]
    prob = R.softmax(dtype, N, S, C, x)
    pd, td = U.to_device(prob, dtype), torch.from_numpy(target).cuda()
    # CrossEntropy with class indices
    loss_ref, mask_ref = R.sparse_cross_entropy(dtype, N, S, C, 255, prob, target)
    loss, mask = empty((N * S,), dtype), empty((N * S,), dtype)
    K.sparse_cross_entropy(N, S, C, 255, pd, td, loss, mask)
    assert np.array_equal(U.to_host(mask), mask_ref)
    assert U.normwise(U.to_host(loss), loss_ref) <= tol
    # CrossEntropy with dense targets
    dense = U.rng_for(5).random(prob.shape).astype(dtype)
    dl_ref = R.cross_entropy(dtype, prob, dense)
    dloss = empty(prob.shape, dtype)
    K.cross_entropy(prob.size, pd, U.to_device(dense, dtype), dloss)
    assert U.normwise(U.to_host(dloss), dl_ref) <= tol
    # SoftmaxCrossEntropyGrad patches a copy of the probabilities in place
    dx_ref = prob.copy()
    gmask_ref = R.softmax_cross_entropy_grad(dtype, N, S, C, 255, target, dx_ref)
    dx, gmask = pd.clone(), empty((N * S,), dtype)
    K.softmax_cross_entropy_grad(N, S, C, 255, pd, td, dx, gmask)
    assert np.array_equal(U.to_host(gmask), gmask_ref)
    assert np.array_equal(U.to_host(dx), dx_ref)       # subtracting 1 and clearing are exact
    # ReduceLoss / ReduceLossGrad with every normalisation, BroadcastLossGrad
    for normalizer, use_mask in ((-1.0, True), (float(N * S), True), (1.0, False), (3.0, False)):
        m_ref = mask_ref if use_mask else None
        y_ref = R.reduce_loss(dtype, normalizer, loss_ref, m_ref)
        y = empty((1,), dtype)
        K.reduce_loss(N * S, N * S if use_mask else 0, normalizer, loss, mask if use_mask else None, y)
        assert abs(float(U.to_host(y)[0]) - float(y_ref)) <= tol * max(1.0, abs(float(y_ref)))
        dlv = np.array([1.7], dtype)
        g_ref = R.reduce_loss_grad(dtype, normalizer, dlv, dx_ref.copy(), m_ref)
        g = dx.clone()
        K.reduce_loss_grad(g.numel(), N * S if use_mask else 0, normalizer,
                           U.to_device(dlv, dtype), gmask if use_mask else None, g)
        assert U.normwise(U.to_host(g), g_ref) <= tol
    dlp = U.rng_for(6).standard_normal(N * S).astype(dtype)
    b_ref = R.broadcast_loss_grad(dtype, N, S, C, dlp, dx_ref.copy())
    b = dx.clone()
    K.broadcast_loss_grad(N, S, C, U.to_device(dlp, dtype), b)
    assert U.normwise(U.to_host(b), b_ref) <= tol


@pytest.mark.parametrize("reduction", ["none", "sum", "mean", "batch_mean", "valid"])
@pytest.mark.parametrize("dtype,tdtype", [("float32", "int64"), ("float32", "int32"),
                                          ("float64", "int64")])
@pytest.mark.parametrize("shape,axis", SCE_SHAPES)
def test_fused_softmax_cross_entropy_loss(K, shape, axis, dtype, tdtype, reduction):
    import torch
    x, target, tshape, N, C, S = _sce_case(shape, axis, dtype, tdtype, 1400 + len(shape))
    tol = U.TIGHT[dtype]
    loss_ref, prob_ref = R.op_softmax_cross_entropy_loss(dtype, x, target, axis, 255, reduction)
    xd, td = U.to_device(x, dtype), torch.from_numpy(target).cuda()
    prob = empty(shape, dtype)
    loss = empty(tshape if reduction == "none" else (1,), dtype)
    # BATCH_MEAN divides by the leading extent of x, which is N only for a 2-d view
    if reduction == "batch_mean" and shape[0] != N:
        pytest.skip("the fused entry point takes N as the batch extent")
    K.softmax_cross_entropy_loss_forward(N, S, C, 255, reduction, xd, td, prob, loss)
    # the oracle's sequential fp32 sums over 40000 classes are themselves ~1e-5 off
    x64 = np.moveaxis(np.asarray(x, np.float64), axis % len(shape), -1)
    e = np.exp(x64 - x64.max(-1, keepdims=True))
    p64 = np.moveaxis(e / e.sum(-1, keepdims=True), -1, axis % len(shape))
    ok, *errs = U.close3(U.to_host(prob), prob_ref, p64, tol)
    assert ok, errs
    got = U.to_host(loss).reshape(np.shape(loss_ref))
    assert np.max(np.abs(got - loss_ref)) <= 4 * tol * max(1.0, float(np.max(np.abs(loss_ref))))
    # backward from the probabilities the forward produced
    ph = U.to_host(prob)
    dl = (U.rng_for(7).standard_normal(tshape).astype(dtype) if reduction == "none"
          else np.array(1.7, dtype))
    dx_ref = R.op_softmax_cross_entropy_loss_grad(dtype, ph, target, dl, axis, 255, reduction)
    dx = empty(shape, dtype)
    K.softmax_cross_entropy_loss_backward(N, S, C, 255, reduction, prob, td,
                                          U.to_device(np.atleast_1d(dl), dtype), dx)
    assert U.normwise(U.to_host(dx), dx_ref) <= tol
    ignored = np.expand_dims(target == 255, axis % len(shape))
    assert np.all(U.to_host(dx)[np.broadcast_to(ignored, shape)] == 0)


def test_fused_softmax_cross_entropy_loss_out_of_range_target_is_ignored(K):
    import torch
    x = np.zeros((4, 8), np.float32)
    target = np.array([1, 8, -3, 2], np.int64)     # 8 and -3 are outside [0, 8)
    xd, td = U.to_device(x, "float32"), torch.from_numpy(target).cuda()
    prob, loss = empty((4, 8), "float32"), empty((4,), "float32")
    K.softmax_cross_entropy_loss_forward(4, 1, 8, 2 ** 31 - 1, "none", xd, td, prob, loss)
    got = U.to_host(loss)
    assert got[1] == 0 and got[2] == 0
    assert np.allclose(got[[0, 3]], np.log(8.0), rtol=1e-6)


# ---------------------------------------------------------------- unaligned bases, ragged widths

@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16", "float64"])
@pytest.mark.parametrize("shape", [(7, 197), (5, 1001), (3, 4099), (2, 66001)])
def test_rows_at_element_aligned_addresses(K, dtype, shape):
    """Tensors that start one element past a 16-byte boundary, with widths that
    are not whole packets: the ragged tiles and the looped kernels."""
    import torch
    N, C = shape
    rng = U.rng_for(1500 + C)
    x = R.to_bits(rng.standard_normal(shape).astype(np.float32) * 2, dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)
    x64 = np.asarray(xo, np.float64)

    def shifted(bits):
        buf = empty((N * C + 1,), dtype)
        view = buf[1:].view(N, C)
        view.copy_(U.to_device(bits, dtype))
        assert view.data_ptr() % 16 != 0
        return view

    def out():
        return empty((N * C + 1,), dtype)[1:].view(N, C)

    xd, dyd = shifted(x), shifted(dy)
    tol = U.TIGHT[dtype]
    # softmax forward / backward
    y = out()
    K.softmax(N, 1, C, xd, y)
    e = np.exp(x64 - x64.max(1, keepdims=True))
    y64 = e / e.sum(1, keepdims=True)
    yw = U.widen(U.to_host(y.contiguous()), dtype).reshape(shape)
    assert U.rowwise_normwise(yw, y64) <= tol
    dx = out()
    K.softmax_grad(N, 1, C, dyd, y, dx)
    yo, _ = oracle_dtype_inputs(U.to_host(y.contiguous()).reshape(shape), dtype)
    dx_ref = R.op_softmax_grad(od, yo, dyo)
    assert U.normwise(U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape), dx_ref) <= tol
    # log-softmax forward
    K.log_softmax(N, 1, C, xd, y)
    ly64 = (x64 - x64.max(1, keepdims=True)) - np.log(e.sum(1, keepdims=True))
    lyw = U.widen(U.to_host(y.contiguous()), dtype).reshape(shape)
    assert np.max(np.abs(lyw - ly64) / np.maximum(np.abs(ly64), 1.0)) <= tol
    # layer norm forward (gamma / beta element-aligned too)
    an = acc_name(dtype)
    g, b = U.affine_params(rng, C, dtype)
    gbuf, bbuf = empty((C + 1,), an), empty((C + 1,), an)
    gbuf[1:].copy_(U.to_device(g, an))
    bbuf[1:].copy_(U.to_device(b, an))
    mu, rsig = empty((N,), an), empty((N,), an)
    K.layer_norm(N, C, 1e-5, xd, gbuf[1:], bbuf[1:], mu, rsig, y)
    mean64 = x64.mean(1, keepdims=True)
    ln64 = (x64 - mean64) / np.sqrt(x64.var(1, keepdims=True) + 1e-5) * g + b
    assert U.normwise(U.widen(U.to_host(y.contiguous()), dtype).reshape(shape), ln64) <= tol
    assert U.normwise(U.to_host(mu), mean64.ravel()) <= (1e-12 if dtype == "float64" else 1e-5)
    # l2 normalisation forward / backward
    K.l2_norm(N, 1, C, 1.0, 1e-12, xd, y)
    y64n, dx64n, term = _lp_fp64(xo, dyo, 1, 2, 1.0, 1e-12)
    assert U.normwise(U.widen(U.to_host(y.contiguous()), dtype).reshape(shape), y64n) <= tol
    K.l2_norm_grad(N, 1, C, 1.0, 1e-12, dyd, xd, dx)
    dxw = U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape)
    assert np.max(np.abs(dxw - dx64n)) / term <= tol


# ---------------------------------------------------------------- more than 2^31 elements

def _rows_to_bits(t, rows, dtype):
    """Rows `rows` of device tensor t as the oracle's storage (bits for 16-bit types)."""
    import torch
    sel = t[torch.as_tensor(rows, device=t.device)].contiguous()
    return U.to_host(sel)


def test_softmax_rows_beyond_int32_elements(K):
    """[2^20 + 7, 2304] fp16: element offsets pass 2^31. Sampled rows against the oracle,
    every row through the size-independent properties (sums to one; dx sums to zero)."""
    import torch
    dtype = "float16"
    N, C = (1 << 20) + 7, 2304
    assert N * C > 2 ** 31
    gen = torch.Generator(device="cuda").manual_seed(31)
    x = torch.empty((N, C), dtype=torch.float16, device="cuda").normal_(0.0, 2.0, generator=gen)
    y = torch.empty_like(x)
    K.softmax(N, 1, C, x, y)
    sums = y.sum(1, dtype=torch.float32)
    assert float((sums - 1).abs().max()) < 2e-2
    rows = [0, 1, N // 2, (2 ** 31) // C, (2 ** 31) // C + 1, N - 2, N - 1]
    xs = _rows_to_bits(x, rows, dtype)
    xo, od = oracle_dtype_inputs(xs, dtype)
    y_ref = R.op_softmax(od, xo, 1)
    got = U.widen(_rows_to_bits(y, rows, dtype), dtype)
    assert U.normwise(got, y_ref) <= U.TIGHT[dtype]
    dy = torch.empty_like(x).normal_(0.0, 1.0, generator=gen)
    dx = torch.empty_like(x)
    K.softmax_grad(N, 1, C, dy, y, dx)
    # sum_j dx_j = sum_j y_j (dy_j - s) = s - s sum_j y_j ~ 0 (fp16 outputs: 2304 roundings)
    assert float(dx.sum(1, dtype=torch.float32).abs().max()) < 5e-2
    yo, _ = oracle_dtype_inputs(_rows_to_bits(y, rows, dtype), dtype)
    dyo, _ = oracle_dtype_inputs(_rows_to_bits(dy, rows, dtype), dtype)
    dx_ref = R.op_softmax_grad(od, yo, dyo, 1)
    assert U.normwise(U.widen(_rows_to_bits(dx, rows, dtype), dtype), dx_ref) <= U.TIGHT[dtype]


def test_layer_norm_rows_beyond_int32_elements(K):
    """[2^20 + 7, 2304] bf16 LayerNorm forward: sampled rows against the oracle, every row
    through mean(y) ~ 0 and mean(y^2) ~ 1 (gamma = 1, beta = 0)."""
    import torch
    dtype = "bfloat16"
    N, C = (1 << 20) + 7, 2304
    gen = torch.Generator(device="cuda").manual_seed(32)
    x = torch.empty((N, C), dtype=torch.bfloat16, device="cuda").normal_(0.5, 2.0, generator=gen)
    y = torch.empty_like(x)
    g = torch.ones(C, device="cuda")
    b = torch.zeros(C, device="cuda")
    mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    K.layer_norm(N, C, 1e-5, x, g, b, mu, rsig, y)
    yf = y.float()
    assert float(yf.mean(1).abs().max()) < 1e-2
    assert float(((yf * yf).mean(1) - 1).abs().max()) < 2e-2
    del yf
    rows = [0, N // 2, (2 ** 31) // C, (2 ** 31) // C + 1, N - 1]
    xs = _rows_to_bits(x, rows, dtype)
    y_ref, mu_ref, rsig_ref = R.layer_norm(dtype, xs, np.ones(C, np.float32), np.zeros(C, np.float32), 1e-5)
    got = U.widen(_rows_to_bits(y, rows, dtype), dtype)
    assert U.normwise(got, U.widen(y_ref, dtype)) <= U.TIGHT[dtype]
    idx = torch.as_tensor(rows, device="cuda")
    assert np.max(np.abs(U.to_host(mu[idx]) - mu_ref)) <= 1e-4
    assert np.max(np.abs(U.to_host(rsig[idx]) / rsig_ref - 1)) <= 1e-4


def test_layer_norm_backward_beyond_int32_elements(K):
    """[2^20 + 7, 2304] bf16 LayerNorm backward: sampled rows of dx, ds, db against the oracle;
    dgamma / dbeta against fp64 sums of the same products on the device."""
    import torch
    dtype = "bfloat16"
    N, C = (1 << 20) + 7, 2304
    gen = torch.Generator(device="cuda").manual_seed(33)
    x = torch.empty((N, C), dtype=torch.bfloat16, device="cuda").normal_(0.5, 2.0, generator=gen)
    dy = torch.empty_like(x).normal_(0.0, 1.0, generator=gen)
    g = torch.empty(C, device="cuda").uniform_(0.5, 1.5, generator=gen)
    b = torch.zeros(C, device="cuda")
    mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    y = torch.empty_like(x)
    K.layer_norm(N, C, 1e-5, x, g, b, mu, rsig, y)
    del y
    params = torch.empty(2 * N, device="cuda")
    dg, db, dx = torch.empty(C, device="cuda"), torch.empty(C, device="cuda"), torch.empty_like(x)
    K.group_norm_grad(N, 1, C, 1, "NHWC", x, mu, rsig, g, dy, params, params, dg, db, dx)
    rows = [0, N // 2, (2 ** 31) // C, (2 ** 31) // C + 1, N - 1]
    idx = torch.as_tensor(rows, device="cuda")
    xs = R.from_bits(_rows_to_bits(x, rows, dtype), dtype)
    dys = R.from_bits(_rows_to_bits(dy, rows, dtype), dtype)
    dx_ref, _, _, ds_ref, db_ref = R.group_norm_grad(
        "float32", len(rows), 1, C, 1, "NHWC", xs, U.to_host(mu[idx]), U.to_host(rsig[idx]),
        U.to_host(g), dys)
    assert U.normwise(U.widen(_rows_to_bits(dx, rows, dtype), dtype), dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(U.to_host(params[:N][idx]), ds_ref) <= 2e-5
    assert U.normwise(U.to_host(params[N:][idx]), db_ref) <= 2e-5
    # column sums over a million rows, in chunks to bound the fp64 temporaries
    dg64 = torch.zeros(C, dtype=torch.float64, device="cuda")
    db64 = torch.zeros(C, dtype=torch.float64, device="cuda")
    step = 1 << 17
    for r0 in range(0, N, step):
        xc = x[r0:r0 + step].double()
        dc = dy[r0:r0 + step].double()
        m = mu[r0:r0 + step].double()[:, None]
        r = rsig[r0:r0 + step].double()[:, None]
        dg64 += (dc * (xc - m) * r).sum(0)
        db64 += dc.sum(0)
    assert U.normwise(U.to_host(dg), dg64.cpu().numpy()) <= 2e-5
    assert U.normwise(U.to_host(db), db64.cpu().numpy()) <= 2e-5


def test_l2_norm_and_cross_entropy_beyond_int32_elements(K):
    """The same for the sibling row kernels: L2 norm of a bf16 and fused softmax
    cross-entropy of an fp32 [2^20 + 7, 2304] matrix; sampled rows against the oracle,
    every row through |y| = 1 and loss = -log prob[target]."""
    import torch
    N, C = (1 << 20) + 7, 2304
    rows = [0, N // 2, (2 ** 31) // C, (2 ** 31) // C + 1, N - 1]
    idx = torch.as_tensor(rows, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(34)
    x = torch.empty((N, C), dtype=torch.bfloat16, device="cuda").normal_(0.0, 2.0, generator=gen)
    y = torch.empty_like(x)
    K.l2_norm(N, 1, C, 1.0, 1e-12, x, y)
    norms = (y.float() ** 2).sum(1)
    assert float((norms - 1).abs().max()) < 2e-2
    y_ref = R.lp_norm("float32", 2, len(rows), 1, C, 1.0, 1e-12,
                      R.from_bits(_rows_to_bits(x, rows, "bfloat16"), "bfloat16"))
    assert U.normwise(U.widen(_rows_to_bits(y, rows, "bfloat16"), "bfloat16"), y_ref) <= U.TIGHT["bfloat16"]
    del x, y, norms

    logits = torch.empty((N, C), dtype=torch.float32, device="cuda").normal_(0.0, 2.0, generator=gen)
    target = torch.randint(0, C, (N,), generator=gen, device="cuda", dtype=torch.int64)
    prob = torch.empty_like(logits)
    loss = torch.empty(N, device="cuda")
    K.softmax_cross_entropy_loss_forward(N, 1, C, -1, "none", logits, target, prob, loss)
    picked = prob.gather(1, target[:, None])[:, 0]
    assert float((loss + picked.log()).abs().max()) < 1e-5
    assert float((prob.sum(1) - 1).abs().max()) < 1e-4
    loss_ref, prob_ref = R.op_softmax_cross_entropy_loss(
        "float32", U.to_host(logits[idx]), U.to_host(target[idx]), reduction="none")
    assert U.normwise(U.to_host(prob[idx]), prob_ref) <= U.TIGHT["float32"]
    assert U.normwise(U.to_host(loss[idx]), loss_ref) <= U.TIGHT["float32"]


# ---------------------------------------------------------------- channel ops at shifted bases

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", [(4, 12, 9, 9), (2, 6, 40, 41)])
@pytest.mark.parametrize("shift", [1, 3])
def test_channel_ops_at_shifted_bases(K, dtype, shape, shift):
    """NCHW tensors that start `shift` elements past a 16-byte boundary (views into a larger
    buffer): BatchNorm and GroupNorm forward and backward take the staged short-row kernels
    ((n, c) rows of 81 elements) or one wavefront per row (1640 elements), whose first and
    last packets reach outside the tensors. Nothing outside the outputs may be written."""
    rng = U.rng_for(900 + shift)
    N, C = shape[0], shape[1]
    S = shape[2] * shape[3]
    total = N * C * S
    an = acc_name(dtype)
    guard = 8
    x = R.to_bits((2 * rng.standard_normal(shape) + 0.5).astype(np.float32), dtype)
    dy = R.to_bits(rng.standard_normal(shape).astype(np.float32), dtype)
    g, b = U.affine_params(rng, C, dtype)
    xo, od = oracle_dtype_inputs(x, dtype)
    dyo, _ = oracle_dtype_inputs(dy, dtype)

    def shifted(bits=None):
        buf = empty((total + shift + guard,), dtype)
        buf.zero_()
        view = buf[shift:shift + total].view(shape)
        if bits is not None:
            view.copy_(U.to_device(bits, dtype).view(shape))
        return buf, view

    def untouched(buf):
        flat = U.widen(U.to_host(buf), dtype).ravel()
        return np.all(flat[:shift] == 0) and np.all(flat[shift + total:] == 0)

    _, xd = shifted(x)
    _, dyd = shifted(dy)
    gd, bd = U.to_device(g, an), U.to_device(b, an)

    # BatchNorm
    rm_ref = np.zeros(C, U.acc_np(dtype))
    rv_ref = np.ones(C, U.acc_np(dtype))
    y_ref, mu_ref, rsig_ref, _ = R.op_batch_norm_train(
        od, np.asarray(xo).reshape(shape), g, b, rm_ref, rv_ref, 1, 0.9, 1e-5)
    dx_ref, dg_ref, db_ref = R.op_batch_norm_train_grad(
        od, np.asarray(xo).reshape(shape), g, np.asarray(dyo).reshape(shape), mu_ref, rsig_ref, 1)
    mu, rsig, params = empty((C,), an), empty((C,), an), empty((2 * C,), an)
    rm, rv = U.to_device(np.zeros(C, U.acc_np(dtype)), an), U.to_device(np.ones(C, U.acc_np(dtype)), an)
    ybuf, y = shifted()
    K.batch_norm_training_forward(N, C, S, "NCHW", 0.9, 1e-5, xd, gd, bd, rm, rv, mu, rsig, params, y)
    assert U.normwise(U.to_host(mu), mu_ref) <= 1e-5
    assert U.normwise(U.widen(U.to_host(y.contiguous()), dtype).reshape(shape), y_ref) <= U.TIGHT[dtype]
    assert untouched(ybuf)
    dxbuf, dx = shifted()
    dg, db = empty((C,), an), empty((C,), an)
    K.batch_norm_training_backward(N, C, S, float(N * S), "NCHW", xd, U.to_device(mu_ref, an),
                                   U.to_device(rsig_ref, an), gd, dyd, dg, db, dx)
    assert U.normwise(U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape), dx_ref) <= U.TIGHT[dtype]
    assert U.normwise(U.to_host(dg), dg_ref) <= 2e-5 and U.normwise(U.to_host(db), db_ref) <= 2e-5
    assert untouched(dxbuf)

    # GroupNorm, 3 groups
    G = 3
    D = C // G
    y_ref, mu_ref, rsig_ref = R.op_group_norm(dtype, x, g, b, 1, G, 1e-5)
    mu, rsig = empty((N * G,), an), empty((N * G,), an)
    ybuf, y = shifted()
    K.group_norm_forward(N, G, D, S, "NCHW", 1e-5, xd, gd, bd, mu, rsig, y)
    assert U.normwise(U.to_host(mu), mu_ref) <= 1e-5
    assert U.normwise(U.widen(U.to_host(y.contiguous()), dtype).reshape(shape),
                      U.widen(y_ref, dtype).reshape(shape)) <= U.TIGHT[dtype]
    assert untouched(ybuf)
    dx_ref, dg_ref, db_ref, _, _ = R.group_norm_grad(od, N, G, D, S, "NCHW", xo, mu_ref, rsig_ref, g, dyo)
    dxbuf, dx = shifted()
    pr = empty((2 * N * G,), an)
    K.group_norm_grad(N, G, D, S, "NCHW", xd, U.to_device(mu_ref, an), U.to_device(rsig_ref, an), gd,
                      dyd, pr, pr, dg, db, dx)
    assert U.normwise(U.widen(U.to_host(dx.contiguous()), dtype).reshape(shape),
                      np.asarray(dx_ref).reshape(shape)) <= U.TIGHT[dtype]
    assert U.normwise(U.to_host(dg), dg_ref) <= 2e-5 and U.normwise(U.to_host(db), db_ref) <= 2e-5
    assert untouched(dxbuf)
