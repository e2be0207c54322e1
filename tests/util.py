"""Shared helpers of the GPU parity tests: seeded inputs, host<->device moves
for 16-bit storage, and the error metrics the tolerances are stated in."""

import numpy as np

from oracle import ref_cpu as R

TORCH_DTYPES = None


def torch_dtype(name):
    import torch
    return {"float16": torch.float16, "bfloat16": torch.bfloat16,
            "float32": torch.float32, "float64": torch.float64}[name]


def to_device(bits, dtype):
    """numpy storage (uint16 bit patterns for 16-bit types) -> CUDA tensor of ``dtype``."""
    import torch
    a = np.ascontiguousarray(bits)
    if dtype in ("float16", "bfloat16"):
        t = torch.from_numpy(a.view(np.int16)).cuda()
        return t.view(torch_dtype(dtype))
    return torch.from_numpy(a).cuda()


def to_host(t):
    """CUDA tensor -> numpy storage (uint16 bit patterns for 16-bit types)."""
    import torch
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def widen(bits, dtype):
    """Storage -> float64 values."""
    return np.asarray(R.from_bits(bits, dtype), dtype=np.float64)


def acc_np(dtype):
    return np.float64 if dtype == "float64" else np.float32


def normwise(got, want):
    """max|got - want| / max|want| over the whole tensor (0 when both are 0)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = np.max(np.abs(want)) if want.size else 0.0
    if got.size == 0:
        return 0.0
    err = np.max(np.abs(got - want))
    return float(err / scale) if scale > 0 else float(err)


def rowwise_normwise(got, want, axis=-1):
    """Worst per-row max|d| / max|want| (used for softmax, whose rows have their own scale)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.max(np.abs(got - want), axis=axis)
    scale = np.maximum(np.max(np.abs(want), axis=axis), 1e-30)
    return float(np.max(err / scale)) if err.size else 0.0


# Tolerances of the parity bar: 1e-5 relative for fp32 I/O, 1e-2 for fp16/bf16
# I/O against the fp32 CPU reference; fp64 is held to 1e-12.
TOL = {"float32": 1e-5, "float64": 1e-12, "float16": 1e-2, "bfloat16": 1e-2}
# What a correct kernel should actually reach for 16-bit outputs: one rounding
# ulp of the 16-bit result (2^-10 for fp16, 2^-7 for bf16: a value that sits on a
# rounding boundary may round the other way than in the oracle).
TIGHT = {"float32": 1e-5, "float64": 1e-12, "float16": 1.5e-3, "bfloat16": 8e-3}


def rng_for(seed):
    return np.random.default_rng(seed)


def affine_params(rng, C, dtype):
    """gamma ~ U(0.5, 1.5), beta ~ N(0, 0.1) in the accumulator type."""
    a = acc_np(dtype)
    return (rng.uniform(0.5, 1.5, C).astype(a), (rng.standard_normal(C) * 0.1).astype(a))


def close3(got, oracle, exact, tol):
    """Three-way check for long reductions, where the oracle's strictly
    sequential fp32 sums are themselves off: the distance to the oracle may
    exceed ``tol`` only by the oracle's own distance to the fp64 result.
    Returns (ok, gpu_vs_oracle, gpu_vs_exact, oracle_vs_exact), all normwise."""
    e_go = normwise(got, oracle)
    e_ge = normwise(got, exact)
    e_oe = normwise(oracle, exact)
    return e_go <= tol + e_oe and e_ge <= tol, e_go, e_ge, e_oe
