#!/usr/bin/env python3
"""Benchmark of the norm / softmax hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-sweep] [--no-cpu]

A step is one pass of the workload's kernels (forward then backward) over one
batch of synthetic input that is already resident in HBM. The headline
workload is Softmax forward+backward, fp16 I/O, [16, 32, 512, 512] along the
last axis; `value` is its algorithmic bytes per step divided by the time per
step. One JSON line is printed.

Cold and warm. The device has a 256 MB last-level cache in front of HBM, and a
kernel re-run on the same tensors finds part of them there. Every workload is
therefore built several times over (distinct tensor sets, as many as it takes
for more than 1 GiB to be touched between two uses of a set) and the calls
rotate over the sets: that is the *cold* figure, the one `value`, `roofline`
and `frac_hbm_peak` quote. The *warm* figure (the same set again and again) is
reported beside it.

  roofline      the dominant kernel of the headline workload against the
                MI355X HBM peak of 8 TB/s: cold average launch duration from
                events on the launch stream over the timed region, HBM traffic
                from the hardware counters recorded under profiles/,
  cpu_baseline  the CPU oracle (a loop-for-loop port of the reference's CPU
                kernels, single thread as the reference runs them) timed on the
                same workload on the host cores,
  kernels       per kernel of every workload of the sweep (the BASELINE
                configs, the >= 8192x4096 target shapes, shapes at the ends of
                the row-length range): cold mean / median / p10 / p90, warm mean,
                GB/s, elements/s, fraction of the HBM peak, fraction of the
                best streaming probe of the kernel's read : write mix at the kernel's
                tensor size (a ceiling: the probe is quoted on its fastest repetition
                and shape), and for the
                BASELINE configs the CPU oracle's rate and the speed-up.
"""

import argparse
import glob
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak
LLC_BYTES = 256 << 20  # last-level cache in front of HBM
COLD_BYTES = 4 * LLC_BYTES  # bytes touched between two uses of a tensor set


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="softmax_f16_16x32x512x512")
    ap.add_argument("--no-sweep", action="store_true", help="measure the headline workload only")
    ap.add_argument("--sweep", default="", help="comma-separated workloads to sweep instead of all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--timeline", default="", metavar="WORKLOAD",
                    help="print where the time of a LayerNorm workload's backward row kernel goes "
                         "(per-workgroup phase clock, per XCD) instead of the bench line")
    ap.add_argument("--structures", type=int, default=0, metavar="MB",
                    help="print what streaming two reads and one write over tensors of MB megabytes "
                         "reaches with one chunk per workgroup, as a persistent kernel, and with "
                         "store wavefronts, instead of the bench line")
    return ap.parse_args()


def measured_traffic():
    """{(workload, kernel): HBM bytes per launch} from the counter summaries under
    profiles/ (lines `traffic_bytes <workload> <kernel> <bytes>`)."""
    out = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "hbm_traffic_*.txt"))):
        for line in open(path):
            parts = line.lstrip("# ").split()
            if len(parts) == 4 and parts[0] == "traffic_bytes":
                out[(parts[1], parts[2])] = float(parts[3])
    return out


# ----------------------------------------------------------------------------
# Workloads: synthetic inputs with the distributions and seeds of the configs,
# generated on the device (the timed region starts with everything in HBM).
# Each factory takes the index of the tensor set (which only moves the seed)
# and returns (kernels, meta): kernels = [(name, fn, algorithmic_bytes, mix)],
# mix = the read : write ratio of the kernel ("1:1" or "2:1").
# ----------------------------------------------------------------------------

def _randn(shape, dtype, gen, scale=1.0, shift=0.0):
    import torch
    t = torch.empty(shape, dtype=torch.float32, device="cuda")
    t.normal_(generator=gen)
    if scale != 1.0 or shift != 0.0:
        t.mul_(scale).add_(shift)
    return t.to(dtype)


def _affine(C, gen):
    import torch
    g = torch.empty(C, device="cuda").uniform_(0.5, 1.5, generator=gen)
    b = torch.empty(C, device="cuda").normal_(generator=gen).mul_(0.1)
    return g, b


def _gen(seed):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


def wl_softmax(shape, dtype_name, seed=1, k=0):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed + 1000 * k)
    C = shape[-1]
    N = 1
    for d in shape[:-1]:
        N *= d
    x = _randn((N, C), torch.float32, gen, scale=3.0)
    mask = torch.empty((N, C), device="cuda").uniform_(generator=gen) < 0.05
    x[mask] = -1e4
    x = x.to(dtype)
    del mask
    dy = _randn((N, C), dtype, gen)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    nbytes = x.numel() * x.element_size()
    kernels = [
        ("softmax", lambda: K.softmax(N, 1, C, x, y), 2 * nbytes, "1:1"),
        ("softmax_grad", lambda: K.softmax_grad(N, 1, C, dy, y, dx), 3 * nbytes, "2:1"),
    ]
    return kernels, {"rows": N, "width": C}


def wl_lp_norm(N, C, dtype_name, p=2, seed=5, k=0):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed + 1000 * k)
    x = _randn((N, C), dtype, gen)
    dy = _randn((N, C), dtype, gen)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    nbytes = x.numel() * x.element_size()
    fwd, bwd = (K.l1_norm, K.l1_norm_grad) if p == 1 else (K.l2_norm, K.l2_norm_grad)
    kernels = [
        ("l%d_norm" % p, lambda: fwd(N, 1, C, 1.0, 1e-12, x, y), 2 * nbytes, "1:1"),
        ("l%d_norm_grad" % p, lambda: bwd(N, 1, C, 1.0, 1e-12, dy, x, dx), 3 * nbytes, "2:1"),
    ]
    return kernels, {"rows": N, "width": C}


def wl_softmax_cross_entropy(N, C, seed=6, k=0):
    """fp32 logits [N, C], int64 class indices, VALID reduction, 1 in 16 targets ignored."""
    import torch
    from dragon_amd import kernels as K
    gen = _gen(seed + 1000 * k)
    x = _randn((N, C), torch.float32, gen, scale=2.0)
    target = torch.randint(0, C, (N,), generator=gen, device="cuda", dtype=torch.int64)
    target[::16] = 255 if C > 255 else -1
    ignore = 255 if C > 255 else -1
    prob, dx = torch.empty_like(x), torch.empty_like(x)
    loss, dl = torch.empty(1, device="cuda"), torch.ones(1, device="cuda")
    nbytes = x.numel() * 4
    kernels = [
        ("softmax_cross_entropy_loss_forward",
         lambda: K.softmax_cross_entropy_loss_forward(N, 1, C, ignore, "valid", x, target, prob, loss),
         2 * nbytes + N * 8, "1:1"),
        ("softmax_cross_entropy_loss_backward",
         lambda: K.softmax_cross_entropy_loss_backward(N, 1, C, ignore, "valid", prob, target, dl, dx),
         2 * nbytes + N * 8, "1:1"),
    ]
    return kernels, {"rows": N, "width": C}


def wl_layer_norm(N, C, dtype_name, seed, backward=True, outliers=False, k=0):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed + 1000 * k)
    x = _randn((N, C), torch.float32, gen)
    if outliers:
        m = torch.empty((N, C), device="cuda").uniform_(generator=gen) < 0.01
        x[m] *= 50
        del m
    x = x.to(dtype)
    g, b = _affine(C, gen)
    y = torch.empty_like(x)
    mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    nbytes = x.numel() * x.element_size()
    kernels = [("layer_norm", lambda: K.layer_norm(N, C, 1e-5, x, g, b, mu, rsig, y),
                2 * nbytes + 2 * C * 4 + 2 * N * 4, "1:1")]
    if backward:
        dy = _randn((N, C), dtype, gen)
        dx = torch.empty_like(x)
        params = torch.empty(2 * N, device="cuda")
        dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
        kernels.append(("layer_norm_grad",
                        lambda: K.group_norm_grad(N, 1, C, 1, "NHWC", x, mu, rsig, g, dy, params,
                                                  params, dg, db, dx),
                        3 * nbytes + C * 4 + 2 * N * 4 + 2 * C * 4, "2:1"))
    return kernels, {"rows": N, "width": C}


def wl_group_norm(shape, G, dtype_name, seed=3, k=0, layout="NCHW"):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed + 1000 * k)
    N, C = shape[0], shape[1] if layout == "NCHW" else shape[-1]
    S = 1
    for d in (shape[2:] if layout == "NCHW" else shape[1:-1]):
        S *= d
    D = C // G
    x = _randn(shape, dtype, gen)
    dy = _randn(shape, dtype, gen)
    g, b = _affine(C, gen)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    mu, rsig = torch.empty(N * G, device="cuda"), torch.empty(N * G, device="cuda")
    params = torch.empty(2 * N * G, device="cuda")
    dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    nbytes = x.numel() * x.element_size()
    kernels = [
        ("group_norm_forward",
         lambda: K.group_norm_forward(N, G, D, S, layout, 1e-5, x, g, b, mu, rsig, y), 2 * nbytes,
         "1:1"),
        ("group_norm_grad",
         lambda: K.group_norm_grad(N, G, D, S, layout, x, mu, rsig, g, dy, params, params, dg, db, dx),
         3 * nbytes, "2:1"),
    ]
    return kernels, {"shape": list(shape), "groups": G, "layout": layout}


def wl_batch_norm(shape, dtype_name, seed=2, k=0):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed + 1000 * k)
    N, C = shape[0], shape[1]
    S = 1
    for d in shape[2:]:
        S *= d
    x = _randn(shape, dtype, gen, scale=2.0, shift=0.5)
    dy = _randn(shape, dtype, gen)
    g, b = _affine(C, gen)
    rm, rv = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
    y, dx = torch.empty_like(x), torch.empty_like(x)
    mu, rsig = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    params, wg = torch.empty(2 * C, device="cuda"), torch.empty(2 * C, device="cuda")
    nbytes = x.numel() * x.element_size()

    def backward():
        K.batch_norm_training_backward(N, C, S, float(N * S), "NCHW", x, mu, rsig, g, dy, wg, wg, dx)

    kernels = [
        ("batch_norm_training_forward",
         lambda: K.batch_norm_training_forward(N, C, S, "NCHW", 0.9, 1e-5, x, g, b, rm, rv, mu, rsig,
                                               params, y), 2 * nbytes, "1:1"),
        ("batch_norm_training_backward", backward, 3 * nbytes, "2:1"),
    ]
    return kernels, {"shape": list(shape)}


WORKLOADS = {
    # BASELINE configs
    "softmax_f16_16x32x512x512": lambda k: wl_softmax((16, 32, 512, 512), "float16", 1, k=k),
    "layer_norm_f32_8192x1024_fwd": lambda k: wl_layer_norm(8192, 1024, "float32", 0, backward=False, k=k),
    "batch_norm_f32_64x256x56x56": lambda k: wl_batch_norm((64, 256, 56, 56), "float32", 2, k=k),
    "group_norm_bf16_32x512x64x64_g32": lambda k: wl_group_norm((32, 512, 64, 64), 32, "bfloat16", 3, k=k),
    "layer_norm_bf16_8192x12288": lambda k: wl_layer_norm(8192, 12288, "bfloat16", 4, outliers=True, k=k),
    "layer_norm_bf16_65536x1000": lambda k: wl_layer_norm(65536, 1000, "bfloat16", 4, outliers=True, k=k),
    # target shapes (>= 8192 x 4096)
    "layer_norm_bf16_8192x4096": lambda k: wl_layer_norm(8192, 4096, "bfloat16", 4, k=k),
    "layer_norm_f32_8192x4096": lambda k: wl_layer_norm(8192, 4096, "float32", 4, k=k),
    # the same row widths with four times the rows: what the kernels sustain once the fixed
    # cost of a call (first loads, last stores, the second stage of dgamma / dbeta) is spread
    "layer_norm_bf16_32768x4096": lambda k: wl_layer_norm(32768, 4096, "bfloat16", 4, k=k),
    "layer_norm_bf16_32768x12288": lambda k: wl_layer_norm(32768, 12288, "bfloat16", 4, k=k),
    "softmax_f16_8192x4096": lambda k: wl_softmax((8192, 4096), "float16", 1, k=k),
    "softmax_f32_8192x4096": lambda k: wl_softmax((8192, 4096), "float32", 1, k=k),
    # sibling row reductions on the same skeleton
    "softmax_cross_entropy_f32_8192x4096": lambda k: wl_softmax_cross_entropy(8192, 4096, k=k),
    "l2_norm_bf16_8192x4096": lambda k: wl_lp_norm(8192, 4096, "bfloat16", 2, k=k),
    "l2_norm_f32_8192x4096": lambda k: wl_lp_norm(8192, 4096, "float32", 2, k=k),
    # shapes at the ends of the row-length range: attention rows of a vision transformer,
    # per-head normalisation, vocabulary-sized logits
    "softmax_bf16_605184x197": lambda k: wl_softmax((605184, 197), "bfloat16", 1, k=k),
    "layer_norm_bf16_1048576x64": lambda k: wl_layer_norm(1048576, 64, "bfloat16", 4, k=k),
    "softmax_f32_2048x128256": lambda k: wl_softmax((2048, 128256), "float32", 1, k=k),
    # feature maps that are not whole 16-byte packets (the BASELINE BatchNorm shape at 57x57)
    "batch_norm_f32_64x256x57x57": lambda k: wl_batch_norm((64, 256, 57, 57), "float32", 2, k=k),
    # a vocabulary whose rows are not whole 16-byte packets
    "softmax_bf16_4096x50257": lambda k: wl_softmax((4096, 50257), "bfloat16", 1, k=k),
    # the BASELINE GroupNorm tensor channels-last: samples of 4 MB cut into slices of rows
    "group_norm_bf16_32x64x64x512_g32_nhwc": lambda k: wl_group_norm((32, 64, 64, 512), 32, "bfloat16", 3,
                                                                     k=k, layout="NHWC"),
}


def build_sets(name):
    """The workload's tensor sets: enough of them that more than COLD_BYTES are touched
    between two uses of a set even when only its smallest kernel is being timed."""
    import torch
    first = WORKLOADS[name](0)
    smallest = min(k[2] for k in first[0])
    count = max(2, min(24, int(math.ceil(COLD_BYTES / smallest)) + 1))
    sets = [first] + [WORKLOADS[name](k) for k in range(1, count)]
    for kernels, _ in sets:  # backward kernels read what the forward of their set wrote
        for _, fn, _, _ in kernels:
            fn()
    torch.cuda.synchronize()
    return sets


def time_calls(fns, steps, warmup):
    """fns[i % len(fns)] is call i. Returns (mean ms over `steps` calls from one pair of
    events around the region, sorted per-call ms from an event between any two calls);
    events are recorded on the stream the kernels are launched on."""
    import torch
    n = len(fns)
    for i in range(max(warmup, n)):
        fns[i % n]()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fns[i % n]()
    stop.record()
    torch.cuda.synchronize()
    mean = start.elapsed_time(stop) / steps
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    marks[0].record()
    for i in range(steps):
        fns[i % n]()
        marks[i + 1].record()
    torch.cuda.synchronize()
    each = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    return mean, each


def _pct(sorted_values, q):
    return sorted_values[min(len(sorted_values) - 1, int(q * len(sorted_values)))]


def measure_workload(name, steps, warmup):
    import torch
    sets = build_sets(name)
    meta = sets[0][1]
    elems = 1
    for d in meta.get("shape", (meta.get("rows", 1), meta.get("width", 1))):
        elems *= d
    per_kernel = []
    for j, (kname, _, nbytes, mix) in enumerate(sets[0][0]):
        cold_mean, cold_each = time_calls([s[0][j][1] for s in sets], steps, warmup)
        warm_mean, _ = time_calls([sets[0][0][j][1]], steps, warmup)
        gbs = nbytes / (cold_mean * 1e-3) / 1e9
        warm_gbs = nbytes / (warm_mean * 1e-3) / 1e9
        per_kernel.append({
            "workload": name, "kernel": kname, "mix": mix, "tensor_sets": len(sets),
            "us": round(cold_mean * 1e3, 2),
            "us_median": round(_pct(cold_each, 0.5) * 1e3, 2),
            "us_p10": round(_pct(cold_each, 0.1) * 1e3, 2),
            "us_p90": round(_pct(cold_each, 0.9) * 1e3, 2),
            "algorithmic_bytes": nbytes, "GB/s": round(gbs, 1),
            "Gelem/s": round(elems / (cold_mean * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "warm_us": round(warm_mean * 1e3, 2),
            "frac_hbm_peak_warm": round(warm_gbs / HBM_PEAK_GBS, 4)})

    def step(i):
        for _, fn, _, _ in sets[i % len(sets)][0]:
            fn()

    # the contract's timed region: W warm-up steps, then exactly K steps between syncs,
    # rotating over the tensor sets
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    total_bytes = sum(k[2] for k in sets[0][0])
    del sets
    torch.cuda.empty_cache()
    return per_kernel, ms_step, total_bytes


PROBE_SHAPES = ((64, 1), (64, 2), (64, 4), (256, 1), (256, 2), (256, 4), (512, 2))


def streaming_ceiling(steps, warmup):
    """Achieved GB/s of plain streaming kernels over 1 GiB buffers of non-zero data (far
    beyond the last-level cache): read only, copy, fill, and two reads with one write."""
    import torch
    from dragon_amd import kernels as K
    n = 1 << 30
    a = torch.randint(1, 255, (2 * n,), dtype=torch.uint8, device="cuda")
    b = torch.empty(n, dtype=torch.uint8, device="cuda")
    out = {}
    for name, mode, moved in (("read", 0, n), ("copy", 1, 2 * n), ("fill", 2, n),
                              ("two_reads_one_write", 3, 3 * n)):
        ms, _ = time_calls([lambda: K.stream_probe(mode, a, b, n)], steps, warmup)
        out[name] = round(moved / (ms * 1e-3) / 1e9, 1)
    return out


_probe_cache = {}


def probe_ceiling(tensor_bytes, mix, steps=16, reps=3):
    """What a kernel of this read : write mix can reach at most at this tensor size: the best
    streaming probe, over the probe's shapes (threads per workgroup x loads in flight) and
    over `reps` repetitions (the fastest one, where kernels are quoted on their mean), of a
    copy ("1:1") or of two reads and one write ("2:1") over tensors of `tensor_bytes` each,
    cold: rotating over as many buffer sets as the workloads do. Returns (GB/s, shape)."""
    import torch
    from dragon_amd import kernels as K
    tensor_bytes = max(16, (int(tensor_bytes) + 15) // 16 * 16)
    key = (tensor_bytes, mix)
    if key in _probe_cache:
        return _probe_cache[key]
    reads, mode = (1, 1) if mix == "1:1" else (2, 3)
    moved = (reads + 1) * tensor_bytes
    count = max(2, min(24, int(math.ceil(COLD_BYTES / moved)) + 1))
    sets = [(torch.randint(1, 255, (reads * tensor_bytes,), dtype=torch.uint8, device="cuda"),
             torch.empty(tensor_bytes, dtype=torch.uint8, device="cuda")) for _ in range(count)]
    best = (0.0, None)
    for shape in PROBE_SHAPES:
        fns = [(lambda a=a, b=b: K.stream_probe(mode, a, b, tensor_bytes, shape)) for a, b in sets]
        for _ in range(reps):
            ms, _each = time_calls(fns, steps, count)
            gbs = moved / (ms * 1e-3) / 1e9
            if gbs > best[0]:
                best = (gbs, shape)
    del sets
    torch.cuda.empty_cache()
    _probe_cache[key] = (round(best[0], 1), "%dx%d" % best[1])
    return _probe_cache[key]


# ----------------------------------------------------------------------------
# CPU baseline: the oracle (a port of the reference's CPU kernels, one thread,
# as the reference runs them) on the same seeded distributions, full size where
# a pass takes about a second, otherwise on a stated share of the rows.
# Returns {(workload, kernel): {"GB/s": ..., "sample": ...}} with the same
# algorithmic bytes per element the GPU figure is quoted on.
# ----------------------------------------------------------------------------

def _timed(fn, reps):
    times = []
    out = None
    for _ in range(reps):
        t0 = time.perf_counter()
        out = fn()
        times.append(time.perf_counter() - t0)
    return sorted(times)[len(times) // 2], out


def cpu_baselines(reps=3):
    import numpy as np
    from oracle import ref_cpu as R
    out = {}

    def put(workload, kernel, nbytes, seconds, sample, passes=reps):
        out[(workload, kernel)] = {"GB/s": round(nbytes / seconds / 1e9, 3),
                                   "sample": "%s, median of %d, %.2f s per pass" % (sample, passes, seconds)}

    def rounded(a, dtype):
        return R.from_bits(R.to_bits(a, dtype), dtype)

    # cfg 2: Softmax + SoftmaxGrad, fp32 kernels on the fp16-rounded inputs, every row
    N, C = 16 * 32 * 512, 512
    rng = np.random.default_rng(1)
    x = rng.standard_normal((N, C), dtype=np.float32) * 3
    x[rng.random((N, C), dtype=np.float32) < 0.05] = -1e4
    x = rounded(x, "float16")
    dy = rounded(rng.standard_normal((N, C), dtype=np.float32), "float16")
    t_f, y = _timed(lambda: R.softmax("float32", N, 1, C, x), reps)
    t_b, _ = _timed(lambda: R.softmax_grad("float32", N, 1, C, dy, y), reps)
    name = "softmax_f16_16x32x512x512"
    what = "all %d rows of %d, fp32 oracle on fp16-rounded inputs" % (N, C)
    put(name, "softmax", 2 * N * C * 2, t_f, what)
    put(name, "softmax_grad", 3 * N * C * 2, t_b, what)
    del x, dy, y

    # cfg 1: LayerNorm forward fp32, full size
    N, C = 8192, 1024
    rng = np.random.default_rng(0)
    x = rng.standard_normal((N, C), dtype=np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = (rng.standard_normal(C) * 0.1).astype(np.float32)
    t, _ = _timed(lambda: R.layer_norm("float32", x, g, b, 1e-5), reps)
    put("layer_norm_f32_8192x1024_fwd", "layer_norm", 2 * N * C * 4, t, "full [%d, %d] fp32" % (N, C))

    # cfg 3: BatchNorm training forward + backward fp32 NCHW, full size
    shape = (64, 256, 56, 56)
    rng = np.random.default_rng(2)
    x = (2 * rng.standard_normal(shape, dtype=np.float32) + 0.5).astype(np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    g = rng.uniform(0.5, 1.5, shape[1]).astype(np.float32)
    b = (rng.standard_normal(shape[1]) * 0.1).astype(np.float32)
    rm, rv = np.zeros(shape[1], np.float32), np.ones(shape[1], np.float32)
    t_f, (y, mu, rsig, _) = _timed(
        lambda: R.op_batch_norm_train("float32", x, g, b, rm.copy(), rv.copy(), 1, 0.9, 1e-5), 1)
    t_b, _ = _timed(lambda: R.op_batch_norm_train_grad("float32", x, g, dy, mu, rsig, 1), 1)
    name = "batch_norm_f32_64x256x56x56"
    put(name, "batch_norm_training_forward", 2 * x.size * 4, t_f, "full %s fp32" % (list(shape),), 1)
    put(name, "batch_norm_training_backward", 3 * x.size * 4, t_b, "full %s fp32" % (list(shape),), 1)
    del x, dy, y

    # cfg 4: GroupNorm bf16 NCHW, 32 groups: 4 of the 32 samples (the forward in the
    # reference's software bf16, the backward as its fp32 kernel on the rounded inputs)
    shape = (4, 512, 64, 64)
    rng = np.random.default_rng(3)
    xb = R.to_bits(rng.standard_normal(shape, dtype=np.float32), "bfloat16")
    dyf = rounded(rng.standard_normal(shape, dtype=np.float32), "bfloat16")
    g = rng.uniform(0.5, 1.5, shape[1]).astype(np.float32)
    b = (rng.standard_normal(shape[1]) * 0.1).astype(np.float32)
    t_f, (_, mu, rsig) = _timed(lambda: R.op_group_norm("bfloat16", xb, g, b, 1, 32, 1e-5), reps)
    xf = R.from_bits(xb, "bfloat16")
    t_b, _ = _timed(lambda: R.op_group_norm_grad("float32", xf, g, dyf, mu, rsig, 1, 32), reps)
    name = "group_norm_bf16_32x512x64x64_g32"
    put(name, "group_norm_forward", 2 * xb.size * 2, t_f, "4 of 32 samples, %s bf16" % (list(shape),))
    put(name, "group_norm_grad", 3 * xb.size * 2, t_b,
        "4 of 32 samples, %s, fp32 oracle on bf16-rounded inputs" % (list(shape),))
    del xb, xf, dyf

    # cfg 5: LayerNorm bf16 forward + backward on a share of the rows
    for (rows, C, sample) in ((8192, 12288, 512), (65536, 1000, 4096)):
        rng = np.random.default_rng(4)
        x = rng.standard_normal((sample, C), dtype=np.float32)
        x[rng.random((sample, C), dtype=np.float32) < 0.01] *= 50
        xb = R.to_bits(x, "bfloat16")
        dyf = rounded(rng.standard_normal((sample, C), dtype=np.float32), "bfloat16")
        g = rng.uniform(0.5, 1.5, C).astype(np.float32)
        b = (rng.standard_normal(C) * 0.1).astype(np.float32)
        t_f, (_, mu, rsig) = _timed(lambda: R.layer_norm("bfloat16", xb, g, b, 1e-5), reps)
        xf = R.from_bits(xb, "bfloat16")
        t_b, _ = _timed(lambda: R.group_norm_grad("float32", sample, 1, C, 1, "NHWC", xf, mu, rsig, g,
                                                  dyf), reps)
        name = "layer_norm_bf16_%dx%d" % (rows, C)
        put(name, "layer_norm", 2 * sample * C * 2, t_f, "%d of %d rows of %d, bf16" % (sample, rows, C))
        put(name, "layer_norm_grad", 3 * sample * C * 2, t_b,
            "%d of %d rows of %d, fp32 oracle on bf16-rounded inputs" % (sample, rows, C))
    return out


def timeline_report(name, reps=5):
    """Phase clock of the persistent row kernel behind a LayerNorm workload's backward: one cold
    call per tensor set with every workgroup recording (start, first row summed, row loop end,
    end). Prints, per call, the spread over the workgroups and per XCD; times in microseconds
    since the first workgroup's start."""
    import torch
    from dragon_amd import kernels as K
    import re
    m = re.match(r"layer_norm_(bf16|f32)_(\d+)x(\d+)", name)
    if not m:
        raise SystemExit("--timeline takes a layer_norm_<dtype>_<rows>x<width> workload")
    dtype = torch.bfloat16 if m.group(1) == "bf16" else torch.float32
    N, C = int(m.group(2)), int(m.group(3))
    gen = _gen(4)
    sets = []
    nbytes = N * C * (2 if dtype == torch.bfloat16 else 4)
    for k in range(max(3, int(math.ceil(COLD_BYTES / (3 * nbytes))) + 1)):
        x, dy = _randn((N, C), dtype, gen), _randn((N, C), dtype, gen)
        g, b = _affine(C, gen)
        y, dx = torch.empty_like(x), torch.empty_like(x)
        mu, rsig = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
        K.layer_norm(N, C, 1e-5, x, g, b, mu, rsig, y)
        sets.append((x, dy, g, mu, rsig, dx, torch.empty(2 * N, device="cuda"),
                     torch.empty(C, device="cuda"), torch.empty(C, device="cuda")))
    torch.cuda.synchronize()
    print("# %s: LayerNorm backward, %d tensor sets of %.0f MB, plan %s" % (
        name, len(sets), 3 * nbytes / 1e6,
        K.plan_name("layer_norm_grad", "bfloat16" if dtype == torch.bfloat16 else "float32", (N, C))))
    import numpy as np
    calls = []
    for rep in range(reps + 1):  # the first round warms the code up and is not counted
        for x, dy, g, mu, rsig, dx, params, dg, db in sets:
            stamps = K.group_norm_grad_timeline(N, 1, C, 1, "NHWC", x, mu, rsig, g, dy, params, params,
                                                dg, db, dx)
            torch.cuda.synchronize()
            if rep == 0:
                continue
            t = stamps.cpu().numpy()
            t = t[t[:, 0] > 0]
            if not len(t):
                raise SystemExit("this workload does not take the persistent row kernel")
            calls.append((t[:, 4].copy(), (t[:, :4] - t[:, 0].min()) * 0.01, t[:, 5].copy()))
    us = np.stack([c[1] for c in calls])  # [call, workgroup, phase]
    print("%d cold calls, %d workgroups, %d rows per row group; microseconds since the first "
          "workgroup's start, averaged over the calls" % (len(calls), us.shape[1], int(calls[0][2].max())))
    for c, what in enumerate(("start", "first row summed", "row loop end", "workgroup end")):
        print("  %-17s first %6.2f   mean %6.2f   last %6.2f" % (
            what, us[:, :, c].min(1).mean(), us[:, :, c].mean(1).mean(), us[:, :, c].max(1).mean()))
    span = us[:, :, 3].max(1)
    busy = (us[:, :, 3] - us[:, :, 0]).mean(1)
    print("  kernel span (first start to last end) %.2f us; a workgroup is busy %.2f us on average: "
          "%.2f us (%.1f%%) of the span is waiting for the slowest workgroups"
          % (span.mean(), busy.mean(), (span - busy).mean(), 100 * ((span - busy) / span).mean()))
    steps = int(calls[0][2].max())
    first = (us[:, :, 1] - us[:, :, 0]).mean()
    steady = ((us[:, :, 2] - us[:, :, 1]).mean()) / max(1, steps - 1)
    print("  first row %.2f us after the workgroup's start, then %.2f us per row-loop trip; the partial "
          "row takes %.2f us" % (first, steady, (us[:, :, 3] - us[:, :, 2]).mean()))
    print("  per XCD (mean over calls and workgroups):")
    xcd_of = calls[0][0]
    for xcd in sorted(set(xcd_of)):
        rows = [c[1][c[0] == xcd] for c in calls]
        sel = np.concatenate(rows)
        print("   XCD %d: start %.2f  row loop %.2f  end %.2f (last %.2f)" % (
            xcd, sel[:, 0].mean(), (sel[:, 2] - sel[:, 0]).mean(), sel[:, 3].mean(),
            np.mean([r[:, 3].max() for r in rows])))


def structures_report(mb, steps=32, reps=3):
    """What the *structure* of a kernel costs when it streams two reads and one write over three
    tensors of `mb` megabytes, cold: one chunk per workgroup (the probe's shapes), persistent
    workgroups with chunks requested ahead, and persistent workgroups whose stores are issued
    by separate wavefronts."""
    import torch
    from dragon_amd import kernels as K
    nbytes = mb << 20
    moved = 3 * nbytes
    count = max(3, int(math.ceil(COLD_BYTES / moved)) + 1)
    sets = [(torch.randint(1, 255, (2 * nbytes,), dtype=torch.uint8, device="cuda"),
             torch.empty(nbytes, dtype=torch.uint8, device="cuda")) for _ in range(count)]

    def best(make):
        fns = [make(a, b) for a, b in sets]
        return min(time_calls(fns, steps, count)[0] for _ in range(reps)) * 1e3

    print("# two reads and one write, 3 x %d MB, %d buffer sets, best of %d runs of %d calls" % (
        mb, count, reps, steps))
    for shape in PROBE_SHAPES + ((1024, 2),):
        us = best(lambda a, b, shape=shape: (lambda: K.stream_probe(3, a, b, nbytes, shape)))
        print("one chunk per workgroup   %4d threads x %d in flight                      %7.2f us  %.3f of 8 TB/s"
              % (shape + (us, moved / us / 8e6)))
    for threads, flight, per_cu, depth, barrier, split in (
            (256, 2, 8, 0, 0, 0), (256, 2, 4, 1, 0, 0), (256, 2, 4, 2, 0, 0), (512, 2, 2, 1, 1, 0),
            (1024, 2, 1, 1, 0, 0), (1024, 2, 1, 1, 1, 0), (1024, 2, 1, 2, 1, 0), (1024, 1, 1, 3, 1, 0),
            (1024, 2, 1, 1, 1, 1), (1024, 2, 1, 2, 1, 1), (512, 2, 2, 1, 1, 1)):
        us = best(lambda a, b: (lambda: K.stream_probe_persistent(a, b, nbytes, threads, flight, per_cu, depth,
                                                                  barrier, split)))
        print("persistent %-14s %4d threads x %d in flight, %d per CU, %d ahead%s  %7.2f us  %.3f of 8 TB/s"
              % ("store waves" if split else "", threads, flight, per_cu, depth,
                 ", barrier" if barrier else "         ", us, moved / us / 8e6))


def contract_problems(line):
    """What is wrong with a parsed bench line, as a list of sentences (empty when nothing is):
    the fields the driver reads, the roofline arithmetic, and the probe as a ceiling, i.e. no
    kernel row above 1.00 of the best streaming kernel of its mix and tensor size."""
    bad = []
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline",
                "cpu_baseline"):
        if key not in line:
            bad.append("missing field %s" % key)
    roof = line.get("roofline") or {}
    if roof:
        if roof.get("bound") != "hbm" or roof.get("peak") != HBM_PEAK_GBS:
            bad.append("roofline is not against the HBM peak")
        if abs(roof.get("frac", 0) - roof.get("achieved", 0) / HBM_PEAK_GBS) > 1e-3:
            bad.append("roofline.frac is not achieved / peak")
        if roof.get("frac", 0) > 1.0:
            bad.append("roofline.frac above 1")
    for k in line.get("kernels", []):
        name = "%s/%s" % (k.get("workload"), k.get("kernel"))
        if k.get("frac_hbm_peak", 0) > 1.0:
            bad.append("%s: above the HBM peak" % name)
        if abs(k.get("frac_hbm_peak", 0) - k.get("GB/s", 0) / HBM_PEAK_GBS) > 1e-3:
            bad.append("%s: frac_hbm_peak is not GB/s over the peak" % name)
        if "frac_stream_probe" in k and k["frac_stream_probe"] > 1.0:
            bad.append("%s: %.3f of the streaming probe, which is meant to be a ceiling"
                       % (name, k["frac_stream_probe"]))
    return bad


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from dragon_amd import _lib
    _lib.lib()  # fail loudly if the HIP library is not built
    if args.timeline:
        return timeline_report(args.timeline)
    if args.structures:
        return structures_report(args.structures)

    head = args.workload
    per_kernel, ms_step, total_bytes = measure_workload(head, args.steps, args.warmup)
    value = total_bytes / (ms_step * 1e-3) / 1e9
    dominant = max(per_kernel, key=lambda k: k["us"])
    all_kernels = list(per_kernel)
    if not args.no_sweep:
        for name in (args.sweep.split(",") if args.sweep else WORKLOADS):
            if name != head:
                all_kernels += measure_workload(name, args.steps, args.warmup)[0]
    ceiling = streaming_ceiling(20, 5)
    for k in all_kernels:
        # the second denominator: the best plain streaming kernel of the same mix at the same
        # tensor size, measured cold like the kernel itself; no kernel can stream faster
        tensors = 2 if k["mix"] == "1:1" else 3
        probe, shape = probe_ceiling(k["algorithmic_bytes"] / tensors, k["mix"])
        # the probe had a slow moment: ask it again, more often and over as many calls per
        # repetition as the kernel's own figure averages (it is a best-of, so it can only rise)
        for reps in (8, 16):
            if k["GB/s"] <= probe:
                break
            _probe_cache.pop((max(16, (int(k["algorithmic_bytes"] / tensors) + 15) // 16 * 16), k["mix"]), None)
            again, again_shape = probe_ceiling(k["algorithmic_bytes"] / tensors, k["mix"],
                                               steps=max(16, args.steps), reps=reps)
            if again > probe:
                probe, shape = again, again_shape
        k["probe_GB/s"] = probe
        k["probe_shape"] = shape
        k["frac_stream_probe"] = round(k["GB/s"] / probe, 3)

    cpu = None
    if not args.no_cpu:
        cpus = cpu_baselines()
        for k in all_kernels:
            c = cpus.get((k["workload"], k["kernel"]))
            if c:
                k["cpu_GB/s"] = c["GB/s"]
                k["cpu_sample"] = c["sample"]
                k["speedup_vs_cpu"] = round(k["GB/s"] / c["GB/s"], 1)
        mine = [cpus[(head, k["kernel"])] for k in per_kernel if (head, k["kernel"]) in cpus]
        if len(mine) == len(per_kernel):
            # the whole step on the CPU: total bytes over the summed pass times
            secs = sum(k["algorithmic_bytes"] / (c["GB/s"] * 1e9) for k, c in zip(per_kernel, mine))
            cpu = {"value": round(total_bytes / secs / 1e9, 3), "unit": "GB/s", "cores": 1,
                   "kind": "port", "host_cores": os.cpu_count(),
                   "sample": "; ".join("%s: %s" % (k["kernel"], c["sample"])
                                       for k, c in zip(per_kernel, mine))}

    out = {
        "metric": "GB/s and % of HBM roofline per norm/softmax kernel; speedup vs host-CPU ref",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # every reduction and the element-wise math run in fp32; I/O type is in config
        "data": "synthetic",
        "config": {"workload": head, "io_dtype": "f16" if "f16" in head else ("bf16" if "bf16" in head else "f32"),
                   "step": "forward + backward, inputs resident in HBM, rotating over tensor sets "
                           "so that no call finds its tensors in the last-level cache",
                   "algorithmic_bytes_per_step": total_bytes},
        "roofline": {"bound": "hbm", "kernel": dominant["kernel"],
                     "achieved": dominant["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dominant["GB/s"] / HBM_PEAK_GBS, 4),
                     "avg_launch_us": dominant["us"],
                     "frac_warm": dominant["frac_hbm_peak_warm"],
                     "traffic": measured_traffic().get((head, dominant["kernel"])),
                     "streaming_kernels_GB/s": ceiling},
        "cpu_baseline": cpu,
        "kernels": all_kernels,
    }
    if cpu:
        out["speedup_vs_cpu"] = round(value / cpu["value"], 1)
    for problem in contract_problems(out):
        print("bench.py: " + problem, file=sys.stderr)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
