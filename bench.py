#!/usr/bin/env python3
"""Benchmark of the norm / softmax hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-sweep] [--no-cpu]

A step is one pass of the workload's kernels (forward then backward) over one
batch of synthetic input that is already resident in HBM. The headline
workload is Softmax forward+backward, fp16 I/O, [16, 32, 512, 512] along the
last axis; `value` is its algorithmic bytes per step divided by the time per
step. One JSON line is printed. It also carries
  roofline      the dominant kernel of the headline workload against the
                MI355X HBM peak of 8 TB/s (average launch duration measured
                with events on the launch stream),
  cpu_baseline  the CPU oracle (a loop-for-loop port of the reference's CPU
                kernels, single thread as the reference runs them) timed on the
                same workload on the host cores,
  kernels       the same per-kernel measurement for every workload of the
                sweep (LayerNorm, GroupNorm, BatchNorm and the >= 8192x4096
                target shapes).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE hardware counters, each
# scaled by what it reads for the 1 GiB streaming-copy probe (figures and
# commands: profiles/hbm_traffic_softmax_f16_16x32x512x512.txt).
MEASURED_TRAFFIC_BYTES = {
    ("softmax_f16_16x32x512x512", "softmax"): 536.9e6,
    ("softmax_f16_16x32x512x512", "softmax_grad"): 805.4e6,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="softmax_f16_16x32x512x512")
    ap.add_argument("--no-sweep", action="store_true", help="measure the headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    return ap.parse_args()


# ----------------------------------------------------------------------------
# Workloads: synthetic inputs with the distributions and seeds of the configs,
# generated on the device (the timed region starts with everything in HBM).
# Each returns (kernels, meta): kernels = [(name, fn, algorithmic_bytes)].
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


def wl_softmax(shape, dtype_name, seed=1):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed)
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
        ("softmax", lambda: K.softmax(N, 1, C, x, y), 2 * nbytes),
        ("softmax_grad", lambda: K.softmax_grad(N, 1, C, dy, y, dx), 3 * nbytes),
    ]
    return kernels, {"rows": N, "width": C, "tensors": (x, dy, y, dx)}


def wl_lp_norm(N, C, dtype_name, p=2, seed=5):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed)
    x = _randn((N, C), dtype, gen)
    dy = _randn((N, C), dtype, gen)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    nbytes = x.numel() * x.element_size()
    fwd, bwd = (K.l1_norm, K.l1_norm_grad) if p == 1 else (K.l2_norm, K.l2_norm_grad)
    kernels = [
        ("l%d_norm" % p, lambda: fwd(N, 1, C, 1.0, 1e-12, x, y), 2 * nbytes),
        ("l%d_norm_grad" % p, lambda: bwd(N, 1, C, 1.0, 1e-12, dy, x, dx), 3 * nbytes),
    ]
    return kernels, {"rows": N, "width": C}


def wl_softmax_cross_entropy(N, C, seed=6):
    """fp32 logits [N, C], int64 class indices, VALID reduction, 1 in 16 targets ignored."""
    import torch
    from dragon_amd import kernels as K
    gen = _gen(seed)
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
         2 * nbytes + N * 8),
        ("softmax_cross_entropy_loss_backward",
         lambda: K.softmax_cross_entropy_loss_backward(N, 1, C, ignore, "valid", prob, target, dl, dx),
         2 * nbytes + N * 8),
    ]
    return kernels, {"rows": N, "width": C}


def wl_layer_norm(N, C, dtype_name, seed, backward=True, outliers=False):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed)
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
                2 * nbytes + 2 * C * 4 + 2 * N * 4)]
    if backward:
        dy = _randn((N, C), dtype, gen)
        dx = torch.empty_like(x)
        params = torch.empty(2 * N, device="cuda")
        dg, db = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
        kernels.append(("layer_norm_grad",
                        lambda: K.group_norm_grad(N, 1, C, 1, "NHWC", x, mu, rsig, g, dy, params,
                                                  params, dg, db, dx),
                        3 * nbytes + C * 4 + 2 * N * 4 + 2 * C * 4))
    return kernels, {"rows": N, "width": C}


def wl_group_norm(shape, G, dtype_name, seed=3):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed)
    N, C = shape[0], shape[1]
    S = 1
    for d in shape[2:]:
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
         lambda: K.group_norm_forward(N, G, D, S, "NCHW", 1e-5, x, g, b, mu, rsig, y), 2 * nbytes),
        ("group_norm_grad",
         lambda: K.group_norm_grad(N, G, D, S, "NCHW", x, mu, rsig, g, dy, params, params, dg, db, dx),
         3 * nbytes),
    ]
    return kernels, {"shape": list(shape), "groups": G}


def wl_batch_norm(shape, dtype_name, seed=2):
    import torch
    from dragon_amd import kernels as K
    dtype = getattr(torch, dtype_name)
    gen = _gen(seed)
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
                                               params, y), 2 * nbytes),
        ("batch_norm_training_backward", backward, 3 * nbytes),
    ]
    return kernels, {"shape": list(shape)}


WORKLOADS = {
    # BASELINE configs
    "softmax_f16_16x32x512x512": lambda: wl_softmax((16, 32, 512, 512), "float16", 1),
    "layer_norm_f32_8192x1024_fwd": lambda: wl_layer_norm(8192, 1024, "float32", 0, backward=False),
    "batch_norm_f32_64x256x56x56": lambda: wl_batch_norm((64, 256, 56, 56), "float32", 2),
    "group_norm_bf16_32x512x64x64_g32": lambda: wl_group_norm((32, 512, 64, 64), 32, "bfloat16", 3),
    "layer_norm_bf16_8192x12288": lambda: wl_layer_norm(8192, 12288, "bfloat16", 4, outliers=True),
    "layer_norm_bf16_65536x1000": lambda: wl_layer_norm(65536, 1000, "bfloat16", 4, outliers=True),
    # target shapes (>= 8192 x 4096)
    "layer_norm_bf16_8192x4096": lambda: wl_layer_norm(8192, 4096, "bfloat16", 4),
    "layer_norm_f32_8192x4096": lambda: wl_layer_norm(8192, 4096, "float32", 4),
    "softmax_f16_8192x4096": lambda: wl_softmax((8192, 4096), "float16", 1),
    "softmax_f32_8192x4096": lambda: wl_softmax((8192, 4096), "float32", 1),
    # sibling row reductions on the same skeleton
    "softmax_cross_entropy_f32_8192x4096": lambda: wl_softmax_cross_entropy(8192, 4096),
    "l2_norm_bf16_8192x4096": lambda: wl_lp_norm(8192, 4096, "bfloat16", 2),
    "l2_norm_f32_8192x4096": lambda: wl_lp_norm(8192, 4096, "float32", 2),
    # shapes at the ends of the row-length range: attention rows of a vision transformer,
    # per-head normalisation, vocabulary-sized logits
    "softmax_bf16_605184x197": lambda: wl_softmax((605184, 197), "bfloat16", 1),
    "layer_norm_bf16_1048576x64": lambda: wl_layer_norm(1048576, 64, "bfloat16", 4),
    "softmax_f32_2048x128256": lambda: wl_softmax((2048, 128256), "float32", 1),
}


def time_calls(fn, steps, warmup):
    """Average milliseconds per call of fn over `steps` calls, events on the launch stream."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def measure_workload(name, steps, warmup):
    import torch
    kernels, meta = WORKLOADS[name]()
    per_kernel = []
    for kname, fn, nbytes in kernels:
        ms = time_calls(fn, steps, warmup)
        gbs = nbytes / (ms * 1e-3) / 1e9
        elems = 1
        for d in meta.get("shape", (meta.get("rows", 1), meta.get("width", 1))):
            elems *= d
        per_kernel.append({"workload": name, "kernel": kname, "us": round(ms * 1e3, 2),
                           "algorithmic_bytes": nbytes, "GB/s": round(gbs, 1),
                           "Gelem/s": round(elems / (ms * 1e-3) / 1e9, 1),
                           "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)})

    def step():
        for _, fn, _ in kernels:
            fn()

    # the contract's timed region: W warm-up steps, then exactly K steps between syncs
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    total_bytes = sum(k[2] for k in kernels)
    del kernels, meta
    torch.cuda.empty_cache()
    return per_kernel, ms_step, total_bytes


def streaming_ceiling(steps, warmup):
    """Achieved GB/s of plain streaming kernels over 1 GiB buffers (far beyond the
    256 MB last-level cache): read only, copy (read + write bytes) and fill."""
    import torch
    from dragon_amd import kernels as K
    n = 1 << 30
    a = torch.zeros(n, dtype=torch.uint8, device="cuda")
    b = torch.empty(n, dtype=torch.uint8, device="cuda")
    out = {}
    for name, mode, moved in (("read", 0, n), ("copy", 1, 2 * n), ("fill", 2, n)):
        ms = time_calls(lambda: K.stream_probe(mode, a, b, n), steps, warmup)
        out[name] = round(moved / (ms * 1e-3) / 1e9, 1)
    return out


def cpu_baseline_softmax(shape, reps=3):
    """Oracle Softmax + SoftmaxGrad (fp32 kernels on the fp16-rounded inputs) on the
    full headline workload, single thread, median of `reps`."""
    import numpy as np
    from oracle import ref_cpu as R
    C = shape[-1]
    N = int(np.prod(shape[:-1]))
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((N, C), dtype=np.float32) * 3)
    x[rng.random((N, C), dtype=np.float32) < 0.05] = -1e4
    x = R.from_bits(R.to_bits(x, "float16"), "float16")
    dy = R.from_bits(R.to_bits(rng.standard_normal((N, C), dtype=np.float32), "float16"), "float16")
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        y = R.softmax("float32", N, 1, C, x)
        R.softmax_grad("float32", N, 1, C, dy, y)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[len(times) // 2]
    nbytes_fp16 = 5 * N * C * 2  # the same algorithmic bytes the GPU number is quoted on
    return {"value": round(nbytes_fp16 / t / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "host_cores": os.cpu_count(),
            "sample": "full workload [%d, %d], Softmax+SoftmaxGrad fp32 oracle on fp16-rounded "
                      "inputs, median of %d, %.2f s per pass" % (N, C, reps, t)}


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

    head = args.workload
    per_kernel, ms_step, total_bytes = measure_workload(head, args.steps, args.warmup)
    value = total_bytes / (ms_step * 1e-3) / 1e9
    dominant = max(per_kernel, key=lambda k: k["us"])
    all_kernels = list(per_kernel)
    if not args.no_sweep:
        for name in WORKLOADS:
            if name != head:
                all_kernels += measure_workload(name, max(10, args.steps // 2), args.warmup)[0]
    ceiling = streaming_ceiling(20, 5)
    for k in all_kernels:  # the second denominator: an achieved 1:1 streaming copy on this device
        k["frac_copy_probe"] = round(k["GB/s"] / ceiling["copy"], 3)

    cpu = None
    if not args.no_cpu and head == "softmax_f16_16x32x512x512":
        cpu = cpu_baseline_softmax((16, 32, 512, 512))

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
                   "step": "forward + backward, inputs resident in HBM",
                   "algorithmic_bytes_per_step": total_bytes},
        "roofline": {"bound": "hbm", "kernel": dominant["kernel"],
                     "achieved": dominant["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dominant["GB/s"] / HBM_PEAK_GBS, 4),
                     "avg_launch_us": dominant["us"],
                     "traffic": MEASURED_TRAFFIC_BYTES.get((head, dominant["kernel"])),
                     "streaming_kernels_GB/s": ceiling},
        "cpu_baseline": cpu,
        "kernels": all_kernels,
    }
    if cpu:
        out["speedup_vs_cpu"] = round(value / cpu["value"], 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
