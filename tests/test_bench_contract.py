"""bench.py's bookkeeping that needs no GPU: the HBM traffic it reports for the headline kernels
comes from the counter summaries under profiles/ and stays consistent with the algorithmic
bytes; every workload of the sweep is named by a parity test at its full size; a bench line
whose kernel rows beat the streaming probe is reported as broken (the probe is a ceiling)."""

import json
import os
import re

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_roofline_traffic_comes_from_the_committed_counter_summaries():
    traffic = bench.measured_traffic()
    elems = 16 * 32 * 512 * 512
    fwd = traffic[("softmax_f16_16x32x512x512", "softmax")]
    bwd = traffic[("softmax_f16_16x32x512x512", "softmax_grad")]
    # measured HBM bytes per launch: never below what the algorithm must move, and within a
    # few per cent of it (a larger figure would mean re-fetched data)
    assert 2 * elems * 2 <= fwd * 1.001 and fwd <= 2 * elems * 2 * 1.03
    assert 3 * elems * 2 <= bwd * 1.001 and bwd <= 3 * elems * 2 * 1.03
    for (workload, kernel), nbytes in traffic.items():
        assert workload in bench.WORKLOADS and nbytes > 0, (workload, kernel)


def test_every_swept_workload_has_a_full_size_parity_test():
    text = ""
    for name in ("test_gpu_bench_shapes.py", "test_gpu_operators.py"):
        text += open(os.path.join(ROOT, "tests", name)).read()
    text = re.sub(r"\s+", "", text)
    shapes = {
        "softmax_f16_16x32x512x512": "16,32,512,512", "layer_norm_f32_8192x1024_fwd": "8192,1024",
        "batch_norm_f32_64x256x56x56": "64,256,56,56", "group_norm_bf16_32x512x64x64_g32": "32,512,64,64",
        "layer_norm_bf16_8192x12288": "8192,12288", "layer_norm_bf16_65536x1000": "65536,1000",
        "layer_norm_bf16_8192x4096": "8192,4096", "layer_norm_f32_8192x4096": "8192,4096",
        "softmax_f16_8192x4096": "8192,4096", "softmax_f32_8192x4096": "8192,4096",
        "softmax_bf16_605184x197": "605184,197", "layer_norm_bf16_1048576x64": "1048576,64",
        "softmax_f32_2048x128256": "2048,128256",
    }
    for workload, shape in shapes.items():
        assert workload in bench.WORKLOADS
        assert shape in text, "no full-size parity test names the shape of %s" % workload


def _line():
    with open(os.path.join(ROOT, "tests", "golden", "bench_line.json")) as f:
        return json.load(f)


def test_a_well_formed_bench_line_has_no_contract_problems():
    assert bench.contract_problems(_line()) == []


def test_a_kernel_row_above_the_probe_is_a_contract_problem():
    line = _line()
    line["kernels"][1]["frac_stream_probe"] = 1.02
    problems = bench.contract_problems(line)
    assert len(problems) == 1 and "ceiling" in problems[0] and "softmax_grad" in problems[0]


def test_other_contract_problems_are_seen():
    line = _line()
    del line["cpu_baseline"]
    line["roofline"]["frac"] = 0.9
    line["kernels"][0]["frac_hbm_peak"] = 1.2
    text = " ".join(bench.contract_problems(line))
    assert "cpu_baseline" in text and "achieved / peak" in text and "above the HBM peak" in text
