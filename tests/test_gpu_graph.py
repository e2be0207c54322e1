"""The entry points allocate nothing, clear nothing with memset and never
synchronise, so a caller may capture them into a HIP graph. Replays are
separated by eager work and synchronisations and each one is checked against
the eager result on fresh inputs."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _step(K, t):
    N, C = t["x"].shape
    K.layer_norm(N, C, 1e-5, t["x"], t["g"], t["b"], t["mu"], t["rsig"], t["y"])
    K.group_norm_grad(N, 1, C, 1, "NHWC", t["x"], t["mu"], t["rsig"], t["g"], t["dy"], t["params"],
                      t["params"], t["dg"], t["db"], t["dx"])
    K.softmax(N, 1, C, t["y"], t["p"])
    K.softmax_grad(N, 1, C, t["dy"], t["p"], t["dp"])
    K.batch_norm_training_forward(N, C, 1, "NCHW", 0.9, 1e-5, t["x32"], t["g"], t["b"], t["rm"],
                                  t["rv"], t["bmu"], t["brsig"], t["bparams"], t["by"])
    # the same tensor as [8, 64, N*C/512]: the single-read path, several slices per channel
    n, c = 8, 64
    s = N * C // (n * c)
    K.batch_norm_training_forward(n, c, s, "NCHW", 0.9, 1e-5, t["x32"], t["g64"], t["b64"], t["rm64"],
                                  t["rv64"], t["cmu"], t["crsig"], t["cparams"], t["cy"])
    K.batch_norm_training_backward(n, c, s, float(n * s), "NCHW", t["x32"], t["cmu"], t["crsig"],
                                   t["g64"], t["cy"], t["cwg"], t["cwg"], t["cdx"])
    # the entry point for callers that cannot allocate: the library's static scratch
    K.batch_norm_training_forward_noalloc(n, c, s, "NCHW", 0.9, 1e-5, t["x32"], t["g64"], t["b64"],
                                          t["rm64n"], t["rv64n"], t["nmu"], t["nrsig"], t["nparams"],
                                          t["ny"])


def _tensors(N, C):
    import torch
    dev = "cuda"
    t = {k: torch.empty((N, C), dtype=torch.bfloat16, device=dev) for k in ("x", "dy", "y", "p", "dp", "dx")}
    t["x32"] = torch.empty((N, C), device=dev)
    t["by"] = torch.empty((N, C), device=dev)
    for k in ("g", "b", "dg", "db", "rm", "rv", "bmu", "brsig"):
        t[k] = torch.zeros(C, device=dev)
    t["g"].fill_(1.0)
    t["rv"].fill_(1.0)
    t["bparams"] = torch.empty(2 * C, device=dev)
    for k in ("cy", "cdx", "ny"):
        t[k] = torch.empty((N, C), device=dev)
    for k in ("g64", "rv64", "rv64n"):
        t[k] = torch.ones(64, device=dev)
    for k in ("b64", "rm64", "cmu", "crsig", "rm64n", "nmu", "nrsig"):
        t[k] = torch.zeros(64, device=dev)
    t["cparams"], t["cwg"] = torch.empty(128, device=dev), torch.empty(128, device=dev)
    t["nparams"] = torch.empty(128, device=dev)
    t["mu"], t["rsig"] = torch.empty(N, device=dev), torch.empty(N, device=dev)
    t["params"] = torch.empty(2 * N, device=dev)
    return t


def test_entry_points_replay_from_a_captured_graph():
    import torch
    from dragon_amd import kernels as K
    N, C = 512, 4096
    t = _tensors(N, C)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)

    def refill():
        t["x"].copy_(torch.randn((N, C), device="cuda", generator=gen))
        t["dy"].copy_(torch.randn((N, C), device="cuda", generator=gen))
        t["x32"].copy_(torch.randn((N, C), device="cuda", generator=gen))

    refill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # warm-up on the capture stream: scratch, cached launch plans
        _step(K, t)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _step(K, t)
    outs = ("y", "dx", "dg", "db", "p", "dp", "by", "bmu", "brsig", "cy", "cmu", "crsig", "cdx", "cwg",
            "ny", "nmu", "nrsig", "nparams")
    for _ in range(3):
        refill()
        rm0, rv0 = t["rm"].clone(), t["rv"].clone()
        rm1, rv1 = t["rm64"].clone(), t["rv64"].clone()
        rm2, rv2 = t["rm64n"].clone(), t["rv64n"].clone()
        graph.replay()
        torch.cuda.synchronize()
        got = {k: t[k].float().cpu().numpy().copy() for k in outs}
        got_rm = t["rm"].cpu().numpy().copy()
        got_rmn = t["rm64n"].cpu().numpy().copy()
        # the same step eagerly from the same inputs and running statistics
        t["rm"].copy_(rm0)
        t["rv"].copy_(rv0)
        t["rm64"].copy_(rm1)
        t["rv64"].copy_(rv1)
        t["rm64n"].copy_(rm2)
        t["rv64n"].copy_(rv2)
        for k in outs:
            t[k].zero_()
        _step(K, t)
        torch.cuda.synchronize()
        for k in outs:
            assert np.array_equal(got[k], t[k].float().cpu().numpy()), k
        assert np.array_equal(got_rm, t["rm"].cpu().numpy())
        assert np.array_equal(got_rmn, t["rm64n"].cpu().numpy())
        # same kernels on caller scratch and on the static scratch: same bits
        assert np.array_equal(got["ny"], got["cy"]) and np.array_equal(got["nmu"], got["cmu"])
