"""HIP graph capture of the library's calls: replays must give the eager results, also when a kernel's very
first launch in the process happens under capture (the streaming kernel raises its dynamic-LDS limit on
first use) and when inputs change between replays."""

import subprocess
import sys
import textwrap

import numpy as np
import pytest
import torch

from gpu_util import to_np

pytestmark = pytest.mark.gpu

# (block_size, column_wise, has_offsets, m, n, k, bf16): tile kernel, streaming kernel (whole rows in LDS, rows per
# slot, row groups), row-wise streaming and row-wise tile kernel; then the bf16 entry points on both kernels
SHAPES = [
    (64, True, True, 300, 512, 256, False), (32, True, False, 1, 256, 512, False), (16, True, True, 16, 64, 8256, False),
    (64, True, True, 96, 256, 512, False), (32, False, True, 8, 128, 256, False), (64, False, False, 500, 256, 128, False),
    (32, True, True, 4, 256, 512, True), (64, True, False, 16, 64, 8256, True), (64, True, True, 300, 512, 256, True),
    (32, False, True, 8, 128, 256, True),
]


def _problem(capi, device, bs, col, zp, m, n, k, bf, seed):
    dtype = torch.bfloat16 if bf else torch.float16
    g = torch.Generator(device="cpu").manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).to(dtype).to(device)
    a = torch.randn(m, k, generator=g).to(dtype).to(device)
    w_elems, meta_elems = capi.quant_size(bs, col, k, n)
    q_w = torch.empty(w_elems, dtype=torch.uint8, device=device)
    q_s = torch.empty(meta_elems, dtype=dtype, device=device)
    q_z = torch.empty(meta_elems, dtype=torch.uint8, device=device) if zp else None
    out = torch.zeros(m, n, dtype=dtype, device=device)
    return w, a, q_w, q_s, q_z, out


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _capture_and_replay(capi, device, warm):
    problems = [_problem(capi, device, *s, seed=50 + i) for i, s in enumerate(SHAPES)]

    def enqueue():
        for (bs, col, zp, m, n, k, bf), (w, a, q_w, q_s, q_z, out) in zip(SHAPES, problems):
            capi.quant(bs, col, w, q_w, q_s, q_z, bf16=bf)
            capi.gemm(bs, col, m, n, k, a, q_w, q_s, q_z, out, bf16=bf)

    if warm:
        enqueue()
        torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            enqueue()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for replay in range(3):
        # new inputs, eager reference, poison the outputs, replay, compare
        for (w, a, q_w, q_s, q_z, out) in problems:
            a.mul_(-0.5 - replay)
            w.add_(0.001 * (replay + 1))
        enqueue()
        torch.cuda.synchronize()
        want = [_bits(p[5]).copy() for p in problems]
        want_w = [to_np(p[2]).copy() for p in problems]
        for p in problems:
            p[5].fill_(float("nan"))
            p[2].fill_(0xA5)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for s, p, c, qw in zip(SHAPES, problems, want, want_w):
            assert np.array_equal(to_np(p[2]), qw), f"replay {replay}: packed weights differ for {s}"
            assert np.array_equal(_bits(p[5]), c), f"replay {replay}: output differs for {s}"


def test_replays_match_eager(capi, device):
    _capture_and_replay(capi, device, warm=True)


def test_first_launch_under_capture():
    """a fresh process whose first calls into the library are recorded, not executed"""
    code = textwrap.dedent("""
        import sys
        sys.path[:0] = [%r, %r]
        import torch
        from gemmlib_amd import capi
        import test_gpu_graph as t
        capi.load()
        t._capture_and_replay(capi, torch.device("cuda:0"), warm=False)
        print("graph ok")
    """) % (str(__import__("pathlib").Path(__file__).resolve().parent.parent), str(__import__("pathlib").Path(__file__).resolve().parent))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "graph ok" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]
