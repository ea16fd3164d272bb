"""The allocation-free entry point blkq4_fp16_gemm_noalloc_sm80, through the C ABI, against the entry point it is
a variant of: the same bits as blkq4_fp16_gemm_sm80 where the plan fits its buffer (same plan, same kernels; only
the split kernels' workspace differs: the buffer inside the library's device image instead of an allocated one), on
two calls in a row, the second one smaller; unsplit shapes; and a shape whose fastest plan needs more workspace
than it holds, which it runs with a plan that fits (checked against the oracle: exact on the reference's
construction, test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472, within 1e-2 on Gaussian data)."""

import numpy as np
import pytest
import torch

from gpu_util import max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_gemm import gaussian_problem, grid_activations

pytestmark = pytest.mark.gpu


def _both(capi, device, bs, zp, m, n, k, seed):
    a, w = gaussian_problem(seed, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, zp)
    a_dev = to_dev(a, device)
    want = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, want)
    got = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, got, noalloc=True)
    torch.cuda.synchronize()
    assert not torch.isnan(want).any()
    return got, want


def test_noalloc_entry_point_gives_the_allocating_entry_points_bits(capi, device):
    # two calls in a row, both with split tiles, the second on a smaller problem (fewer and smaller partial tiles:
    # what the first left behind in the shared buffer must not show)
    first, second = (64, True, 200, 5120, 8192), (64, False, 100, 5120, 5120)
    for bs, zp, m, n, k in (first, second):
        assert " parts" in capi.gemm_plan(bs, True, m, n, k)[2]
    for i, (bs, zp, m, n, k) in enumerate((first, second, first)):
        got, want = _both(capi, device, bs, zp, m, n, k, seed=40 + i)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, n, k)
    # shapes that need no workspace: the streaming kernel, an unsplit tile kernel
    for bs, zp, m, n, k in ((32, True, 4, 1024, 512), (64, True, 300, 1024, 256)):
        got, want = _both(capi, device, bs, zp, m, n, k, seed=50 + m)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, n, k)


def test_noalloc_entry_point_allocates_nothing_and_takes_what_its_buffer_cannot_hold(oracle, capi, device):
    capi.noalloc_init()   # set-up on this device (what a caller does before recording a graph)
    bs, m, n, k = 64, 200, 5120, 8192
    a, w = gaussian_problem(77, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True)
    a_dev = to_dev(a, device)
    out = torch.empty(m, n, dtype=torch.float16, device=device)
    # a stream the library has never seen: blkq4_fp16_gemm_sm80 would allocate its 32 MiB workspace for it
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        torch.zeros(16, device=device).add_(1)   # whatever the tensor library sets up for a new stream happens here
    torch.cuda.synchronize()
    in_use_before = capi.workspace_info(side)[1]
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(side):
        for _ in range(3):
            capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out, noalloc=True)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_before - free_after < (8 << 20), f"device memory went down by {free_before - free_after} bytes"
    assert capi.workspace_info(side)[:2] == (0, in_use_before)   # and the library handed out no buffer for it
    del q_w, q_s, q_zp, a_dev, out

    # 336 tiles of 128 x 256, the last 80 in 3 parts: 30 MiB of partial tiles, more than the 16 MiB it holds.  The
    # allocation-free entry point plans for what it holds and runs the shape all the same.
    bs, m, n, k = 64, 300, 28672, 8192
    assert "workspace 31473664 bytes" in capi.gemm_plan(bs, True, m, n, k)[2]
    kat = oracle.kat_generate(bs, True, k, n, True)
    a = grid_activations(np.random.default_rng(5), m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], True)
    ref = oracle.gemm(a, kat["weights"])
    a_dev = to_dev(a, device)
    for call in range(2):
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
        capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out, noalloc=True)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16)), f"call {call}"
    a, w = gaussian_problem(78, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True)
    canon, s_, z_ = oracle.quantize(bs, True, w, True)
    b = oracle.dequantize(bs, True, canon, s_, z_)
    rows = np.unique(np.linspace(0, m - 1, 16).astype(np.int64))
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, to_dev(a, device), q_w, q_s, q_zp, out, noalloc=True)
    torch.cuda.synchronize()
    got = to_np(out)
    assert not np.isnan(got).any()
    assert max_rel_err(got[rows], oracle.gemm(np.ascontiguousarray(a[rows]), b)) <= 1e-2
