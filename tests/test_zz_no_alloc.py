"""The allocation-free entry point blkq4_fp16_gemm_noalloc_sm80, through the C ABI, against the entry point it is
a variant of: the same bits as blkq4_fp16_gemm_sm80 (same plan, same kernels; only the split kernels' workspace
differs: the buffer inside the library's device image instead of the per-stream buffer), on two calls in a row, the
second one smaller; unsplit shapes; and the rejection of a shape whose plan needs more workspace than it holds."""

import numpy as np
import pytest
import torch

from gpu_util import quantize_on_gpu, to_dev
from test_gpu_gemm import gaussian_problem

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


def test_noalloc_entry_point_allocates_nothing_and_rejects_what_does_not_fit(capi, device):
    bs, m, n, k = 64, 200, 5120, 8192
    a, w = gaussian_problem(77, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True)
    a_dev = to_dev(a, device)
    out = torch.empty(m, n, dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out, noalloc=True)   # first use on this device: set-up
    torch.cuda.synchronize()
    # a stream the library has never seen: blkq4_fp16_gemm_sm80 would allocate its 32 MiB workspace for it
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        torch.zeros(16, device=device).add_(1)   # whatever the tensor library sets up for a new stream happens here
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(side):
        for _ in range(3):
            capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out, noalloc=True)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_before - free_after < (8 << 20), f"device memory went down by {free_before - free_after} bytes"
    # 336 tiles of 128 x 256, the last 80 in 3 parts: 30 MiB of partial tiles, more than the 16 MiB it holds
    m, n, k = 300, 28672, 4096
    assert "workspace 31473664 bytes" in capi.gemm_plan(64, True, m, n, k)[2]
    from gemmlib_amd.capi import RawBuffer
    with pytest.raises(capi.Blkq4Error, match="Workspace of 31473664 bytes needed, the allocation-free entry point holds 16793600"):
        capi.gemm(64, True, m, n, k, RawBuffer(0x100000, m * k * 2), RawBuffer(0x100000, k * n // 2),
                  RawBuffer(0x100000, k // 64 * n * 2), None, RawBuffer(0x100000, m * n * 2), stream=0, noalloc=True)
