"""The GEMV without matrix instructions (blkq4_fp16_gemv_valu_sm80), through the C ABI, against the oracle: the
reference's exact construction bit for bit (test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472) for 1 to 4 rows,
every block size, K that ends inside a 128-deep slice, and Gaussian data within 1e-2 -- and against the entry
point it is an alternative to (which runs it for no shape by itself: the decode kernel measured faster on all)."""

import numpy as np
import pytest
import torch

from gpu_util import max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_gemm import grid_activations, gaussian_problem

pytestmark = pytest.mark.gpu


def _run(capi, device, bs, a, q_w, q_s, q_zp, n, **kw):
    m, k = a.shape
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, to_dev(a, device), q_w, q_s, q_zp, out, **kw)
    torch.cuda.synchronize()
    return to_np(out)


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [
    (64, False, 1, 1024, 576), (32, True, 1, 96, 64), (16, True, 2, 160, 128), (32, True, 3, 672, 576),
    (64, True, 4, 1024, 192), (16, False, 1, 704, 4096), (32, True, 4, 4128, 4160), (64, False, 2, 64, 12288),
    (64, True, 1, 32, 16384), (16, True, 3, 14336, 1088), (64, False, 1, 4096, 4096), (32, True, 4, 256, 8192),
])
def test_exact_on_reference_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = oracle.kat_generate(bs, True, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets)
    ref = oracle.gemm(a, kat["weights"])
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n, valu=True)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [(64, False, 1, 4096, 4096), (32, True, 4, 11008, 4096), (16, True, 2, 2048, 8192)])
def test_gaussian_within_tolerance_and_close_to_the_mfma_form(oracle, capi, device, bs, has_offsets, m, n, k):
    a, w = gaussian_problem(5 + m + n + k, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets)
    canon, s, z = oracle.quantize(bs, True, w, has_offsets)
    ref = oracle.gemm(a, oracle.dequantize(bs, True, canon, s, z))
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n, valu=True)
    assert max_rel_err(got, ref) <= 1e-2
    other = _run(capi, device, bs, a, q_w, q_s, q_zp, n)
    assert max_rel_err(got, other) <= 2e-3   # same weights, fp32 sums in another order
    again = _run(capi, device, bs, a, q_w, q_s, q_zp, n, valu=True)
    assert np.array_equal(again.view(np.uint16), got.view(np.uint16))


def test_rejects_other_shapes(capi):
    from gemmlib_amd.capi import RawBuffer
    text = "The GEMV without matrix instructions takes fp16, 1 to 4 rows of at most 150 KiB together and blocks along K"
    for col, m, k in ((True, 5, 64), (False, 1, 64), (True, 4, 32768)):
        n = 64
        with pytest.raises(capi.Blkq4Error) as e:
            capi.gemm(64, col, m, n, k, RawBuffer(0x1000, m * k * 2), RawBuffer(0x1000, k * n // 2),
                      RawBuffer(0x1000, (k // 64 * n if col else k) * 2), None, RawBuffer(0x1000, m * n * 2), stream=0, valu=True)
        assert str(e.value) == text
