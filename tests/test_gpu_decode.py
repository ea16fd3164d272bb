"""The decode kernel (gemmlib_amd/csrc/blkq4_decode.hip: 1 to 16 rows, blocks along K, all of K requested at once),
through blkq4_fp16_gemm_sm80 / blkq4_bf16_gemm_sm80, against the oracle: the reference's exact construction bit
for bit (test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472) for every block size, with and without zero-points,
every number of slices per wave from 1 to 8, slice counts that do not divide among the waves (the last slot of
some waves stays empty), every wave count, N that is a multiple of 32 and nothing more; Gaussian data within
1e-2; the bias in the epilogue; the same bits on every call."""

import numpy as np
import pytest
import torch

from bf16_util import bf16_kat, grid_activations_bf16
from gpu_util import max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_bf16 import dev_to_bits, gaussian_bits, gemm_bf16, quantize_bf16
from test_gpu_gemm import gaussian_problem, grid_activations

pytestmark = pytest.mark.gpu

# (bs, zero-points, m, n, k): k / 128 slices over 4, 8 or 16 waves
EXACT_CASES = [
    (64, False, 1, 4096, 4096),    # 4 waves x 8
    (64, True, 1, 4128, 4096),     # 8 waves x 4, 258 workgroups
    (32, True, 2, 1024, 128),      # one slice: three of four waves have none
    (16, True, 3, 160, 256), (64, False, 4, 64, 384), (32, False, 1, 96, 640), (16, False, 2, 1056, 1024),
    (64, True, 1, 2048, 1152),     # 9 slices over 8 waves: depth 2, seven waves with an empty slot
    (32, True, 4, 544, 2048), (16, True, 1, 288, 2176), (64, False, 3, 320, 3072), (32, True, 1, 4096, 3200),
    (64, True, 2, 1024, 5120), (16, False, 1, 512, 6144), (32, False, 4, 2080, 7168), (64, True, 1, 4096, 8192),
    (64, False, 1, 1024, 8320),    # 65 slices: 16 waves x 5, one full
    (32, True, 3, 704, 11008), (16, True, 1, 256, 12288), (64, False, 2, 128, 14336), (64, True, 4, 32, 16384),
    (32, False, 1, 128256, 512),   # many workgroups
    (64, False, 1, 256, 28672), (32, True, 4, 128, 18432), (16, True, 2, 64, 17408),   # sixteen waves x 14, 9, 9 (uneven)
    # five to sixteen rows: rows staged slot by slot, 1 to 3 (sixteen rows: 4) column tiles per workgroup
    (32, True, 16, 11008, 4096),   # 3 tiles per workgroup, 230 workgroups, the last one with a tile missing
    (64, False, 8, 4096, 8192), (16, True, 5, 1056, 1152), (32, False, 9, 704, 512), (64, True, 16, 4128, 4096),
    (16, True, 12, 2080, 2048), (64, True, 7, 32, 1024), (32, True, 16, 128, 128), (16, False, 6, 8192, 6144),
    (64, False, 13, 8192, 3200), (32, True, 8, 28672, 1024),
    # sixteen rows, 4 tiles per workgroup: 224 workgroups; 193 with a tile missing in the last; one and two slices per wave
    (64, True, 16, 14336, 4096), (32, False, 9, 12320, 4096), (16, True, 12, 13312, 1024), (64, True, 10, 16384, 2176),
    # eight rows, five slices per wave: one workgroup per compute unit, two rounds of them
    (64, True, 8, 13824, 5120), (32, False, 6, 15360, 5120),
    # up to four rows, 64 slices, 449 to 512 tiles: sixteen waves with four slices each, two workgroups per compute unit
    (64, True, 2, 8192, 8192), (32, False, 1, 7680, 8192), (32, True, 4, 8192, 7680),
]


# blocks along N (up to four rows): 4 and 8 waves, 1 to 8 slices each, waves with an empty slot or none at all
ROW_CASES = [
    (64, False, 1, 4096, 4096), (64, True, 1, 1024, 1024), (32, True, 2, 96, 128), (16, True, 3, 160, 256),
    (32, False, 4, 2080, 384), (64, True, 1, 4160, 2048), (16, False, 1, 704, 3200), (32, True, 4, 1056, 5120),
    (64, False, 2, 1024, 8192), (16, True, 1, 32000, 1152), (64, True, 3, 128, 640), (32, True, 1, 14336, 4096),
    (64, True, 4, 4096, 4096), (32, False, 2, 2048, 4096),   # two to four rows, 32 slices: eight waves with four each
]


def _run(capi, device, bs, a, q_w, q_s, q_zp, n, col=True, **kw):
    m, k = a.shape
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, col, m, n, k, to_dev(a, device), q_w, q_s, q_zp, out, **kw)
    torch.cuda.synchronize()
    return to_np(out)


@pytest.mark.parametrize("bs,has_offsets,m,n,k", ROW_CASES)
def test_blocks_along_n_exact_on_reference_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    """the reference's row-wise construction (test/blkq4_fp16_gemm_sm80_test.cu:480-499), fp16 and bf16"""
    assert capi.gemm_plan(bs, False, m, n, k, has_offsets)[2].startswith("decode (blocks along N):")
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = oracle.kat_generate(bs, False, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets, column_wise=False)
    ref = oracle.gemm(a, kat["weights"])
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n, col=False)
    if not np.array_equal(got.view(np.uint16), ref.view(np.uint16)):
        bad = np.argwhere(got.view(np.uint16) != ref.view(np.uint16))
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}")
    if n <= 8192:
        katb = bf16_kat(oracle, bs, k, n, has_offsets, seed=m + n + k, column_wise=False)
        ab = grid_activations_bf16(oracle, rng, m, k)
        q_w, q_s, q_zp = quantize_bf16(capi, device, bs, katb["weights"], has_offsets, col=False)
        assert np.array_equal(gemm_bf16(capi, device, bs, ab, q_w, q_s, q_zp, n, col=False), oracle.gemm(ab, katb["weights"], bf16=True))


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [(64, False, 1, 4096, 4096), (32, True, 4, 2816, 1152), (16, True, 2, 2048, 8192)])
def test_blocks_along_n_gaussian_and_bias(oracle, capi, device, bs, has_offsets, m, n, k):
    a, w = gaussian_problem(9 + m + n + k, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets, column_wise=False)
    canon, s, z = oracle.quantize(bs, False, w, has_offsets)
    ref = oracle.gemm(a, oracle.dequantize(bs, False, canon, s, z))
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n, col=False)
    assert max_rel_err(got, ref) <= 1e-2
    again = _run(capi, device, bs, a, q_w, q_s, q_zp, n, col=False)
    assert np.array_equal(again.view(np.uint16), got.view(np.uint16))
    g = torch.Generator(device="cpu").manual_seed(n)
    bias = (torch.randn(n, generator=g) * 0.5).to(torch.float16).to(device)
    plain = torch.from_numpy(got.view(np.int16)).to(device).view(torch.float16)
    fused = _run(capi, device, bs, a, q_w, q_s, q_zp, n, col=False, bias=bias)
    plain += bias
    assert np.array_equal(fused.view(np.uint16), to_np(plain).view(np.uint16))


@pytest.mark.parametrize("bs,has_offsets,m,n,k", EXACT_CASES)
def test_exact_on_reference_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    assert capi.gemm_plan(bs, True, m, n, k, has_offsets)[2].startswith("decode:")
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = oracle.kat_generate(bs, True, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets)
    ref = oracle.gemm(a, kat["weights"])
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n)
    if not np.array_equal(got.view(np.uint16), ref.view(np.uint16)):
        bad = np.argwhere(got.view(np.uint16) != ref.view(np.uint16))
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}")


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [c for i, c in enumerate(EXACT_CASES) if i % 2 == 0 and c[3] <= 8192])
def test_exact_on_known_answer_construction_in_bf16(oracle, capi, device, bs, has_offsets, m, n, k):
    assert capi.gemm_plan(bs, True, m, n, k, has_offsets, bf16=True)[2].startswith("decode:")
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = bf16_kat(oracle, bs, k, n, has_offsets, seed=m + n + k)
    a = grid_activations_bf16(oracle, rng, m, k)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, kat["weights"], has_offsets)
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n)
    ref = oracle.gemm(a, kat["weights"], bf16=True)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [
    (64, False, 1, 4096, 4096), (32, True, 4, 11008, 4096), (16, True, 2, 2048, 8192), (64, True, 1, 4096, 11008),
    (32, False, 3, 14336, 1152), (64, False, 1, 128256, 4096), (32, True, 16, 11008, 4096), (16, True, 8, 4096, 8192),
    (64, True, 11, 5120, 2176), (32, True, 16, 14336, 4096), (16, False, 9, 12320, 3072),
])
def test_gaussian_within_tolerance_same_bits_every_call(oracle, capi, device, bs, has_offsets, m, n, k):
    a, w = gaussian_problem(5 + m + n + k, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets)
    canon, s, z = oracle.quantize(bs, True, w, has_offsets)
    ref = oracle.gemm(a, oracle.dequantize(bs, True, canon, s, z))
    got = _run(capi, device, bs, a, q_w, q_s, q_zp, n)
    assert max_rel_err(got, ref) <= 1e-2
    for _ in range(3):
        again = _run(capi, device, bs, a, q_w, q_s, q_zp, n)
        assert np.array_equal(again.view(np.uint16), got.view(np.uint16))
    if m <= 4 and k * (4 if m > 2 else m) * 2 <= 150 * 1024:
        other = _run(capi, device, bs, a, q_w, q_s, q_zp, n, valu=True)   # the GEMV without MFMA: same weights,
        assert max_rel_err(got, other) <= 2e-3                           # fp32 sums in another order


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [(64, True, 1, 4096, 4096), (16, True, 4, 2080, 1152), (32, True, 16, 11008, 4096),
                                                  (64, True, 16, 14336, 4096)])
def test_gaussian_in_bf16(oracle, capi, device, bs, has_offsets, m, n, k):
    a, w = gaussian_bits(oracle, 77 + m + n + k, m, n, k)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, w, has_offsets)
    canon, s, z = oracle.quantize(bs, True, w, has_offsets, bf16=True)
    ref = oracle.gemm(a, oracle.dequantize(bs, True, canon, s, z, bf16=True), bf16=True)
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n)
    assert max_rel_err(oracle.bf16_to_f32(got), oracle.bf16_to_f32(ref)) <= 1e-2


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [(64, False, 1, 4096, 4096), (32, True, 3, 1056, 1152), (16, True, 4, 2048, 8192), (32, True, 16, 11008, 4096),
                                                  (64, False, 13, 14336, 4096)])
def test_bias_in_the_epilogue_equals_a_separate_add(oracle, capi, device, bs, has_offsets, m, n, k):
    """as the reference module adds it (python/ms_blkq4linear.py:26-27): to the rounded output, in the tensor
    library's way of adding two 16-bit tensors"""
    a, w = gaussian_problem(m + n + k, m, n, k)
    g = torch.Generator(device="cpu").manual_seed(n)
    bias = (torch.randn(n, generator=g) * 0.5).to(torch.float16).to(device)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets)
    plain = torch.from_numpy(_run(capi, device, bs, a, q_w, q_s, q_zp, n).view(np.int16)).to(device).view(torch.float16)
    fused = _run(capi, device, bs, a, q_w, q_s, q_zp, n, bias=bias)
    plain += bias
    assert np.array_equal(fused.view(np.uint16), to_np(plain).view(np.uint16))
    ab, wb = gaussian_bits(oracle, m + n + k, m, n, k)
    bias_b = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16).to(device)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, wb, has_offsets)
    plain = torch.from_numpy(gemm_bf16(capi, device, bs, ab, q_w, q_s, q_zp, n).view(np.int16)).to(device).view(torch.bfloat16)
    fused = gemm_bf16(capi, device, bs, ab, q_w, q_s, q_zp, n, bias=bias_b)
    plain += bias_b
    assert np.array_equal(fused, dev_to_bits(plain))
