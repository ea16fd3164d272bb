"""GPU parity of the GEMM on seeded random shapes, through the C ABI, against the oracle.

The shapes are drawn so that every way the library splits the work is hit with ragged edges: K that ends
inside a 128-deep slice, column tile counts that the column groups do not divide, row counts around the
row-group and kernel switches, very wide N (waves with a column tile of their own, workgroups that walk over
several column groups, column groups dealt singly to the XCDs), 33 to 64 rows whose tiles are split along K, both
blockings, with and without zero-points and bias.  Bar: max relative error
<= 1e-2 on Gaussian data, where the error of an output is measured against max(|ref|, 1e-3 * max|ref|).
"""

import numpy as np
import pytest
import torch

from gpu_util import max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_gemm import gaussian_problem

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-2


def draw_cases():
    rng = np.random.default_rng(20240229)
    cases = []
    for i in range(48):
        bs = int(rng.choice([16, 32, 64]))
        col = bool(rng.integers(0, 2))
        zp = bool(rng.integers(0, 2))
        band = i % 4
        if band == 0:    # few rows, very wide
            m = int(rng.integers(1, 17))
            n = int(rng.integers(14336 // 64, 40000 // 64)) * 64
            k = int(rng.integers(1, 24)) * 64
        elif band == 1:  # few rows, moderately wide, long K
            m = int(rng.integers(1, 17))
            n = int(rng.integers(1, 200)) * 64
            k = int(rng.integers(8, 140)) * 64
        elif band == 2:  # row groups
            m = int(rng.integers(17, 400))
            n = int(rng.integers(1, 150)) * 64
            k = int(rng.integers(1, 40)) * 64
        else:            # tile kernel
            m = int(rng.integers(400, 2500))
            n = int(rng.integers(1, 70)) * 64
            k = int(rng.integers(1, 12)) * 64
        if col and rng.integers(0, 2):
            n += 32  # blocks along K allow any multiple of 32
        cases.append((bs, zp, col, m, n, k, bool(rng.integers(0, 2))))
    for i in range(24):
        bs = int(rng.choice([16, 32, 64]))
        col = True if i % 3 else bool(rng.integers(0, 2))
        zp = bool(rng.integers(0, 2))
        band = i % 3
        if band == 0:    # 33 to 64 rows, few tiles, long K: with blocks along K every 64 x 128 tile in parts
            m = int(rng.integers(33, 65))
            n = int(rng.integers(8, 130)) * 64
            k = int(rng.integers(64, 300)) * 64
        elif band == 1:  # five to eight rows, K just above 4096, wide: two rounds of decode workgroups
            m = int(rng.integers(5, 9))
            n = int(rng.integers(12288 // 32, 21000 // 32)) * 32
            k = int(rng.integers(33, 41)) * 128
        else:            # row groups with four and more tiles per workgroup, column groups that eight does not divide
            m = int(rng.integers(17, 200))
            n = int(rng.integers(60, 400)) * 32
            k = int(rng.integers(8, 100)) * 64
        cases.append((bs, zp, col, m, n, k, bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("bs,has_offsets,col,m,n,k,with_bias", draw_cases())
def test_random_shape(oracle, capi, device, bs, has_offsets, col, m, n, k, with_bias):
    a, w = gaussian_problem(m * 7 + n * 3 + k, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets, column_wise=col)
    a_dev = to_dev(a, device)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, out)
    torch.cuda.synchronize()
    got = to_np(out)
    assert not np.isnan(got).any()
    canon, s, z = oracle.quantize(bs, col, w, has_offsets)
    rows = np.arange(m) if m * n * k <= 3e9 else np.unique(np.concatenate([[0, m - 1], np.arange(0, m, max(1, m // 64))]))
    ref = oracle.gemm(np.ascontiguousarray(a[rows]), oracle.dequantize(bs, col, canon, s, z))
    assert max_rel_err(got[rows], ref) <= TOLERANCE
    if with_bias:
        # the fused bias against the separate add, bit for bit (an error bound against the oracle would measure
        # the cancellation between sum and bias, not the kernel)
        g = torch.Generator(device="cpu").manual_seed(n + k)
        bias = (torch.randn(n, generator=g) * 0.25).to(torch.float16).to(device)
        fused = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
        capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, fused, bias=bias)
        torch.cuda.synchronize()
        out += bias
        assert torch.equal(fused.view(torch.int16), out.view(torch.int16))


@pytest.mark.parametrize("bs,has_offsets,col,m,n,k,with_bias", draw_cases())
def test_random_shape_bf16(oracle, capi, device, bs, has_offsets, col, m, n, k, with_bias):
    """the same shapes through blkq4_bf16_quant_sm80 / blkq4_bf16_gemm_sm80: quantizer bit-exact, GEMM within the
    same bound (a bf16 output's unit in the last place is up to 2^-7 = 0.8e-2 of its value)"""
    from test_gpu_bf16 import bits_to_dev, dev_to_bits, gaussian_bits, quantize_bf16
    a, w = gaussian_bits(oracle, m * 7 + n * 3 + k, m, n, k)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, w, has_offsets, col=col)
    canon, s, z = oracle.quantize(bs, col, w, has_offsets, bf16=True)
    assert np.array_equal(q_w.cpu().numpy(), oracle.native_from_canonical(canon))
    ps, pz = oracle.prepack_meta_sm80(bs, col, k, n, s, z)
    assert np.array_equal(dev_to_bits(q_s), ps.view(np.uint16))
    a_dev = bits_to_dev(a, device)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, out, bf16=True)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    got = oracle.bf16_to_f32(dev_to_bits(out))
    rows = np.arange(m) if m * n * k <= 3e9 else np.unique(np.concatenate([[0, m - 1], np.arange(0, m, max(1, m // 64))]))
    ref = oracle.gemm(np.ascontiguousarray(a[rows]), oracle.dequantize(bs, col, canon, s, z, bf16=True), bf16=True)
    assert max_rel_err(got[rows], oracle.bf16_to_f32(ref)) <= TOLERANCE
    if with_bias:
        g = torch.Generator(device="cpu").manual_seed(n + k)
        bias = (torch.randn(n, generator=g) * 0.25).to(torch.bfloat16).to(device)
        fused = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
        capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, fused, bias=bias, bf16=True)
        torch.cuda.synchronize()
        out += bias
        assert torch.equal(fused.view(torch.int16), out.view(torch.int16))
