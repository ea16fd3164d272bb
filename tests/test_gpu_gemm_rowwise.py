"""GPU parity of the GEMM with quantization blocks along N (column_wise_blocking = false), through
the C ABI, against the oracle's dequantize-then-GEMM.

Same two bars as for blocks along K: bit-exact on the reference's own construction (its row-wise
cases, test/blkq4_fp16_gemm_sm80_test.cu:480-499,508-512), max relative error <= 1e-2 on seeded
Gaussian data.
"""

import numpy as np
import pytest
import torch

from gpu_util import gemm_on_gpu, max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_gemm import gaussian_problem, grid_activations

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-2

# (block_size, has_offsets, m, n, k): the reference's row-wise list ...
REFERENCE_CASES = [
    (32, False, 32, 32, 64), (32, True, 32, 32, 64),
    (32, False, 32, 96, 64), (32, True, 32, 96, 64),
    (32, False, 32, 96, 192), (32, True, 32, 96, 192),
    (32, False, 256, 672, 576), (32, True, 256, 672, 576),
    (32, False, 512, 2048 + 32, 960),
    (16, False, 256, 672, 576), (16, True, 256, 672, 576),
    (64, False, 256, 1024, 576), (64, True, 256, 1024, 576),
    (16, False, 16, 704, 576), (16, True, 16, 704, 576),
    (64, False, 16, 1024, 576), (64, True, 16, 1024, 576),
]
# ... and M = 1, ragged M, N that is not a multiple of the 128-column workgroup tile
EDGE_CASES = [
    (64, False, 1, 1024, 576), (32, True, 1, 96, 64), (16, True, 2, 160, 128), (32, True, 3, 672, 576),
    (64, True, 7, 1088, 192), (16, False, 15, 704, 576), (32, True, 17, 96, 192), (64, True, 33, 320, 320),
    (16, True, 65, 544, 256), (32, False, 100, 800, 448), (64, True, 129, 1088, 576), (32, True, 300, 256, 64),
]


# the tile kernel's four shapes (64 x 128, 128 x 128, 128 x 256 and 256 x 256 tiles) with every block size, N that ends
# inside a tile, and row counts just past what the streaming kernel takes
TILE_CASES = [
    (16, True, 400, 672, 576), (32, True, 1000, 4128, 128), (64, False, 1100, 4160, 192), (64, True, 640, 4160, 192),
    (16, True, 4096, 4096, 128), (32, False, 4000, 4128, 64), (64, True, 4096, 4096, 192), (16, False, 4090, 4128, 64),
    (32, True, 160, 96, 8256), (16, False, 130, 2080, 128), (32, True, 400, 2112, 128), (64, False, 300, 4160, 192),
    # one whole round of tiles, dealt to the XCDs in blocks
    (64, True, 2048, 4096, 192), (32, False, 1024, 4096, 128), (16, True, 512, 4096, 128),
]


# very wide N in the streaming kernel: waves with a column tile of their own and all of K, and workgroups that
# walk over several column groups
VERY_WIDE_CASES = [
    (64, False, 1, 14336, 4096), (32, True, 2, 16384, 2112), (16, True, 8, 28672, 1088), (64, True, 16, 16384, 8256),
    (32, True, 16, 14336, 960), (64, False, 5, 32000, 320),
]


@pytest.mark.parametrize("bs,has_offsets,m,n,k", REFERENCE_CASES + EDGE_CASES + TILE_CASES + VERY_WIDE_CASES)
def test_exact_on_reference_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = oracle.kat_generate(bs, False, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets, column_wise=False)
    assert np.array_equal(to_np(q_w), oracle.native_from_canonical(kat["canon_w"]))
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=False)
    ref = oracle.gemm(a, kat["weights"])
    if not np.array_equal(got.view(np.uint16), ref.view(np.uint16)):
        bad = np.argwhere(got.view(np.uint16) != ref.view(np.uint16))
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}: "
                             f"got {got[tuple(bad[0])]} want {ref[tuple(bad[0])]}")


@pytest.mark.parametrize("bs,has_offsets,m,n,k,seed", [
    (32, True, 64, 1024, 1024, 2235), (64, False, 1, 4096, 4096, 2236), (16, True, 16, 2816, 1024, 2237),
    (64, True, 200, 1152, 512, 2238), (16, False, 96, 352, 512, 2239), (32, False, 5, 352, 512, 2240),
])
def test_gaussian(oracle, capi, device, bs, has_offsets, m, n, k, seed):
    a, w = gaussian_problem(seed, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets, column_wise=False)
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=False)
    assert not np.isnan(got).any()
    canon, s, z = oracle.quantize(bs, False, w, has_offsets)
    ref = oracle.gemm(a, oracle.dequantize(bs, False, canon, s, z))
    err = max_rel_err(got, ref)
    print(f"row-wise m={m} n={n} k={k} bs={bs} zp={has_offsets}: max rel err {err:.3e}")
    assert err <= TOLERANCE


@pytest.mark.parametrize("m", [1, 4, 11, 16, 17, 31, 64, 96, 127, 128, 129, 200])
@pytest.mark.parametrize("bs,has_offsets", [(16, False), (32, True), (64, False)])
def test_every_m_band(oracle, capi, device, m, bs, has_offsets):
    """short K: most k slices of the streaming kernel's ring lie past the end (and are multiplied by zero
    scales), which is where a missing wait shows as garbage."""
    test_gaussian(oracle, capi, device, bs, has_offsets, m, 384, 512, seed=3000 + m + bs)


def test_prefill_shape_sampled_rows(oracle, capi, device):
    """the prefill shape with blocks along N; the oracle evaluates a sample of output rows."""
    m, n, k, bs = 2048, 4096, 4096, 64
    a, w = gaussian_problem(2241, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True, column_wise=False)
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=False)
    canon, s, z = oracle.quantize(bs, False, w, True)
    b = oracle.dequantize(bs, False, canon, s, z)
    rows = np.unique(np.concatenate([[0, m - 1], np.random.default_rng(1).integers(0, m, 64)]))
    assert max_rel_err(got[rows], oracle.gemm(np.ascontiguousarray(a[rows]), b)) <= TOLERANCE


def test_rejects_misaligned_scales(capi, device):
    k, n = 64, 64
    w = torch.zeros(k * n // 2, dtype=torch.uint8, device=device)
    s = torch.zeros(k * n // 32 + 8, dtype=torch.float16, device=device)
    a = torch.zeros((4, k), dtype=torch.float16, device=device)
    out = torch.zeros((4, n), dtype=torch.float16, device=device)
    with pytest.raises(capi.Blkq4Error, match="Misaligned Operand"):
        capi.gemm(32, False, 4, n, k, a, w, s[1:1 + k * n // 32], None, out)
