"""GPU parity of the GEMM / GEMV path, through the C ABI, against the oracle's
dequantize-then-GEMM (fp32 accumulation, one rounding to fp16).

Two bars:
  * the reference's own construction (test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472): weights from
    the known-answer generator, activations on the 0.25 grid in [-4, 4]; every partial sum is exact in
    fp32, so the output must be BIT-EXACT whatever the summation order;
  * seeded Gaussian data (the benchmark configurations): max relative error <= 1e-2, where the error
    of an output is measured against max(|ref|, 1e-3 * max|ref|).
"""

import numpy as np
import pytest
import torch

from gpu_util import gemm_on_gpu, max_rel_err, quantize_on_gpu, to_dev, to_np

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-2


def grid_activations(rng, m, k):
    """uniform on the 0.25 grid in [-4, 4] (cutlass TensorFillRandomUniform(view, seed, 4, -4, bits=2))."""
    return (rng.integers(-16, 17, (m, k)) / 4.0).astype(np.float16)


def run_kat(oracle, capi, device, bs, has_offsets, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = oracle.kat_generate(bs, True, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets)
    # the quantizer must hand back the generator's data, otherwise the GEMM check below is moot
    assert np.array_equal(to_np(q_w), oracle.native_from_canonical(kat["canon_w"]))
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n)
    ref = oracle.gemm(a, kat["weights"])
    if not np.array_equal(got.view(np.uint16), ref.view(np.uint16)):
        bad = np.argwhere(got.view(np.uint16) != ref.view(np.uint16))
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}: "
                             f"got {got[tuple(bad[0])]} want {ref[tuple(bad[0])]}")


# (block_size, has_offsets, m, n, k): the column-wise cases of the reference's test list
# (test/blkq4_fp16_gemm_sm80_test.cu:501-518) ...
REFERENCE_CASES = [
    (16, False, 256, 672, 576), (16, True, 256, 672, 576),
    (64, False, 256, 1024, 576), (64, True, 256, 1024, 576),
    (16, False, 16, 672, 576), (16, True, 16, 672, 576),
    (64, False, 16, 1024, 576), (64, True, 16, 1024, 576),
]
# ... the shapes it runs row-wise only, here column-wise (:480-493) ...
EXTRA_CASES = [
    (32, False, 32, 32, 64), (32, True, 32, 32, 64),
    (32, False, 32, 96, 64), (32, True, 32, 96, 192),
    (32, True, 256, 672, 576), (32, False, 512, 2048 + 32, 960),
]
# ... and what the reference never tests: M = 1, ragged M, M around the kernel switch at 16
EDGE_CASES = [
    (64, False, 1, 1024, 576), (32, True, 1, 96, 64), (16, True, 2, 160, 128), (32, True, 3, 672, 576),
    (64, True, 7, 1024, 192), (16, False, 15, 704, 576), (32, True, 17, 96, 192), (64, True, 33, 288, 320),
    (16, True, 65, 544, 256), (32, False, 100, 800, 448), (64, True, 129, 1056, 576), (32, True, 300, 256, 64),
]
# wide N at M <= 16, where the kernel gives a workgroup 1, 2 or 3 column tiles depending on how the
# tile count fills the chip (258 tiles: 2; 514: 3 with a ragged last workgroup; 1792: 1)
# shapes with at least 256 tiles of 256 x 256, which take the kernel variant with 256-row waves
LARGE_TILE_CASES = [(64, True, 4096, 4096, 128), (16, True, 4000, 4128, 64), (32, False, 4096, 4096, 192)]
# shapes that 64 x 128 tiles cover in one round of workgroups (and the streaming kernel is not expected to beat)
SMALL_TILE_CASES = [(64, True, 300, 4128, 192), (16, True, 500, 2080, 128), (32, False, 257, 4096, 64)]
# very wide N and rows that the streaming kernel cannot keep in LDS for all of K: up to 16 rows it takes more
# column tiles per workgroup (the rows are fetched once per workgroup and slice), 17 to 64 rows go to the tile
# kernel's 32- and 64-row tiles (128 columns up to one round of them, else 256)
WIDE_TILE32_CASES = [
    (64, True, 16, 28672, 5184), (32, True, 9, 28704, 5248), (16, False, 32, 28672, 2624), (64, False, 20, 28672, 2688),
    (32, True, 24, 36864, 2624), (64, True, 48, 28672, 256), (32, False, 64, 36864, 128),
    # the 128-column tiles of one row tile half-filling the chip (144 and 160 workgroups), where two rounds of streaming
    # workgroups would take longer
    (64, True, 64, 18432, 1024), (32, False, 24, 28672, 1088), (16, True, 48, 20480, 2048), (64, False, 33, 18464, 4096),
]
WIDE_SKINNY_CASES = [
    (16, True, 12, 4128, 128), (32, True, 8, 8224, 128), (64, False, 3, 8224, 192), (32, False, 5, 28672, 64),
]


# long K, where the activation rows no longer fit in LDS as a whole and are staged per k slice, and
# more than 16 rows in the streaming kernel: row groups of 32 rows (two row tiles share one conversion of
# the weights), one, two or four column tiles per workgroup
LONG_K_CASES = [
    (32, True, 16, 64, 8192 + 64), (64, False, 9, 64, 12288), (16, True, 3, 32, 40960 + 128),
    (16, True, 32, 64, 4096), (32, True, 20, 96, 6144), (64, True, 64, 64, 4096), (32, False, 50, 96, 2112),
    (64, True, 31, 4128, 320), (16, False, 64, 4128, 128), (32, True, 32, 8224, 2112), (16, True, 25, 8192 + 64, 4160),
    (64, True, 100, 96, 8256), (16, True, 77, 4128, 192), (32, False, 130, 4128, 128), (64, False, 250, 1056, 320),
]


# very wide N in the streaming kernel: few rows, where every wave streams all of K for a column tile of its own
# (several rounds of its ring, K that ends inside a slice), and more rows, where a workgroup walks over
# several column groups (rows whole in LDS, rows staged per slice, row groups of 32)
VERY_WIDE_CASES = [
    (64, False, 1, 32000, 4096), (32, True, 2, 32032, 4032), (16, True, 4, 32768, 320), (64, True, 1, 32000, 8192),
    (64, False, 1, 14336, 4096), (32, True, 2, 16416, 4160), (32, False, 16, 32032, 256), (16, True, 9, 32000, 448),
    (64, True, 8, 32800, 4096), (32, True, 16, 16416, 8256), (32, True, 96, 5440, 4160), (16, False, 12, 28672, 1088),
    (64, False, 1, 13824, 5120), (32, True, 4, 14336, 4096), (16, True, 3, 22016, 4096), (32, True, 2, 13856, 5184),
]


# row groups of 32 with six and eight column tiles per workgroup (rows whole in LDS and staged per slice), the last
# workgroup of a row group with tiles missing
SIX_AND_EIGHT_TILE_CASES = [
    (64, True, 48, 11008, 1152), (32, False, 64, 11008, 4096), (16, True, 96, 8192, 640), (64, True, 100, 8224, 4096),
    (32, True, 33, 11040, 2176), (64, False, 60, 14336, 4160),
]

# five to sixteen rows on wide layers, rows staged per slice: five, six and seven column tiles per workgroup of four
# or eight waves (as many as give every compute unit the same number of tiles), a last slice of two units only
# (K = 64 mod 128), a last workgroup with tiles missing
FIVE_TO_SEVEN_TILE_CASES = [
    (64, True, 16, 18432, 4096), (32, False, 9, 22016, 2048), (16, True, 16, 28672, 1088), (32, True, 13, 36864, 4160),
    (64, True, 16, 57344, 2048), (32, True, 6, 22016, 8192), (64, False, 5, 20480, 8256), (64, True, 11, 40960, 1088),
    (32, True, 16, 24608, 4096),
    # two to four rows with K >= 8192 take the same shapes
    (64, True, 4, 22016, 8192), (32, False, 2, 28672, 8256), (16, True, 3, 24576, 8192),
    # and a single row once K is longer than 8192
    (64, False, 1, 22016, 11008), (32, True, 1, 28672, 8320),
    # six tiles with four waves: three workgroups per compute unit
    (32, False, 7, 69664, 1088),
]


# 128 x 32 tiles whose four computing waves split the k tile (one round of them covers the problem): a whole number of
# trips through the unrolled loop and not (K = 3008 is 47 k tiles), rows past M in the last tile, every block size
K_SPLIT_WAVES_CASES = [
    (64, True, 256, 4096, 4096), (64, False, 255, 4096, 3008), (32, True, 256, 4096, 2112), (16, True, 200, 4096, 4096),
]


@pytest.mark.parametrize("bs,has_offsets,m,n,k", K_SPLIT_WAVES_CASES)
def test_k_split_waves_cases_run_the_tile_they_are_meant_for(capi, bs, has_offsets, m, n, k):
    for bf16 in (False, True):
        text = capi.gemm_plan(bs, True, m, n, k, has_offsets, bf16)[2]
        assert text.startswith("tile: 128 x 32, 4 + 4 waves (the computing waves split the k tile)"), text


@pytest.mark.parametrize("bs,has_offsets,m,n,k", K_SPLIT_WAVES_CASES[:2])
def test_k_split_waves_on_gaussian_data_and_with_bias(oracle, capi, device, bs, has_offsets, m, n, k):
    got, q_w, q_s, q_zp, a = run_gaussian(oracle, capi, device, bs, has_offsets, m, n, k, seed=3000 + m + k, sample_rows=40)
    # every call the same bits (the four waves' sums are added in wave order), and the bias as a separate add would
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(n)) * 0.5).to(torch.float16)
    fused = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, to_dev(a, device), q_w, q_s, q_zp, fused, bias=bias.to(device))
    torch.cuda.synchronize()
    again = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n)
    assert np.array_equal(again.view(np.uint16), got.view(np.uint16))
    want = (torch.from_numpy(got.view(np.int16).copy()).view(torch.float16) + bias).view(torch.int16).numpy()
    assert np.array_equal(fused.cpu().view(torch.int16).numpy(), want)


@pytest.mark.parametrize("bs,has_offsets,m,n,k", REFERENCE_CASES + EXTRA_CASES + K_SPLIT_WAVES_CASES + EDGE_CASES + WIDE_SKINNY_CASES + LARGE_TILE_CASES + SMALL_TILE_CASES + WIDE_TILE32_CASES + LONG_K_CASES + VERY_WIDE_CASES + SIX_AND_EIGHT_TILE_CASES + FIVE_TO_SEVEN_TILE_CASES)
def test_exact_on_reference_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    run_kat(oracle, capi, device, bs, has_offsets, m, n, k)


@pytest.mark.parametrize("bs,has_offsets,m,n,k", FIVE_TO_SEVEN_TILE_CASES)
def test_five_to_seven_tile_cases_run_the_shapes_they_are_meant_for(capi, bs, has_offsets, m, n, k):
    text = capi.gemm_plan(bs, True, m, n, k, has_offsets)[2]
    assert text.startswith("streaming:") and any(f"{t} column tile(s) x 16 rows" in text for t in (5, 6, 7)) and "rows staged per slice" in text


def gaussian_problem(seed, m, n, k):
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = torch.randn(m, k, generator=g, dtype=torch.float32).to(torch.float16)
    w = (torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    return a.view(torch.int16).numpy().view(np.float16), w.view(torch.int16).numpy().view(np.float16)


def run_gaussian(oracle, capi, device, bs, has_offsets, m, n, k, seed, sample_rows=None):
    a, w = gaussian_problem(seed, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets)
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n)
    assert not np.isnan(got).any()
    canon, s, z = oracle.quantize(bs, True, w, has_offsets)
    b = oracle.dequantize(bs, True, canon, s, z)
    rows = np.arange(m) if sample_rows is None else np.unique(
        np.concatenate([[0, m - 1], np.random.default_rng(seed).integers(0, m, sample_rows)]))
    ref = oracle.gemm(np.ascontiguousarray(a[rows]), b)
    err = max_rel_err(got[rows], ref)
    exact = float(np.mean(got[rows].view(np.uint16) == ref.view(np.uint16)))
    print(f"m={m} n={n} k={k} bs={bs} zp={has_offsets}: max rel err {err:.3e}, bit-identical outputs {exact:.4f}")
    assert err <= TOLERANCE
    return got, q_w, q_s, q_zp, a


def test_config1_cpu_runnable_case(oracle, capi, device):
    run_gaussian(oracle, capi, device, 32, True, 64, 1024, 1024, seed=1235)


def test_config2_decode_gemv(oracle, capi, device):
    run_gaussian(oracle, capi, device, 64, False, 1, 4096, 4096, seed=1236)


def test_config3_skinny(oracle, capi, device):
    run_gaussian(oracle, capi, device, 32, True, 16, 11008, 4096, seed=1237)


def test_config4_prefill(oracle, capi, device):
    run_gaussian(oracle, capi, device, 64, True, 2048, 4096, 4096, seed=1238, sample_rows=96)


def test_config5_large_layer(oracle, capi, device):
    """full shape on the GPU; the oracle evaluates a sample of output rows, and linearity
    (C(2a) = 2 C(a) exactly, scaling by 2 commutes with every rounding) covers the rest."""
    m, n, k, bs = 4096, 28672, 8192, 16
    got, q_w, q_s, q_zp, a = run_gaussian(oracle, capi, device, bs, True, m, n, k, seed=1239, sample_rows=6)
    got2 = gemm_on_gpu(capi, device, bs, (a * np.float16(2)).astype(np.float16), q_w, q_s, q_zp, n)
    # outputs in fp16's subnormal range gain one bit when doubled, so they are compared by distance
    normal = np.abs(got) >= np.float16(2.0 ** -13)
    twice = (got.astype(np.float32) * 2).astype(np.float16)
    assert np.array_equal(twice[normal].view(np.uint16), got2[normal].view(np.uint16))
    assert np.all(np.abs(twice[~normal].astype(np.float32) - got2[~normal].astype(np.float32)) <= 2.0 ** -23)


@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 11, 16, 17, 31, 64, 96, 127, 128, 200])
@pytest.mark.parametrize("bs,has_offsets", [(16, True), (32, False), (64, True)])
def test_every_m_band(oracle, capi, device, m, bs, has_offsets):
    run_gaussian(oracle, capi, device, bs, has_offsets, m, 352, 512, seed=m * 10 + bs)


# whole rounds of tiles dealt to the XCDs in blocks (the plan says so): one round, several rounds with a partly filled
# last one, rows that end inside the last tile row, every tile shape that takes blocks
XCD_BLOCK_CASES = [(64, True, 2048, 11008, 512), (32, True, 512, 4096, 512), (16, True, 1024, 4096, 256),
                   (64, True, 1000, 8192, 512), (64, False, 2048, 4096, 256)]


@pytest.mark.parametrize("bs,has_offsets,m,n,k", XCD_BLOCK_CASES)
def test_tiles_in_blocks_per_xcd_on_gaussian_data(oracle, capi, device, bs, has_offsets, m, n, k):
    assert "tiles per XCD" in capi.gemm_plan(bs, True, m, n, k, has_offsets)[2]
    # every row and column is checked where the oracle takes a second or two, else 40 rows spread over all tile rows
    run_gaussian(oracle, capi, device, bs, has_offsets, m, n, k, seed=m + n + k, sample_rows=None if m * n <= 2 ** 22 else 40)


def test_rows_are_independent(oracle, capi, device):
    """row r of C depends only on row r of A: the M=1 result equals row 0 of the M=16 and M=64 results."""
    a, w = gaussian_problem(77, 64, 512, 1024)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, 32, w, True)
    c64 = gemm_on_gpu(capi, device, 32, a, q_w, q_s, q_zp, 512)
    c16 = gemm_on_gpu(capi, device, 32, a[:16], q_w, q_s, q_zp, 512)
    c1 = gemm_on_gpu(capi, device, 32, a[:1], q_w, q_s, q_zp, 512)
    assert max_rel_err(c16, c64[:16]) <= 2e-3   # different kernels, different summation order
    assert max_rel_err(c1, c16[:1]) <= 2e-3


def test_weights_repacked_from_reference_order(oracle, capi, device):
    """a buffer in the reference's sm80 byte order (as the reference's quantizer would have written
    it) converts with blkq4_fp16_repack_sm80 and gives the same GEMM result."""
    rng = np.random.default_rng(8)
    kat = oracle.kat_generate(32, True, 192, 96, True)
    sm80_w, ps, pz = oracle.quant_sm80(32, True, kat["weights"], True)
    src = to_dev(sm80_w, device)
    dst = torch.empty_like(src)
    capi.repack(False, 192, 96, src, dst)
    a = grid_activations(rng, 32, 192)
    got = gemm_on_gpu(capi, device, 32, a, dst, to_dev(ps, device), to_dev(pz, device), 96)
    assert np.array_equal(got.view(np.uint16), oracle.gemm(a, kat["weights"]).view(np.uint16))


# (block_size, has_offsets, column_wise, m, n, k): every kernel and epilogue that stores outputs: streaming kernel
# with sums across waves (M = 1, 16), with row groups (M = 64), with waves that keep whole sums (wide N), and
# the tile kernel's three shapes
BIAS_CASES = [
    (64, False, True, 1, 4096, 512), (32, True, True, 16, 1056, 576), (16, True, True, 64, 352, 256),
    (64, False, True, 2, 32000, 256), (32, True, False, 3, 16384, 128), (64, True, True, 300, 4128, 192),
    (32, True, True, 1100, 4160, 128), (16, True, True, 4096, 4096, 64), (64, True, False, 1200, 1088, 192),
]


@pytest.mark.parametrize("bs,has_offsets,col,m,n,k", BIAS_CASES)
def test_bias_in_the_epilogue_equals_a_separate_add(oracle, capi, device, bs, has_offsets, col, m, n, k):
    """blkq4_fp16_gemm_bias_sm80 == blkq4_fp16_gemm_sm80 followed by the tensor library's in-place fp16 add
    (what the reference module does, python/ms_blkq4linear.py:26-27), bit for bit."""
    a, w = gaussian_problem(m + n + k, m, n, k)
    g = torch.Generator(device="cpu").manual_seed(n)
    bias = (torch.randn(n, generator=g) * 0.5).to(torch.float16).to(device)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets, column_wise=col)
    a_dev = to_dev(a, device)
    plain = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    fused = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, plain)
    capi.gemm(bs, col, m, n, k, a_dev, q_w, q_s, q_zp, fused, bias=bias)
    torch.cuda.synchronize()
    plain += bias
    assert not torch.isnan(fused).any()
    assert torch.equal(fused.view(torch.int16), plain.view(torch.int16))


def test_non_default_stream(oracle, capi, device):
    a, w = gaussian_problem(5, 8, 256, 256)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, 64, w, True)
    ref = gemm_on_gpu(capi, device, 64, a, q_w, q_s, q_zp, 256)
    s = torch.cuda.Stream()
    a_dev = to_dev(a, device)
    out = torch.zeros((8, 256), dtype=torch.float16, device=device)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        capi.gemm(64, True, 8, 256, 256, a_dev, q_w, q_s, q_zp, out, stream=s)
    s.synchronize()
    assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("m,n,k,plans", [
    (16, 1024, 1024, ["auto", "decode 16 1 8 1", "decode 16 2 8 1", "streaming 4 1 1 8 1 8", "streaming 2 1 1 16 1 16"]),
    (200, 2048, 2048, ["auto", "tile 2 1 1 4 4 1 1", "tile 4 1 1 4 4 1 1", "tile 4 1 1 4 4 1 2", "tile 4 2 1 4 4 1 1",
                       "tile 8 2 1 4 0 1 1", "tile 8 1 1 4 4 1 1", "tile 4 1 1 1 4 4 1", "streaming 2 4 2 8 1 8",
                       "streaming 2 2 2 8 2 8"]),
    # one whole round of 256 tiles plus a partly filled one (8 x 33 and 4 x 65 tiles): the tile order of the whole
    # round in every cut per XCD, alone and with the rest split; 8 row bands do not exist for 4 tile rows
    (512, 4224, 256, ["auto", "tile 2 1 1 4 4 1 1 0", "tile 2 1 1 4 4 1 1 1", "tile 2 1 1 4 4 1 1 2", "tile 2 1 1 4 4 1 1 4",
                      "tile 2 1 1 4 4 1 1 8", "tile 2 1 1 4 4 1 2 2", "tile 4 1 1 4 4 1 1 1", "tile 4 1 1 4 4 1 1 2",
                      "tile 4 1 1 4 4 1 1 4", "tile 4 1 1 4 4 1 2 4"]),
    # 256 x 256 tiles in parts, which no plan of the library's own asks for (the workgroup that adds the parts up is slow
    # with 256 accumulators): 3 x 4 tiles, the last row of them 8 rows high
    (520, 1024, 2048, ["auto", "tile 8 2 1 4 0 1 2", "tile 8 2 1 4 0 1 4", "tile 4 2 1 4 4 1 3"]),
])
def test_every_plan_given_as_text_is_exact_on_reference_construction(oracle, capi, device, m, n, k, plans):
    """blkq4_gemm_with_plan_sm80: whichever kernel is asked for by name, the reference's exact construction
    (test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472) comes out bit for bit."""
    bs, has_offsets = 64, True
    rng = np.random.default_rng(m + n + k)
    kat = oracle.kat_generate(bs, True, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets)
    ref = oracle.gemm(a, kat["weights"])
    a_dev = to_dev(a, device)
    for plan in plans:
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
        capi.gemm_with_plan(plan, bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out)
        torch.cuda.synchronize()
        assert np.array_equal(to_np(out).view(np.uint16), ref.view(np.uint16)), plan
    with pytest.raises(capi.Blkq4Error, match="Kernel execution failed: invalid argument"):
        capi.gemm_with_plan("decode 16 1 8 2", bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out)   # K is not 16 slices
    with pytest.raises(capi.Blkq4Error, match="Kernel execution failed: invalid argument"):
        capi.gemm_with_plan("tile 4 1 1 4 4 1 1 3", bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out)  # no such cut
