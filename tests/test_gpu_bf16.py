"""GPU parity of the bf16 entry points (blkq4_bf16_quant_sm80, blkq4_bf16_gemm_sm80), through the C ABI.

Bars:
  * quantizer, both blockings: bit-exact against the oracle (nibbles in the library's order, scales, zero-points),
    on the bf16-exact known-answer construction and on Gaussian data, ragged and strided sources included;
  * GEMM on the known-answer construction with activations on the 0.25 grid (the reference's own
    exact-equality test, test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472, with the element type changed):
    every partial sum is exact in fp32, so the output is BIT-EXACT whatever the summation order;
  * GEMM on seeded Gaussian data: max relative error <= 1e-2 against the oracle's dequantize-then-GEMM, the
    error of an output measured against max(|ref|, 1e-3 * max|ref|) -- a bf16 output has 8 significant
    bits, so one unit in the last place is up to 2^-7 = 0.8e-2; and <= 2^-8 against the float64 product of
    the same dequantized weights (half a unit plus the fp32 accumulation).
"""

import numpy as np
import pytest
import torch

from bf16_util import bf16_kat, grid_activations_bf16
from gpu_util import max_rel_err

pytestmark = pytest.mark.gpu

TOLERANCE = 1e-2


def bits_to_dev(bits: np.ndarray, device):
    return torch.from_numpy(bits.view(np.int16).copy()).to(device).view(torch.bfloat16)


def dev_to_bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def quantize_bf16(capi, device, bs, weights_bits, has_offsets, w_dev=None, rows=None, columns=None, ld=None, col=True):
    n, k = weights_bits.shape if columns is None else (columns, rows)
    w_elems, meta_elems = capi.quant_size(bs, col, k, n)
    if w_dev is None:
        w_dev = bits_to_dev(weights_bits, device)
    q_w = torch.full((w_elems,), 0xA5, dtype=torch.uint8, device=device)
    q_s = torch.full((meta_elems,), float("nan"), dtype=torch.bfloat16, device=device)
    q_zp = torch.full((meta_elems,), 0xEE, dtype=torch.uint8, device=device) if has_offsets else None
    capi.quant(bs, col, w_dev, q_w, q_s, q_zp, bf16=True, rows=rows, columns=columns, ld=ld)
    torch.cuda.synchronize()
    return q_w, q_s, q_zp


def gemm_bf16(capi, device, bs, a_bits, q_w, q_s, q_zp, n, bias=None, col=True):
    m, k = a_bits.shape
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=device)
    capi.gemm(bs, col, m, n, k, bits_to_dev(a_bits, device), q_w, q_s, q_zp, out, bias=bias, bf16=True)
    torch.cuda.synchronize()
    assert not torch.isnan(out).any()
    return dev_to_bits(out)


def check_quantizer(oracle, capi, device, bs, weights_bits, has_offsets, col=True, **kw):
    n, k = weights_bits.shape
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, weights_bits, has_offsets, col=col, **kw)
    canon, s, z = oracle.quantize(bs, col, weights_bits, has_offsets, bf16=True)
    # scales and zero-points in the order the reference's entry point returns them (blocks along K: row-major
    # [K/bs, N]; blocks along N: its 16-row rearrangement), which is a matter of 16-bit patterns only
    ps, pz = oracle.prepack_meta_sm80(bs, col, k, n, s, z)
    assert np.array_equal(dev_to_bits(q_s), ps.view(np.uint16)), "scales differ"
    if col:
        assert np.array_equal(ps.view(np.uint16).reshape(k // bs, n), s.T)
    if has_offsets:
        assert np.array_equal(q_zp.cpu().numpy(), pz), "zero-points differ"
    got_w = q_w.cpu().numpy()
    want = oracle.native_from_canonical(canon)
    if not np.array_equal(got_w, want):
        bad = np.nonzero(got_w != want)[0]
        raise AssertionError(f"packed weights differ in {bad.size} bytes, first at {bad[:8]}")
    return q_w, q_s, q_zp, canon, s, z


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("has_offsets", [True, False])
@pytest.mark.parametrize("rows,columns", [(64, 32), (128, 96), (256, 256), (576, 672)])
def test_quantizer_gives_back_the_known_answers(oracle, capi, device, bs, has_offsets, rows, columns):
    kat = bf16_kat(oracle, bs, rows, columns, has_offsets, seed=rows + columns + bs)
    _, _, _, canon, s, z = check_quantizer(oracle, capi, device, bs, kat["weights"], has_offsets)
    assert np.array_equal(canon, kat["canon_w"]) and np.array_equal(s, kat["scales"])
    if has_offsets:
        assert np.array_equal(z, kat["zps"])


def gaussian_bits(oracle, seed, m, n, k, w_std=0.02):
    g = torch.Generator(device="cpu").manual_seed(seed)
    a = torch.randn(m, k, generator=g, dtype=torch.float32)
    w = torch.randn(n, k, generator=g, dtype=torch.float32) * w_std
    return oracle.f32_to_bf16(a.numpy()), oracle.f32_to_bf16(w.numpy())


@pytest.mark.parametrize("bs,has_offsets,rows,columns", [
    (16, True, 512, 352), (32, False, 1024, 1024), (64, True, 4096, 512), (32, True, 4096, 11008), (64, False, 448, 800),
])
def test_quantizer_on_gaussian_weights(oracle, capi, device, bs, has_offsets, rows, columns):
    _, w = gaussian_bits(oracle, rows + columns, 1, columns, rows)
    check_quantizer(oracle, capi, device, bs, w, has_offsets)


def test_quantizer_on_values_outside_fp16(oracle, capi, device):
    """magnitudes from 1e-30 to 1e30 per block (a bf16 has the exponent range of a float), zeros of both signs,
    all-zero blocks"""
    rng = np.random.default_rng(3)
    n, k = 128, 512
    mag = 10.0 ** rng.integers(-30, 31, (n, k // 16)).astype(np.float64)
    w = (rng.standard_normal((n, k)) * np.repeat(mag, 16, axis=1)).astype(np.float32)
    w[5, 64:128] = 0.0
    w[6, 0:64] = -0.0
    w[7, 128:192] = np.abs(w[7, 128:192])          # a block of one sign
    w[8, 192:256] = 3.0e38                           # a range that overflows a float: the scale is infinite
    w[8, 200] = -3.0e38
    w[9, 256:320] = 2.0 ** -133                      # bf16 subnormals
    w[9, 300] = -3 * 2.0 ** -133
    bits = oracle.f32_to_bf16(w)
    for bs in (16, 32, 64):
        for has_offsets in (True, False):
            for col in (True, False):
                check_quantizer(oracle, capi, device, bs, bits, has_offsets, col=col)


def test_quantizer_on_strided_and_unaligned_source(oracle, capi, device):
    _, w = gaussian_bits(oracle, 21, 1, 96, 192)
    ld = 200
    padded = torch.zeros(96 * ld + 3, dtype=torch.bfloat16, device=device)
    for shift in (0, 3):   # 3 elements: a source that is not 16-byte aligned
        view = padded[shift:shift + 96 * ld].view(96, ld)
        view[:, :192] = bits_to_dev(w, device)
        q_w, q_s, q_zp = quantize_bf16(capi, device, 32, w, True, w_dev=view, rows=192, columns=96, ld=ld)
        canon, s, z = oracle.quantize(32, True, w, True, bf16=True)
        assert np.array_equal(q_w.cpu().numpy(), oracle.native_from_canonical(canon))
        assert np.array_equal(dev_to_bits(q_s).reshape(6, 96), s.T)
        assert np.array_equal(q_zp.cpu().numpy().reshape(6, 96), z.T)


# (block_size, has_offsets, m, n, k): the reference's column-wise cases (test/blkq4_fp16_gemm_sm80_test.cu:501-518),
# then M = 1 and ragged M, wide N (waves with column tiles of their own, several column groups per workgroup),
# long K (rows staged per slice), row groups of 32, and the tile kernel's shapes (256 x 256, 128 x 256, 128 x 128 and
# 64 x 128 tiles, 32- and 64-row tiles on very wide layers, ragged edges)
EXACT_CASES = [
    (16, False, 256, 672, 576), (16, True, 256, 672, 576), (64, False, 256, 1024, 576), (64, True, 256, 1024, 576),
    (16, False, 16, 672, 576), (16, True, 16, 672, 576), (64, False, 16, 1024, 576), (64, True, 16, 1024, 576),
    (32, True, 1, 96, 64), (64, False, 1, 4096, 4096), (32, True, 3, 672, 576), (16, True, 17, 160, 128),
    (64, True, 33, 288, 320), (32, False, 100, 800, 448), (32, True, 300, 256, 64), (64, True, 1, 32000, 1024),
    (32, True, 2, 14336, 1024), (16, True, 9, 16416, 448), (32, True, 16, 64, 8192 + 64), (64, False, 9, 64, 12288),
    (32, True, 16, 11008, 1024), (64, True, 64, 4128, 320), (16, False, 96, 5440, 192), (32, True, 1500, 544, 128),
    (64, False, 2048 + 5, 96, 192), (64, True, 4096, 4096, 128), (16, True, 4000, 4128, 64), (32, False, 4096, 4096, 192),
    (64, True, 300, 4128, 192), (16, True, 500, 2080, 128), (32, False, 257, 4096, 64), (32, True, 1100, 4160, 128),
    (64, True, 48, 28672, 256), (32, False, 64, 36864, 128), (16, False, 32, 28672, 2624), (32, True, 24, 36864, 2624),
    (64, True, 768, 1056, 576), (16, True, 129, 1056, 576),
    # five to seven column tiles per workgroup (wide layers, rows staged per slice)
    (64, True, 16, 18432, 1088), (32, False, 9, 22016, 1088), (16, True, 12, 28672, 1216), (32, True, 16, 57344, 1024),
    # 128 x 32 tiles whose four computing waves split the k tile
    (64, False, 255, 4096, 3008), (16, True, 200, 4096, 4096),
]


@pytest.mark.parametrize("bs,has_offsets,m,n,k", EXACT_CASES)
def test_gemm_exact_on_known_answer_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = bf16_kat(oracle, bs, k, n, has_offsets, seed=m + n + k)
    a = grid_activations_bf16(oracle, rng, m, k)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, kat["weights"], has_offsets)
    assert np.array_equal(q_w.cpu().numpy(), oracle.native_from_canonical(kat["canon_w"]))
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n)
    ref = oracle.gemm(a, kat["weights"], bf16=True)
    # the oracle itself against exact arithmetic: float64 holds these sums exactly
    c64 = oracle.bf16_to_f32(a).astype(np.float64) @ kat["exact"].T
    assert np.array_equal(c64.astype(np.float32).astype(np.float64), c64)   # the sums fit a float
    assert np.array_equal(ref, oracle.f32_to_bf16(c64.astype(np.float32)))
    if not np.array_equal(got, ref):
        bad = np.argwhere(got != ref)
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}: "
                             f"got {got[tuple(bad[0])]:#06x} want {ref[tuple(bad[0])]:#06x}")


@pytest.mark.parametrize("bs,has_offsets,m,n,k,seed", [
    (32, True, 64, 1024, 1024, 2235), (64, False, 1, 4096, 4096, 2236), (32, True, 16, 11008, 4096, 2237),
    (64, True, 128, 4096, 4096, 2238), (16, True, 8, 2048, 8192, 2239), (64, True, 1100, 1056, 512, 2240),
    (64, True, 2048, 4096, 4096, 2241), (16, True, 512, 4096, 2048, 2242),
])
def test_gemm_on_gaussian_data(oracle, capi, device, bs, has_offsets, m, n, k, seed):
    a, w = gaussian_bits(oracle, seed, m, n, k)
    q_w, q_s, q_zp, canon, s, z = check_quantizer(oracle, capi, device, bs, w, has_offsets)
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n)
    b = oracle.dequantize(bs, True, canon, s, z, bf16=True)
    ref = oracle.gemm(a, b, bf16=True)
    gf, rf = oracle.bf16_to_f32(got), oracle.bf16_to_f32(ref)
    err = max_rel_err(gf, rf)
    c64 = oracle.bf16_to_f32(a).astype(np.float64) @ oracle.bf16_to_f32(b).astype(np.float64).T
    err64 = max_rel_err(gf, c64)
    print(f"bf16 m={m} n={n} k={k} bs={bs} zp={has_offsets}: max rel err {err:.3e} (oracle), {err64:.3e} (float64), "
          f"bit-identical outputs {float(np.mean(got == ref)):.4f}")
    assert err <= TOLERANCE
    assert err64 <= 2.0 ** -8 + 1e-4   # half a unit in the last place plus the fp32 accumulation


@pytest.mark.parametrize("bs,has_offsets,m,n,k", [(64, False, 1, 4096, 512), (32, True, 16, 1056, 576),
                                                  (16, True, 64, 352, 256), (64, True, 2, 32000, 256),
                                                  (32, True, 1100, 544, 128), (64, True, 300, 4128, 192),
                                                  (16, True, 4096, 4096, 64)])
def test_bias_equals_a_separate_add(oracle, capi, device, bs, has_offsets, m, n, k):
    """the bias is added to the bf16 output the way the tensor library adds two bf16 tensors (in fp32, one
    rounding), which is what the reference module does with fp16 (python/ms_blkq4linear.py:26-27)"""
    a, w = gaussian_bits(oracle, m + n + k, m, n, k)
    g = torch.Generator(device="cpu").manual_seed(n)
    bias = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16).to(device)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, w, has_offsets)
    plain = torch.from_numpy(gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n).view(np.int16)).to(device).view(torch.bfloat16)
    fused = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n, bias=bias)
    plain += bias
    assert np.array_equal(fused, dev_to_bits(plain))


def test_packed_weights_and_offsets_are_those_of_the_fp16_quantizer(oracle, capi, device):
    """on data exact in both 16-bit types the two quantizers pack the same nibbles and offsets; only the scales
    differ in their encoding"""
    kat = bf16_kat(oracle, 32, 256, 96, True, seed=4)
    w16 = kat["exact"].astype(np.float16)
    assert np.array_equal(w16.astype(np.float64), kat["exact"])
    from gpu_util import quantize_on_gpu, to_np
    h_w, h_s, h_z = quantize_on_gpu(capi, device, 32, np.ascontiguousarray(w16), True)
    b_w, b_s, b_z = quantize_bf16(capi, device, 32, kat["weights"], True)
    assert torch.equal(h_w, b_w) and torch.equal(h_z, b_z)
    assert np.array_equal(to_np(h_s).astype(np.float32), oracle.bf16_to_f32(dev_to_bits(b_s)))


@pytest.mark.parametrize("scale_only", [False, True])
@pytest.mark.parametrize("m", [1, 16, 80])
def test_module_takes_bfloat16(oracle, capi, device, scale_only, m):
    """BlkQ4Linear built from bfloat16 weights: bfloat16 scales, bias and output, the result that of the C entry
    points (which the tests above hold against the oracle); a float16 input to such a layer is refused"""
    import ms_blkq4linear as mod
    g = torch.Generator(device="cpu").manual_seed(13 + m)
    k, n, bs = 512, 384, 64
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    x = torch.randn(3, m, k, generator=g).to(torch.bfloat16)
    layer = mod.BlkQ4Linear(bs, True, scale_only, w.to(device), bias.to(device))
    assert layer.q_scales.dtype == torch.bfloat16 and layer.q_weights.dtype == torch.uint8
    y = layer(x.to(device))
    assert y.shape == (3, m, n) and y.dtype == torch.bfloat16
    w_bits = w.view(torch.int16).numpy().view(np.uint16)
    canon, _, _ = oracle.quantize(bs, True, w_bits, not scale_only, bf16=True)
    assert np.array_equal(layer.q_weights.cpu().numpy(), oracle.native_from_canonical(canon))
    x_bits = x.reshape(3 * m, k).view(torch.int16).numpy().view(np.uint16)

    def check(out, col):
        """against the oracle's GEMM plus the bias: an output's error is measured against the larger of the two
        summands (the sum itself may cancel), as a separate add of two bf16 tensors would be"""
        canon, s, z = oracle.quantize(bs, col, w_bits, not scale_only, bf16=True)
        c = oracle.gemm(x_bits, oracle.dequantize(bs, col, canon, s, z, bf16=True), bf16=True)
        c = torch.from_numpy(c.view(np.int16)).view(torch.bfloat16)
        ref = (c + bias).float().numpy()
        scale = np.maximum(np.maximum(np.abs(c.float().numpy()), np.abs(bias.float().numpy())[None, :]), 1e-3)
        got = out.reshape(3 * m, n).float().cpu().numpy()
        # a unit in the last place of the GEMM output (2^-7) plus the rounding of the sum (2^-8 of up to twice the scale)
        assert np.max(np.abs(got - ref) / scale) <= 2 * TOLERANCE

    check(y, True)
    with pytest.raises(RuntimeError, match="must have the input's element type"):
        layer(x.to(device).to(torch.float16))
    # blocks along N through the module
    row_layer = mod.BlkQ4Linear(bs, False, scale_only, w.to(device), bias.to(device))
    check(row_layer(x.to(device)), False)


# ---------------------------------------------------------------------------------------------
# blocks along N (column_wise_blocking = false)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("has_offsets", [True, False])
@pytest.mark.parametrize("rows,columns", [(64, 64), (128, 192), (576, 704)])
def test_row_wise_quantizer_gives_back_the_known_answers(oracle, capi, device, bs, has_offsets, rows, columns):
    kat = bf16_kat(oracle, bs, rows, columns, has_offsets, seed=rows + columns + bs, column_wise=False)
    _, _, _, canon, s, z = check_quantizer(oracle, capi, device, bs, kat["weights"], has_offsets, col=False)
    assert np.array_equal(canon, kat["canon_w"]) and np.array_equal(s, kat["scales"])
    if has_offsets:
        assert np.array_equal(z, kat["zps"])


@pytest.mark.parametrize("bs,has_offsets,rows,columns", [(16, True, 512, 352), (32, False, 1024, 1024), (64, True, 448, 832)])
def test_row_wise_quantizer_on_gaussian_weights(oracle, capi, device, bs, has_offsets, rows, columns):
    _, w = gaussian_bits(oracle, rows + columns + 1, 1, columns, rows)
    check_quantizer(oracle, capi, device, bs, w, has_offsets, col=False)


# the reference's row-wise cases (test/blkq4_fp16_gemm_sm80_test.cu:480-499,508-512), M = 1 and ragged M, the tile
# kernel's four tile shapes, very wide N in the streaming kernel
ROW_WISE_EXACT_CASES = [
    (32, False, 32, 32, 64), (32, True, 32, 96, 192), (32, True, 256, 672, 576), (32, False, 512, 2048 + 32, 960),
    (16, True, 256, 672, 576), (64, False, 256, 1024, 576), (16, False, 16, 704, 576), (64, True, 16, 1024, 576),
    (64, False, 1, 1024, 576), (16, True, 2, 160, 128), (64, True, 7, 1088, 192), (32, True, 17, 96, 192),
    (16, True, 65, 544, 256), (64, True, 129, 1088, 576), (16, True, 400, 672, 576), (32, True, 1000, 4128, 128),
    (64, True, 640, 4160, 192), (16, True, 4096, 4096, 128), (64, True, 4096, 4096, 192), (32, True, 160, 96, 8256),
    (64, False, 1, 14336, 4096), (32, True, 2, 16384, 2112), (16, True, 8, 28672, 1088), (64, True, 16, 16384, 8256),
]


@pytest.mark.parametrize("bs,has_offsets,m,n,k", ROW_WISE_EXACT_CASES)
def test_row_wise_gemm_exact_on_known_answer_construction(oracle, capi, device, bs, has_offsets, m, n, k):
    rng = np.random.default_rng(m * 131 + n * 17 + k + bs + has_offsets)
    kat = bf16_kat(oracle, bs, k, n, has_offsets, seed=m + n + k, column_wise=False)
    a = grid_activations_bf16(oracle, rng, m, k)
    q_w, q_s, q_zp = quantize_bf16(capi, device, bs, kat["weights"], has_offsets, col=False)
    assert np.array_equal(q_w.cpu().numpy(), oracle.native_from_canonical(kat["canon_w"]))
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n, col=False)
    c64 = oracle.bf16_to_f32(a).astype(np.float64) @ kat["exact"].T
    assert np.array_equal(c64.astype(np.float32).astype(np.float64), c64)   # the sums fit a float
    ref = oracle.gemm(a, kat["weights"], bf16=True)
    assert np.array_equal(ref, oracle.f32_to_bf16(c64.astype(np.float32)))
    if not np.array_equal(got, ref):
        bad = np.argwhere(got != ref)
        raise AssertionError(f"{bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}: "
                             f"got {got[tuple(bad[0])]:#06x} want {ref[tuple(bad[0])]:#06x}")


@pytest.mark.parametrize("bs,has_offsets,m,n,k,seed", [
    (32, True, 64, 1024, 1024, 3235), (64, False, 1, 4096, 4096, 3236), (16, True, 16, 2816, 1024, 3237),
    (64, True, 200, 1152, 512, 3238), (64, True, 2048, 4096, 1024, 3239),
])
def test_row_wise_gemm_on_gaussian_data(oracle, capi, device, bs, has_offsets, m, n, k, seed):
    a, w = gaussian_bits(oracle, seed, m, n, k)
    q_w, q_s, q_zp, canon, s, z = check_quantizer(oracle, capi, device, bs, w, has_offsets, col=False)
    got = gemm_bf16(capi, device, bs, a, q_w, q_s, q_zp, n, col=False)
    ref = oracle.gemm(a, oracle.dequantize(bs, False, canon, s, z, bf16=True), bf16=True)
    err = max_rel_err(oracle.bf16_to_f32(got), oracle.bf16_to_f32(ref))
    print(f"bf16 row-wise m={m} n={n} k={k} bs={bs} zp={has_offsets}: max rel err {err:.3e}, "
          f"bit-identical outputs {float(np.mean(got == ref)):.4f}")
    assert err <= TOLERANCE


def test_module_state_dict_round_trip_in_bfloat16(device):
    """a bfloat16 layer's state travels like a float16 layer's, and neither takes the other's"""
    import ms_blkq4linear as mod
    g = torch.Generator(device="cpu").manual_seed(12)
    k, n, bs = 128, 64, 64
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16).to(device)
    bias = torch.randn(n, generator=g).to(torch.bfloat16).to(device)
    x = torch.randn(7, k, generator=g).to(torch.bfloat16).to(device)
    layer = mod.BlkQ4Linear(bs, True, False, w, bias)
    state = layer.state_dict()
    other = mod.BlkQ4Linear(bs, True, False, torch.zeros_like(w), torch.zeros_like(bias))
    other.load_state_dict(state)
    assert other.q_scales.dtype == torch.bfloat16 and torch.equal(other(x), layer(x))
    half = mod.BlkQ4Linear(bs, True, False, torch.zeros(n, k, dtype=torch.float16, device=device))
    with pytest.raises((ValueError, RuntimeError)):
        half.load_state_dict(state, strict=False)
    with pytest.raises((ValueError, RuntimeError)):
        other.load_state_dict(half.state_dict(), strict=False)
    packed = mod.BlkQ4Linear.from_packed(bs, True, k, n, layer.q_weights, layer.q_scales, layer.q_zp, bias)
    assert torch.equal(packed(x), layer(x))
