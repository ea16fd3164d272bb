"""Pins the bf16 variants of the CPU oracle (no GPU needed) and the host-side checks of the bf16 entry points.

The reference has no bf16 path and therefore no vectors for one (src/blkq4_f16_gemm_sm80.cu:53 rejects the
type), so the oracle's bf16 functions are the fp16 ones with the 16-bit conversions exchanged, and what pins
them is
  * the conversions, exhaustively: every bf16 pattern up, and the rounding of floats against a definition
    written with float64 distances (nearest, ties to the even mantissa);
  * the quantizer: the reference's round-trip property (test/blkq4_fp16_quant_sm80_test.cu:53-68) on data
    built to be exact in bf16: quantize(dequantize(q, s, zp)) gives back q, s and zp;
  * dequantize and GEMM: float64 numpy.
"""

import numpy as np
import pytest

from bf16_util import bf16_kat


def test_bf16_to_float_exhaustive(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = (bits.astype(np.uint32) << 16).view(np.float32)
    got = np.array([L.oracle_b2f(int(b)) for b in bits], np.float32)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)) or np.array_equal(
        got.view(np.uint32) | 0x00400000, ref.view(np.uint32) | 0x00400000)  # a signalling NaN may come back quiet
    assert np.array_equal(oracle.bf16_to_f32(bits).view(np.uint32), ref.view(np.uint32))


def nearest_bf16_by_distance(x: np.ndarray) -> np.ndarray:
    """round to nearest, ties to even, from the definition: the two bf16 neighbours of a finite float and
    their float64 distances to it (no integer rounding trick)."""
    u = x.view(np.uint32)
    lo_bits = (u >> 16).astype(np.uint32)          # truncation: the neighbour nearer to zero
    hi_bits = lo_bits + 1                          # the next pattern away from zero (may be the infinity)
    lo = (lo_bits << 16).view(np.float32).astype(np.float64)
    hi_is_inf = (hi_bits & 0x7F80) == 0x7F80
    # the overflow threshold counts the infinity as the value one step beyond the largest finite number
    step = lo - ((lo_bits - 1) << 16).view(np.float32).astype(np.float64)
    hi = np.where(hi_is_inf, lo + step, (hi_bits << 16).view(np.float32).astype(np.float64))
    xd = x.astype(np.float64)
    d_lo, d_hi = np.abs(xd - lo), np.abs(hi - xd)
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & ((lo_bits & 1) == 1))
    return np.where(pick_hi, hi_bits, lo_bits).astype(np.uint16)


def test_float_to_bf16_rounding(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(11)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 20000).astype(np.float32),
        # exact ties, their float neighbours, the overflow threshold, subnormals, zeros
        np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, np.nextafter(np.float32(1.0 + 2.0 ** -8), np.float32(2)),
                  np.nextafter(np.float32(1.0 + 2.0 ** -8), np.float32(0)), 3.3895313892515355e38, 3.4e38,
                  np.finfo(np.float32).max, 1e-40, 9.2e-41, 2.0 ** -133, 2.0 ** -134, 3 * 2.0 ** -134, 0.0, -0.0,
                  -1.0 - 2.0 ** -8, -255.5, 255.5, 256.5, 257.5], np.float32),
    ])
    xs = xs[np.isfinite(xs)]
    ref = nearest_bf16_by_distance(xs)
    got = np.array([L.oracle_f2b(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, ref)
    assert np.array_equal(oracle.f32_to_bf16(xs), ref)
    # every bf16 value converts to itself
    bits = np.arange(65536, dtype=np.uint16)
    finite = (bits & 0x7F80) != 0x7F80
    assert np.array_equal(oracle.f32_to_bf16(oracle.bf16_to_f32(bits[finite])), bits[finite])
    assert L.oracle_f2b(float("inf")) == 0x7F80 and L.oracle_f2b(float("-inf")) == 0xFF80
    assert (L.oracle_f2b(float("nan")) & 0x7FFF) > 0x7F80


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("has_offsets", [False, True])
@pytest.mark.parametrize("rows,cols", [(64, 64), (128, 192), (256, 320)])
@pytest.mark.parametrize("col", [True, False])
def test_quantizer_round_trip_on_bf16_exact_data(oracle, bs, has_offsets, rows, cols, col):
    kat = bf16_kat(oracle, bs, rows, cols, has_offsets, seed=rows + cols + bs, column_wise=col)
    # the construction is exact: float64 product equals the bf16 weight
    w64 = oracle.bf16_to_f32(kat["weights"]).astype(np.float64)
    assert np.array_equal(w64, kat["exact"])
    cw, s, z = oracle.quantize(bs, col, kat["weights"], has_offsets, bf16=True)
    assert np.array_equal(cw, kat["canon_w"])
    assert np.array_equal(s, kat["scales"])
    if has_offsets:
        assert np.array_equal(z, kat["zps"])
    # and back: the oracle's dequantization reproduces the weights bit for bit
    assert np.array_equal(oracle.dequantize(bs, col, cw, s, z, bf16=True), kat["weights"])


def test_quantizer_scale_is_rounded_to_bf16_not_fp16(oracle):
    """a block whose range / 15 needs more than 8 mantissa bits and lies outside fp16's range"""
    w = np.zeros((32, 64), np.float32)
    w[:, 0] = 1.0e6
    w[:, 1] = -3.0e5
    bits = oracle.f32_to_bf16(w)
    wf = oracle.bf16_to_f32(bits)
    cw, s, z = oracle.quantize(64, True, bits, True, bf16=True)
    rng_f = np.float32(wf[0, 0]) - np.float32(wf[0, 1])
    want = oracle.f32_to_bf16(np.array([rng_f / np.float32(15.0)], np.float32))[0]
    assert np.all(s == want)
    zp = int(np.round(-float(wf[0, 1]) / float(rng_f / np.float32(15.0))))
    assert np.all(z == zp)
    q = oracle.nibbles_from_canonical(cw)
    assert np.all(q[:, 0] == 15) and np.all(q[:, 1] == 0) and np.all(q[:, 2:] == zp)


def test_dequantize_and_gemm_against_float64(oracle):
    rng = np.random.default_rng(5)
    n, k, m, bs = 96, 256, 9, 32
    q = rng.integers(0, 16, (n, k)).astype(np.uint8)
    canon = oracle.canonical_from_nibbles(q)
    scales = oracle.f32_to_bf16((rng.standard_normal((n, k // bs)) * 0.01).astype(np.float32))
    zps = rng.integers(0, 16, (n, k // bs)).astype(np.uint8)
    for z in (zps, None):
        b = oracle.dequantize(bs, True, canon, scales, z, bf16=True)
        s64 = np.repeat(oracle.bf16_to_f32(scales).astype(np.float64), bs, axis=1)
        z64 = np.repeat(zps.astype(np.float64), bs, axis=1) if z is not None else 8.0
        exact = s64 * (q.astype(np.float64) - z64)      # exact in float64, and in float32 (12-bit products)
        assert np.array_equal(b, oracle.f32_to_bf16(exact.astype(np.float32)))
        a = oracle.f32_to_bf16(rng.standard_normal((m, k)).astype(np.float32))
        c = oracle.bf16_to_f32(oracle.gemm(a, b, bf16=True)).astype(np.float64)
        c_strict = oracle.gemm(a, b, strict_order=True, bf16=True)
        c64 = oracle.bf16_to_f32(a).astype(np.float64) @ oracle.bf16_to_f32(b).astype(np.float64).T
        # one rounding to bf16 (2^-9 relative) on top of fp32 accumulation
        assert np.max(np.abs(c - c64) / np.maximum(np.abs(c64), 1e-3 * np.abs(c64).max())) <= 2.0 ** -8
        cs = oracle.bf16_to_f32(c_strict).astype(np.float64)
        assert np.max(np.abs(cs - c64) / np.maximum(np.abs(c64), 1e-3 * np.abs(c64).max())) <= 2.0 ** -8


def test_gemm_exact_integer_case(oracle):
    """small integers: every product and sum is exact, so the output is the bf16 rounding of an integer"""
    rng = np.random.default_rng(9)
    a = rng.integers(-8, 9, (5, 128)).astype(np.float32)
    b = rng.integers(-8, 9, (48, 128)).astype(np.float32)
    c = oracle.gemm(oracle.f32_to_bf16(a), oracle.f32_to_bf16(b), bf16=True)
    want = nearest_bf16_by_distance((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert np.array_equal(c, want)


# ---------------------------------------------------------------------------------------------
# host-side checks of the bf16 entry points (no kernel is reached)
# ---------------------------------------------------------------------------------------------

def _buf(nbytes, address=0x1000):
    from gemmlib_amd.capi import RawBuffer
    return RawBuffer(address, nbytes)


@pytest.mark.parametrize("kwargs,message", [
    (dict(col=False, bs=64, n=96, s=_buf(64 * 1 * 2), c=_buf(4 * 96 * 2)), "Kernel execution failed: Error Invalid Problem"),
    (dict(bs=8), "Unsupported block size: 8"),
    (dict(m=0), "Empty problem size: 0x64x64"),
    (dict(a=_buf(10)), "Unexpected activation tensor size: 10 expected: 512"),
    (dict(s=_buf(100)), "Unexpected scale tensor size: 100 expected: 256"),
    (dict(c=_buf(8)), "Unexpected output tensor size: 8 expected: 512"),
    (dict(bias=_buf(126)), "Unexpected bias tensor size: 126 expected: 128"),
])
def test_bf16_gemm_validation_messages(capi, kwargs, message):
    kw = dict(bs=32, col=True, m=4, n=64, k=64, a=None, s=None, c=None, bias=None)
    kw.update(kwargs)
    bs, m, n, k = kw["bs"], kw["m"], kw["n"], kw["k"]
    a = _buf(m * k * 2) if kw["a"] is None else kw["a"]
    s = _buf((k // max(bs, 1)) * n * 2) if kw["s"] is None else kw["s"]
    c = _buf(m * n * 2) if kw["c"] is None else kw["c"]
    with pytest.raises(capi.Blkq4Error) as e:
        capi.gemm(bs, kw["col"], m, n, k, a, _buf(k * n // 2), s, None, c, stream=0, bias=kw["bias"], bf16=True)
    assert str(e.value) == message


def test_bf16_quant_validation_messages(capi):
    lib = capi.load()

    def call(bs=32, col=True, rows=64, cols=32, qs_bytes=None):
        err = lib.blkq4_error_message_create()
        try:
            qs = (rows // bs) * cols * 2 if qs_bytes is None else qs_bytes
            rc = lib.blkq4_bf16_quant_sm80(bs, col, rows, cols, rows, None, 0x1000, cols * rows * 2, 0x9000,
                                           rows * cols // 2, 0x20000, qs, None, 0, err)
            return rc, lib.blkq4_error_message_cstr(err).decode()
        finally:
            lib.blkq4_error_message_destroy(err)

    assert call(col=False, qs_bytes=60 * 2) == (-1, "Unexpected scale tensor size: 60 expected: 64")
    assert call(bs=128) == (-1, "Unsupported block size: 128")
    assert call(rows=100) == (-1, "Cannot block quantize matrix with rows: 100")
    assert call(qs_bytes=100) == (-1, "Unexpected scale tensor size: 50 expected: 64")
