"""Pins the CPU oracle (no GPU needed).

The oracle is checked against
  * the reference's own round-trip known-answer construction (quantize(dequantize(x)) == x for the
    generator in test/blkq4_fp16_quant_sm80_test.cu:72-186, all shapes of :313-347);
  * an independently derived digest table of the reference's packed buffers and hand-checked spot
    values (tests/golden/kat_digests_independent.json);
  * closed forms of the quantizer arithmetic (all-zero blocks, ties, clamping, the rounding point of
    the scale) and brute force over every nibble value;
  * an independent numpy restatement of the sm80 permutation written from the layout's table form;
  * float64 matmul for the GEMM.
"""

import hashlib
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SHAPES = [(64, 32), (64, 64), (64, 128), (64, 256), (128, 32), (256, 32), (256, 256)]


def digest(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:16]


# ---------------------------------------------------------------------------------------------
# fp16 conversion of the oracle vs numpy (exhaustive one way, dense sample the other)
# ---------------------------------------------------------------------------------------------

def test_half_to_float_exhaustive(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([L.oracle_h2f(int(b)) for b in bits], np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))


def test_float_to_half_rounding(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(7)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 5, 20000).astype(np.float32),
        # exact ties between neighbouring fp16 values and their float neighbours
        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 6.0e-8, -0.0, 0.0, 5.96e-8, 6.1e-5, 6.0975e-5],
                 np.float32),
    ])
    ref = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.oracle_f2h(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, ref)


# ---------------------------------------------------------------------------------------------
# known-answer vectors of the reference
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("column_wise", [True, False])
@pytest.mark.parametrize("rows,columns", SHAPES)
@pytest.mark.parametrize("has_offsets", [True, False])
def test_kat_round_trip(oracle, column_wise, rows, columns, has_offsets):
    """reference: test/blkq4_fp16_quant_sm80_test.cu:53-68 -- quantizing the dequantized data gives
    the original nibbles, scales and zero-points back exactly."""
    kat = oracle.kat_generate(32, column_wise, rows, columns, has_offsets)
    for fused in (True, False):  # the reference vectors do not depend on the FMA contraction
        cw, s, z = oracle.quantize(32, column_wise, kat["weights"], has_offsets, fused=fused)
        assert np.array_equal(cw, kat["canon_w"])
        assert np.array_equal(s.view(np.uint16), kat["scales"].view(np.uint16))
        if has_offsets:
            assert np.array_equal(z, kat["zps"])


@pytest.mark.parametrize("bs", [16, 64])
@pytest.mark.parametrize("column_wise", [True, False])
def test_kat_round_trip_other_block_sizes(oracle, bs, column_wise):
    """block sizes the GEMM test uses (test/blkq4_fp16_gemm_sm80_test.cu:495-518)."""
    for has_offsets in (True, False):
        kat = oracle.kat_generate(bs, column_wise, 576 + 64, 672 - 32, has_offsets)  # 640 x 640
        cw, s, z = oracle.quantize(bs, column_wise, kat["weights"], has_offsets)
        assert np.array_equal(cw, kat["canon_w"])
        assert np.array_equal(s.view(np.uint16), kat["scales"].view(np.uint16))
        if has_offsets:
            assert np.array_equal(z, kat["zps"])


def test_kat_digests_match_independent_table(oracle):
    with open(os.path.join(GOLDEN, "kat_digests_independent.json")) as f:
        table = json.load(f)
    for case in table["cases"]:
        kat = oracle.kat_generate(32, case["column_wise"], case["rows"], case["columns"], True)
        pw, ps, pz = oracle.quant_sm80(32, case["column_wise"], kat["weights"], True)
        assert digest(kat["canon_w"]) == case["canonW"], case
        assert digest(pw) == case["packedW"], case
        assert digest(ps.view(np.uint16)) == case["packedS"], case
        assert digest(pz) == case["packedZ"], case
    spot = table["spot_values_colwise_64x32"]
    kat = oracle.kat_generate(32, True, 64, 32, True)
    pw, ps, pz = oracle.quant_sm80(32, True, kat["weights"], True)
    assert " ".join(f"{b:02x}" for b in kat["canon_w"].reshape(-1)[:16]) == spot["canonW_first16"]
    assert " ".join(f"{b:02x}" for b in pw[:16]) == spot["packedW_first16"]
    assert " ".join(f"{b:04x}" for b in ps.view(np.uint16)[:8]) == spot["packedS_first8_fp16_bits"]
    assert pz[:16].tolist() == spot["packedZ_first16"]
    # hand check of the first packed byte: q(0,0) = 7 (the seed), q(8,0) = 4 -> 0x47
    q = oracle.nibbles_from_canonical(kat["canon_w"])
    assert q[0, 0] == 7 and q[0, 8] == 4 and pw[0] == 0x47


def test_committed_fixture_is_current(oracle):
    """tests/golden/kat_fixtures.json is what make_kat_fixtures.py writes today."""
    with open(os.path.join(GOLDEN, "kat_fixtures.json")) as f:
        fx = json.load(f)
    for case in fx["cases"]:
        kat = oracle.kat_generate(32, case["column_wise"], case["rows"], case["columns"], True)
        pw, ps, pz = oracle.quant_sm80(32, case["column_wise"], kat["weights"], True)
        assert digest(pw) == case["packedW"]
        assert digest(oracle.native_from_canonical(kat["canon_w"])) == case["nativeW"]
        if "hex" in case:
            assert kat["weights"].view(np.uint16).astype("<u2").tobytes().hex() == case["hex"]["weights_fp16"]
            assert pw.tobytes().hex() == case["hex"]["packedW"]


# ---------------------------------------------------------------------------------------------
# sm80 weight permutation against an independent restatement (table form of the layout)
# ---------------------------------------------------------------------------------------------

def _sm80_from_table(q_nk: np.ndarray) -> np.ndarray:
    """For each 16x16 tile at (k0,n0), row 0..3, col 0..7, s 0..3: byte (k0+4row+s, n0/2+col) has
    low = q(k0+2row+(s>>1), n0+col+8(s&1)), high = the same at k+8.  Column-major uint8[K, N/2]."""
    n, k = q_nk.shape
    out = np.zeros((n // 2, k), np.uint8)  # [pc][pr]
    for k0 in range(0, k, 16):
        for n0 in range(0, n, 16):
            for row in range(4):
                for col in range(8):
                    for s in range(4):
                        kk = k0 + 2 * row + (s >> 1)
                        nn = n0 + col + 8 * (s & 1)
                        out[n0 // 2 + col, k0 + 4 * row + s] = q_nk[nn, kk] | (q_nk[nn, kk + 8] << 4)
    return out.reshape(-1)


@pytest.mark.parametrize("rows,columns", [(64, 32), (128, 64), (192, 96)])
def test_prepack_weights_matches_table_form(oracle, rows, columns):
    rng = np.random.default_rng(rows * 1000 + columns)
    q = rng.integers(0, 16, (columns, rows), dtype=np.uint8)
    canon = oracle.canonical_from_nibbles(q)
    got = oracle.prepack_weights_sm80(canon)
    assert np.array_equal(got, _sm80_from_table(q))
    # a permutation of nibbles: the multiset of nibbles is preserved
    assert np.array_equal(np.bincount(got & 15, minlength=16) + np.bincount(got >> 4, minlength=16),
                          np.bincount(q.reshape(-1), minlength=16))


def test_prepack_meta_colwise_is_a_transpose(oracle):
    rng = np.random.default_rng(3)
    k, n, bs = 256, 96, 32
    s = rng.standard_normal((n, k // bs)).astype(np.float16)  # canonical: col-major [K/bs, N]
    z = rng.integers(0, 16, (n, k // bs), dtype=np.uint8)
    ps, pz = oracle.prepack_meta_sm80(bs, True, k, n, s, z)
    assert np.array_equal(ps.reshape(k // bs, n), s.T)
    assert np.array_equal(pz.reshape(k // bs, n), z.T)


def test_prepack_meta_rowwise_permutation(oracle):
    """f16_quant_sm80.cuh:506-512,528-539: per 16-row group, scales [0,1,8,9,2,3,10,11,...],
    zero-points [0,8,1,9,2,10,...]."""
    k, n, bs = 64, 64, 32
    s = np.arange(k * (n // bs), dtype=np.float16).reshape(n // bs, k)
    z = (np.arange(k * (n // bs)) % 251).astype(np.uint8).reshape(n // bs, k)
    ps, pz = oracle.prepack_meta_sm80(bs, False, k, n, s, z)
    s_perm = [0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15]
    z_perm = [0, 8, 1, 9, 2, 10, 3, 11, 4, 12, 5, 13, 6, 14, 7, 15]
    ps = ps.reshape(n // bs, k)
    pz = pz.reshape(n // bs, k)
    for c in range(n // bs):
        for blk in range(0, k, 16):
            assert np.array_equal(ps[c, blk:blk + 16], s[c, blk:blk + 16][s_perm])
            assert np.array_equal(pz[c, blk:blk + 16], z[c, blk:blk + 16][z_perm])


# ---------------------------------------------------------------------------------------------
# quantizer closed forms
# ---------------------------------------------------------------------------------------------

def _one_block(oracle, values, bs, has_offsets, fused=True):
    """Quantize a [64, 32] matrix whose first block (k = 0..bs-1 of column 0) holds `values`."""
    w = np.zeros((32, 64), np.float16)
    w[0, :bs] = np.asarray(values, np.float16)
    cw, s, z = oracle.quantize(bs, True, w, has_offsets, fused=fused)
    q = oracle.nibbles_from_canonical(cw)
    return q[0, :bs], s[0, 0], (None if z is None else z[0, 0]), (q, s, z)


def test_all_zero_block(oracle):
    q, s, z, (qa, sa, za) = _one_block(oracle, np.zeros(32), 32, True)
    # asymmetric: scale +0, zp 0, nibbles 0 (f16_quant_sm80.cuh:107-121, 293)
    assert s.view(np.uint16) == 0x0000 and z == 0 and not q.any()
    assert not qa.any() and not za.any()
    q, s, z, (qa, sa, _) = _one_block(oracle, np.zeros(32), 32, False)
    # symmetric: 0 / -8 = -0.0 (bits 0x8000), reciprocal 0, every nibble = zp = 8 (:132-134, :293)
    assert s.view(np.uint16) == 0x8000 and (q == 8).all() and (qa == 8).all()
    # a block of negative zeros: min = max = -0.0, -0.0 / -8 = +0.0
    q, s, _, _ = _one_block(oracle, -np.zeros(32), 32, False)
    assert s.view(np.uint16) == 0x0000 and (q == 8).all()


def test_asymmetric_extremes_and_scale(oracle):
    vals = np.linspace(-1.0, 2.0, 32).astype(np.float16)
    q, s, z, _ = _one_block(oracle, vals, 32, True)
    f = vals.astype(np.float32)
    scale_f = np.float32(f.max() - f.min()) / np.float32(15)
    assert s.view(np.uint16) == np.float16(scale_f).view(np.uint16)
    assert z == 5  # round(1 / 0.2)
    assert q[0] == 0 and q[-1] == 15 and (np.diff(q.astype(int)) >= 0).all()
    # a block that does not straddle zero is widened to include it (:104-105)
    q, s, z, _ = _one_block(oracle, np.full(32, 3.0), 32, True)
    assert z == 0 and s.view(np.uint16) == np.float16(np.float32(3.0) / np.float32(15)).view(np.uint16)
    assert (q == 15).all()
    q, s, z, _ = _one_block(oracle, np.full(32, -3.0), 32, True)
    assert z == 15 and (q == 0).all()


def test_symmetric_sign_convention_and_tie(oracle):
    vals = np.zeros(32)
    vals[3], vals[7] = 4.0, -2.0
    q, s, _, _ = _one_block(oracle, vals, 32, False)
    assert s == np.float16(-0.5)            # extreme is positive -> negative scale (:132-134)
    assert q[3] == 0 and q[7] == 12 and q[0] == 8
    vals[3], vals[7] = 2.0, -4.0
    q, s, _, _ = _one_block(oracle, vals, 32, False)
    assert s == np.float16(0.5) and q[7] == 0 and q[3] == 12
    vals[3], vals[7] = 4.0, -4.0            # tie: fabsf(max) > fabsf(min) is false -> min
    q, s, _, _ = _one_block(oracle, vals, 32, False)
    assert s == np.float16(0.5) and q[7] == 0 and q[3] == 15  # +4 / 0.5 + 8 = 16 -> clamped to 15


def test_round_half_away_and_clamp_bruteforce(oracle):
    """every nibble value and every half-way point, against an independent float64 evaluation."""
    for s_val, zp in [(0.5, 8), (0.25, 3), (2.0, 12)]:
        # a block whose range gives exactly scale s_val and zero-point zp
        lo, hi = -zp * s_val, (15 - zp) * s_val
        grid = np.arange(-2, 34) * (s_val / 2) + lo      # half steps, below and above the range
        grid = np.clip(grid, lo, hi)[:30]
        vals = np.concatenate([[lo, hi], grid]).astype(np.float16)
        q, s, z, _ = _one_block(oracle, vals, 32, True)
        assert s == np.float16(s_val) and z == zp
        t = vals.astype(np.float64) / s_val + zp
        expect = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), 0, 15).astype(np.uint8)
        assert np.array_equal(q, expect)


def test_scale_is_reread_after_fp16_rounding(oracle):
    """f16_quant_sm80.cuh:291-293: the reciprocal uses the ROUNDED scale.  Pick a range whose fp32 scale
    is not an fp16 value and a weight whose nibble differs between the two choices."""
    rng = np.random.default_rng(11)
    found = 0
    for _ in range(200):
        vals = (rng.standard_normal(32) * 0.02).astype(np.float16)
        q, s, z, _ = _one_block(oracle, vals, 32, True)
        f = vals.astype(np.float32)
        mn, mx = min(f.min(), np.float32(0)), max(f.max(), np.float32(0))
        scale_f = (mx - mn) / np.float32(15)
        r16 = np.float32(1) / np.float32(s)
        r32 = np.float32(1) / scale_f
        t16 = np.round(np.float64(f) * np.float64(r16) + z)   # float64 stand-in for the fused form
        t32 = np.round(np.float64(f) * np.float64(r32) + z)
        differ = t16 != t32
        if differ.any():
            found += 1
            idx = np.nonzero(differ)[0]
            # away from exact .5 ties the float64 stand-in is decisive
            frac = np.abs((np.float64(f) * np.float64(r16) + z) % 1 - 0.5)
            idx = idx[frac[idx] > 1e-3]
            assert np.array_equal(q[idx], np.clip(t16[idx], 0, 15).astype(np.uint8))
    assert found > 0


def test_fma_contraction_sensitivity_is_small_but_nonzero(oracle):
    """the one unpinned detail: fused vs unfused v * r + zp (documented in the oracle header)."""
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((1024, 2048)) * 0.02).astype(np.float16)
    a = oracle.quantize(32, True, w, True, fused=True)[0]
    b = oracle.quantize(32, True, w, True, fused=False)[0]
    diff = np.count_nonzero(oracle.nibbles_from_canonical(a) != oracle.nibbles_from_canonical(b))
    assert 0 < diff < 200, diff


# ---------------------------------------------------------------------------------------------
# the library's own packed order: bijection
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("rows,columns", [(64, 32), (256, 96)])
def test_native_layout_is_a_bijection(oracle, rows, columns):
    rng = np.random.default_rng(rows + columns)
    q = rng.integers(0, 16, (columns, rows), dtype=np.uint8)
    canon = oracle.canonical_from_nibbles(q)
    nat = oracle.native_from_canonical(canon)
    assert nat.size == rows * columns // 2
    assert np.array_equal(oracle.canonical_from_native(nat, rows, columns), canon)
    # definition check on one element: weight (k, n) sits in unit (k//32, n), word (k%32)//8,
    # nibble position (t>>1) + 4*(t&1) with t = k % 8
    k, n = 45, 7
    unit = nat.view("<u4").reshape(rows // 32, columns, 4)[k // 32, n]
    t = k % 8
    assert (int(unit[(k % 32) // 8]) >> (4 * ((t >> 1) + 4 * (t & 1)))) & 15 == q[n, k]


# ---------------------------------------------------------------------------------------------
# dequantize + GEMM
# ---------------------------------------------------------------------------------------------

def test_dequantize_inverts_kat(oracle):
    for bs, cw in [(16, True), (32, True), (64, True), (32, False)]:
        for has_offsets in (True, False):
            kat = oracle.kat_generate(bs, cw, 128, 64, has_offsets)
            b = oracle.dequantize(bs, cw, kat["canon_w"], kat["scales"], kat["zps"] if has_offsets else None)
            assert np.array_equal(b.view(np.uint16), kat["weights"].view(np.uint16))


def test_gemm_against_float64(oracle):
    rng = np.random.default_rng(1)
    m, n, k = 37, 48, 192
    a = rng.standard_normal((m, k)).astype(np.float16)
    b = (rng.standard_normal((n, k)) * 0.05).astype(np.float16)
    ref = a.astype(np.float64) @ b.astype(np.float64).T
    for strict in (True, False):
        c = oracle.gemm(a, b, strict_order=strict).astype(np.float64)
        # fp32 accumulation + one fp16 rounding: error bounded by half an fp16 ulp plus fp32 noise
        assert np.max(np.abs(c - ref) / np.maximum(np.abs(ref), 1e-2)) < 2e-3
    # a transposed operand or a dropped k would not survive this: exact small-integer case
    a = rng.integers(-4, 5, (5, 64)).astype(np.float16)
    b = rng.integers(-8, 8, (7, 64)).astype(np.float16)
    ref = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal(oracle.gemm(a, b, strict_order=True).astype(np.int64), ref)
    assert np.array_equal(oracle.gemm(a, b, strict_order=False).astype(np.int64), ref)


def test_kat_gemm_is_exact_in_any_order(oracle):
    """reference: test/blkq4_fp16_gemm_sm80_test.cu:194-199,469-472 -- with activations on the 0.25
    grid in [-4, 4] every partial sum is exact in fp32, so the result does not depend on the order."""
    rng = np.random.default_rng(2)
    kat = oracle.kat_generate(32, True, 192, 96, True)
    a = (rng.integers(-16, 17, (32, 192)) / 4.0).astype(np.float16)
    c1 = oracle.gemm(a, kat["weights"], strict_order=True)
    c2 = oracle.gemm(a, kat["weights"], strict_order=False)
    ref = a.astype(np.float64) @ kat["weights"].astype(np.float64).T
    assert np.array_equal(c1.view(np.uint16), c2.view(np.uint16))
    assert np.array_equal(c1.view(np.uint16), ref.astype(np.float16).view(np.uint16))
