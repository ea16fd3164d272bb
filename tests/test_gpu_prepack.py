"""GPU parity of the fused quantize+pack kernel and of the layout conversion, through the C ABI.

Bar: bit-exact.  scales and zero-points are compared byte for byte with the buffers the reference's
quantize entry point returns (oracle.quant_sm80); the packed weights are compared (a) in the library's
own order with the oracle's restatement of that order and (b) after blkq4_fp16_repack_sm80 with the
reference's sm80 buffer, byte for byte.
"""

import hashlib
import json
import os

import numpy as np
import pytest
import torch

from gpu_util import quantize_on_gpu, to_dev, to_np

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KAT_SHAPES = [(64, 32), (64, 64), (64, 128), (64, 256), (128, 32), (256, 32), (256, 256)]


def digest(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:16]


def check_against_oracle(oracle, capi, device, bs, weights_nk, has_offsets, w_dev=None, column_wise=True):
    n, k = weights_nk.shape
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, weights_nk, has_offsets, w_dev, column_wise)
    canon, s, z = oracle.quantize(bs, column_wise, weights_nk, has_offsets)
    ps, pz = oracle.prepack_meta_sm80(bs, column_wise, k, n, s, z)
    got_s = to_np(q_s)
    assert np.array_equal(got_s.view(np.uint16), ps.view(np.uint16)), "scales differ"
    if has_offsets:
        assert np.array_equal(to_np(q_zp), pz), "zero-points differ"
    got_w = to_np(q_w)
    want_native = oracle.native_from_canonical(canon)
    if not np.array_equal(got_w, want_native):
        bad = np.nonzero(got_w != want_native)[0]
        raise AssertionError(f"packed weights differ in {bad.size} bytes, first at {bad[:8]}")
    # conversion to the reference's byte order and back
    sm80 = torch.full_like(q_w, 0x5A)
    capi.repack(True, k, n, q_w, sm80)
    back = torch.full_like(q_w, 0x5A)
    capi.repack(False, k, n, sm80, back)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(sm80), oracle.prepack_weights_sm80(canon)), "sm80 export differs"
    assert torch.equal(back, q_w), "sm80 import does not invert the export"
    return to_np(sm80), got_s, (to_np(q_zp) if has_offsets else None), canon


@pytest.mark.parametrize("rows,columns", KAT_SHAPES)
@pytest.mark.parametrize("has_offsets", [True, False])
def test_reference_known_answers(oracle, capi, device, rows, columns, has_offsets):
    """reference: test/blkq4_fp16_quant_sm80_test.cu:336-347 (Colblock cases, block size 32)."""
    kat = oracle.kat_generate(32, True, rows, columns, has_offsets)
    sm80, s, z, canon = check_against_oracle(oracle, capi, device, 32, kat["weights"], has_offsets)
    # the quantizer returns the generator's nibbles, scales and zero-points exactly (:243-307)
    assert np.array_equal(canon, kat["canon_w"])
    assert np.array_equal(s.reshape(rows // 32, columns).view(np.uint16), kat["scales"].T.view(np.uint16))
    if has_offsets:
        assert np.array_equal(z.reshape(rows // 32, columns), kat["zps"].T)


def test_reference_known_answer_digests(oracle, capi, device):
    """both blockings (reference: test/blkq4_fp16_quant_sm80_test.cu:313-347)."""
    with open(os.path.join(GOLDEN, "kat_digests_independent.json")) as f:
        table = json.load(f)
    for case in table["cases"]:
        col = bool(case["column_wise"])
        kat = oracle.kat_generate(32, col, case["rows"], case["columns"], True)
        sm80, s, z, _ = check_against_oracle(oracle, capi, device, 32, kat["weights"], True, column_wise=col)
        assert digest(sm80) == case["packedW"]
        assert digest(s.view(np.uint16)) == case["packedS"]
        assert digest(z) == case["packedZ"]


@pytest.mark.parametrize("rows,columns", KAT_SHAPES)
@pytest.mark.parametrize("has_offsets", [True, False])
def test_reference_known_answers_rowwise(oracle, capi, device, rows, columns, has_offsets):
    """blocks of 1 x 32 along N (reference: test/blkq4_fp16_quant_sm80_test.cu:313-334)."""
    kat = oracle.kat_generate(32, False, rows, columns, has_offsets)
    _, _, _, canon = check_against_oracle(oracle, capi, device, 32, kat["weights"], has_offsets, column_wise=False)
    assert np.array_equal(canon, kat["canon_w"])


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("has_offsets", [True, False])
@pytest.mark.parametrize("rows,columns", [(64, 64), (192, 192), (320, 448), (1024, 1024)])
def test_gaussian_rowwise(oracle, capi, device, bs, has_offsets, rows, columns):
    rng = np.random.default_rng(bs * 104729 + rows * 31 + columns + has_offsets)
    w = (rng.standard_normal((columns, rows)) * 0.02).astype(np.float16)
    w[0, :] = 0.0                    # all-zero blocks, and blocks whose first weight is -0
    w[:, 3] = -0.0
    w[5, 7] = 0.0
    check_against_oracle(oracle, capi, device, bs, w, has_offsets, column_wise=False)


@pytest.mark.parametrize("bs", [16, 32, 64])
@pytest.mark.parametrize("has_offsets", [True, False])
@pytest.mark.parametrize("rows,columns", [(64, 32), (192, 96), (320, 160), (576, 672), (1024, 1024)])
def test_gaussian_and_ragged_shapes(oracle, capi, device, bs, has_offsets, rows, columns):
    """rows not a multiple of the 256-row tile, columns not a multiple of the 64-column tile."""
    rng = np.random.default_rng(bs * 7919 + rows * 31 + columns + has_offsets)
    w = (rng.standard_normal((columns, rows)) * 0.02).astype(np.float16)
    check_against_oracle(oracle, capi, device, bs, w, has_offsets)


@pytest.mark.parametrize("has_offsets", [True, False])
def test_special_values(oracle, capi, device, has_offsets):
    """all-zero blocks (+0 and -0), constant blocks, huge and tiny magnitudes, subnormals."""
    rng = np.random.default_rng(99)
    rows, columns, bs = 256, 64, 32
    w = (rng.standard_normal((columns, rows)) * 0.02).astype(np.float16)
    w[0, :32] = 0.0
    w[1, :32] = -0.0
    w[2, :32] = 0.0
    w[2, 5] = -0.0                      # mixed zeros: first element decides the sign of the symmetric scale
    w[3, 32:64] = 3.0
    w[4, 32:64] = -3.0
    w[5, :32] = (rng.standard_normal(32) * 3000).astype(np.float16)
    w[6, :32] = (rng.standard_normal(32) * 1e-6).astype(np.float16)   # subnormal fp16 inputs
    w[7, :32] = 65504.0
    w[7, 3] = -65504.0                  # tie between +max and -max
    w[8, 64:96] = np.float16(6e-8)
    check_against_oracle(oracle, capi, device, bs, w, has_offsets)


def test_leading_dimension_and_unaligned_source(oracle, capi, device):
    rng = np.random.default_rng(4)
    rows, columns, bs = 192, 64, 32
    for ld, shift in [(rows + 8, 0), (rows + 3, 0), (rows, 1), (rows + 5, 3)]:
        buf = (rng.standard_normal(columns * ld + 8) * 0.02).astype(np.float16)
        w = np.ascontiguousarray(buf[shift:shift + columns * ld].reshape(columns, ld)[:, :rows])
        dev_buf = to_dev(buf, device)
        view = dev_buf[shift:shift + columns * ld]
        w_elems, meta_elems = capi.quant_size(bs, True, rows, columns)
        q_w = torch.zeros(w_elems, dtype=torch.uint8, device=device)
        q_s = torch.zeros(meta_elems, dtype=torch.float16, device=device)
        q_zp = torch.zeros(meta_elems, dtype=torch.uint8, device=device)
        capi.quant(bs, True, view, q_w, q_s, q_zp, rows=rows, columns=columns, ld=ld)
        torch.cuda.synchronize()
        canon, s, z = oracle.quantize(bs, True, w, True)
        ps, pz = oracle.prepack_meta_sm80(bs, True, rows, columns, s, z)
        assert np.array_equal(to_np(q_w), oracle.native_from_canonical(canon)), (ld, shift)
        assert np.array_equal(to_np(q_s).view(np.uint16), ps.view(np.uint16)), (ld, shift)
        assert np.array_equal(to_np(q_zp), pz), (ld, shift)


CONFIG_SHAPES = {
    "C2_decode": (64, False, 4096, 4096),
    "C3_skinny": (32, True, 4096, 11008),
    "C4_prefill": (64, True, 4096, 4096),
    "C5_large": (16, True, 8192, 28672),
}


@pytest.mark.parametrize("name", list(CONFIG_SHAPES))
def test_benchmark_config_shapes(oracle, capi, device, name):
    """N(0, 0.02) weights at the full shapes of the benchmark configurations, every byte compared."""
    bs, has_offsets, rows, columns = CONFIG_SHAPES[name]
    g = torch.Generator(device="cpu").manual_seed(1234 + rows + columns)
    w_t = (torch.randn(columns, rows, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    w = w_t.view(torch.int16).numpy().view(np.float16)
    check_against_oracle(oracle, capi, device, bs, w, has_offsets)


def test_shortened_quantizer_arithmetic_equals_the_ieee_form_over_its_whole_domain(capi, device):
    """blkq4_fp16_quant_selfcheck_sm80: the fp16 quantizer's short division sequences and its one-instruction
    rounding against the IEEE forms of the reference's arithmetic (src/mickey/blk_q4/f16_quant_sm80.cuh:96-122,
    :291-298) for every range a block can have, every nonzero symmetric extreme and every float in [0, 15], on this GPU."""
    counts = torch.full((4,), -1, dtype=torch.int64, device=device)
    capi.quant_selfcheck(counts)
    torch.cuda.synchronize()
    asym, sym, rounding, cases = counts.cpu().tolist()
    assert (asym, sym, rounding) == (0, 0, 0)
    assert cases == 31745 * 31744 + (2 * 31744 - 2) + 0x41700000 + 1
    with pytest.raises(capi.Blkq4Error, match="Unexpected counter buffer"):
        capi.quant_selfcheck(counts[:3])
