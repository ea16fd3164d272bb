"""Known-answer data for the bf16 entry points, in the manner of the reference's generator
(test/blkq4_fp16_quant_sm80_test.cu:53-112): quantized data first, the weights from it, built so that every
weight is exact in bf16 and the quantizer must give the quantized data back.  bf16 values travel as their bit
patterns in ``uint16`` arrays (numpy has no bf16 type)."""

import numpy as np


def bf16_kat(oracle, block_size, rows, columns, has_offsets, seed=0, column_wise=True):
    """Scales m * 2^e with a 4-bit m, |q - zp| <= 15: the product has 8 significant bits, a bf16's worth.
    Every block (``block_size`` consecutive k of a column, or with ``column_wise=False`` consecutive columns of
    a k) holds the nibbles 0 and 15, so its range is 15 scales wide (with offsets: scale and zero-point come
    back exactly) or its extreme is -8 scales (without).

    Returns ``canon_w`` uint8 ``[N, K/2]``, ``scales`` bf16 bits and ``zps`` uint8 in the oracle's canonical
    order ``[N/kCol, K/kRow]``, ``weights`` bf16 bits ``[N, K]`` and ``exact`` float64 ``[N, K]``."""
    rng = np.random.default_rng(seed)
    bs = block_size
    # build with the blocked axis last, then put it where it belongs
    outer, blocks = (columns, rows // bs) if column_wise else (rows, columns // bs)
    q = rng.integers(0, 16, (outer, blocks, bs)).astype(np.uint8)
    pos = rng.integers(0, bs, (outer, blocks))
    off = rng.integers(1, bs, (outer, blocks))
    ii, jj = np.meshgrid(np.arange(outer), np.arange(blocks), indexing="ij")
    q[ii, jj, pos] = 0
    q[ii, jj, (pos + off) % bs] = 15
    mant = rng.integers(1, 16, (outer, blocks)).astype(np.float64)
    expo = rng.integers(-5, -3, (outer, blocks)).astype(np.float64)   # 2^-5 or 2^-4: sums of products stay exact in fp32
    s64 = mant * 2.0 ** expo
    zps = rng.integers(0, 16, (outer, blocks)).astype(np.uint8)
    z_full = zps.astype(np.float64)[:, :, None] if has_offsets else 8.0
    exact = (s64[:, :, None] * (q.astype(np.float64) - z_full)).reshape(outer, blocks * bs)
    q = q.reshape(outer, blocks * bs)
    if not column_wise:   # [K, N] -> [N, K]; meta [K, N/bs] -> [N/bs, K]
        q, exact, s64, zps = q.T, exact.T, s64.T, zps.T
    weights = oracle.f32_to_bf16(np.ascontiguousarray(exact).astype(np.float32))
    return {"canon_w": oracle.canonical_from_nibbles(np.ascontiguousarray(q)),
            "scales": oracle.f32_to_bf16(np.ascontiguousarray(s64).astype(np.float32)),
            "zps": np.ascontiguousarray(zps), "weights": np.ascontiguousarray(weights),
            "exact": np.ascontiguousarray(exact)}


def grid_activations_bf16(oracle, rng, m, k):
    """uniform on the 0.25 grid in [-4, 4] (test/blkq4_fp16_gemm_sm80_test.cu:194-199), exact in bf16"""
    return oracle.f32_to_bf16((rng.integers(-16, 17, (m, k)) / 4.0).astype(np.float32))
