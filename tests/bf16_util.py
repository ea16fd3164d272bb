"""Known-answer data for the bf16 entry points, in the manner of the reference's generator
(test/blkq4_fp16_quant_sm80_test.cu:53-112): quantized data first, the weights from it, built so that every
weight is exact in bf16 and the quantizer must give the quantized data back.  bf16 values travel as their bit
patterns in ``uint16`` arrays (numpy has no bf16 type)."""

import numpy as np


def bf16_kat(oracle, block_size, rows, columns, has_offsets, seed=0):
    """Blocks along K.  Scales m * 2^e with a 4-bit m, |q - zp| <= 15: the product has 8 significant bits, a
    bf16's worth.  Every block holds the nibbles 0 and 15, so its range is 15 scales wide (with offsets: scale
    and zero-point come back exactly) or its extreme is -8 scales (without).

    Returns ``canon_w`` uint8 ``[N, K/2]``, ``scales`` bf16 bits ``[N, K/bs]``, ``zps`` uint8 ``[N, K/bs]``,
    ``weights`` bf16 bits ``[N, K]`` and ``exact`` float64 ``[N, K]``."""
    rng = np.random.default_rng(seed)
    n, k, bs = columns, rows, block_size
    q = rng.integers(0, 16, (n, k // bs, bs)).astype(np.uint8)
    pos = rng.integers(0, bs, (n, k // bs))
    off = rng.integers(1, bs, (n, k // bs))
    ii, jj = np.meshgrid(np.arange(n), np.arange(k // bs), indexing="ij")
    q[ii, jj, pos] = 0
    q[ii, jj, (pos + off) % bs] = 15
    q = q.reshape(n, k)
    mant = rng.integers(1, 16, (n, k // bs)).astype(np.float64)
    expo = rng.integers(-5, -3, (n, k // bs)).astype(np.float64)   # 2^-5 or 2^-4: sums of products stay exact in fp32
    s64 = mant * 2.0 ** expo
    zps = rng.integers(0, 16, (n, k // bs)).astype(np.uint8)
    z_full = np.repeat(zps.astype(np.float64), bs, axis=1) if has_offsets else 8.0
    exact = np.repeat(s64, bs, axis=1) * (q.astype(np.float64) - z_full)
    weights = oracle.f32_to_bf16(exact.astype(np.float32))
    return {"canon_w": oracle.canonical_from_nibbles(q), "scales": oracle.f32_to_bf16(s64.astype(np.float32)),
            "zps": zps, "weights": np.ascontiguousarray(weights), "exact": exact}


def grid_activations_bf16(oracle, rng, m, k):
    """uniform on the 0.25 grid in [-4, 4] (test/blkq4_fp16_gemm_sm80_test.cu:194-199), exact in bf16"""
    return oracle.f32_to_bf16((rng.integers(-16, 17, (m, k)) / 4.0).astype(np.float32))
