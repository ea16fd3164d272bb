"""ctypes/numpy front end of the CPU oracle (``blkq4_oracle.c``) plus the reference's known-answer
generator.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the CPU-baseline leg of
the benchmark, never by the product package.

All arrays are numpy; fp16 data travels as ``np.float16`` and is handed to C as its ``uint16`` view.
Logical weight matrix ``W`` is ``[K, N]`` (``K`` = rows = in_features, ``N`` = columns = out_features)
and the fp16 source is the torch ``[N, K]`` contiguous array (element ``(k, n)`` at ``k + n * K``).
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libblkq4_oracle.so")


def build(force: bool = False) -> str:
    """Compile the C oracle next to its source (gcc via the Makefile in this directory)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-B", "-C", _HERE, "libblkq4_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i, i64p = ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_int64)
        L.oracle_quant_size.argtypes = [i, i, i, i, i64p, i64p]
        L.oracle_quantize.argtypes = [i, i, i, i, i, vp, vp, vp, vp, i]
        L.oracle_quantize_t.argtypes = [i, i, i, i, i, vp, vp, vp, vp, i, i]
        L.oracle_prepack_weights_sm80.argtypes = [i, i, vp, vp]
        L.oracle_prepack_meta_sm80.argtypes = [i, i, i, i, vp, vp, vp, vp]
        L.oracle_dequantize.argtypes = [i, i, i, i, vp, vp, vp, vp]
        L.oracle_dequantize_t.argtypes = [i, i, i, i, vp, vp, vp, vp, i]
        L.oracle_gemm.argtypes = [i, i, i, vp, vp, vp, i]
        L.oracle_gemm_t.argtypes = [i, i, i, vp, vp, vp, i, i]
        L.oracle_b2f.argtypes = [ctypes.c_uint16]
        L.oracle_b2f.restype = ctypes.c_float
        L.oracle_f2b.argtypes = [ctypes.c_float]
        L.oracle_f2b.restype = ctypes.c_uint16
        L.oracle_h2f.argtypes = [ctypes.c_uint16]
        L.oracle_h2f.restype = ctypes.c_float
        L.oracle_f2h.argtypes = [ctypes.c_float]
        L.oracle_f2h.restype = ctypes.c_uint16
        L.oracle_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def quant_size(block_size, column_wise, rows, columns):
    """Reference: src/blkq4_f16_gemm_sm80.cu:155-203.  Returns (err, weights_elems, meta_elems)."""
    w, m = ctypes.c_int64(0), ctypes.c_int64(0)
    err = lib().oracle_quant_size(block_size, int(column_wise), rows, columns, ctypes.byref(w), ctypes.byref(m))
    return err, w.value, m.value


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (``uint16``) -> float32 (a bf16 is the upper half of a binary32)."""
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns (``uint16``), round to nearest even, through the C oracle's scalar
    conversion's vector form (the same integer rule, restated in numpy; NaNs are quieted)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), r)


def _elem_dtype(bf16: bool):
    return np.uint16 if bf16 else np.float16


def quantize(block_size, column_wise, weights_nk: np.ndarray, has_offsets: bool, fused: bool = True,
             bf16: bool = False):
    """Canonical quantized form of the torch-layout ``[N, K]`` fp16 weights (``bf16=True``: the weights
    and the returned scales are bf16 bit patterns in ``uint16`` arrays).

    Reference: src/mickey/blk_q4/f16_quant_sm80.cuh:225-315.  Returns ``(canon_w, scales, zps)``:
    ``canon_w`` uint8 ``[N, K/2]`` (= col-major ``[K/2, N]``), ``scales`` fp16 ``[N/kCol, K/kRow]``
    (= col-major ``[K/kRow, N/kCol]``), ``zps`` uint8 of the same shape or ``None``.
    """
    assert weights_nk.dtype == _elem_dtype(bf16) and weights_nk.ndim == 2 and weights_nk.flags.c_contiguous
    n, k = weights_nk.shape
    err, wsz, msz = quant_size(block_size, column_wise, k, n)
    if err:
        raise ValueError(f"oracle_quant_size failed: {err}")
    krow, kcol = (block_size, 1) if column_wise else (1, block_size)
    canon_w = np.empty((n, k // 2), np.uint8)
    scales = np.empty((n // kcol, k // krow), _elem_dtype(bf16))
    zps = np.empty((n // kcol, k // krow), np.uint8) if has_offsets else None
    err = lib().oracle_quantize_t(block_size, int(column_wise), k, n, k, _p(weights_nk.view(np.uint16)),
                                  _p(canon_w), _p(scales.view(np.uint16)), _p(zps), int(fused), int(bf16))
    if err:
        raise ValueError(f"oracle_quantize failed: {err}")
    return canon_w, scales, zps


def prepack_weights_sm80(canon_w: np.ndarray) -> np.ndarray:
    """Reference: f16_quant_sm80.cuh:362-417 / test/blkq4_fp16_gemm_sm80.h:39-86.

    In: uint8 ``[N, K/2]``.  Out: flat uint8 buffer of ``K*N/2`` bytes = col-major ``uint8[K, N/2]``.
    """
    n, k2 = canon_w.shape
    out = np.empty(n * k2, np.uint8)
    err = lib().oracle_prepack_weights_sm80(k2 * 2, n, _p(np.ascontiguousarray(canon_w)), _p(out))
    if err:
        raise ValueError("oracle_prepack_weights_sm80 failed")
    return out


def prepack_meta_sm80(block_size, column_wise, rows, columns, scales, zps):
    """Reference: f16_quant_sm80.cuh:457-547 / test/blkq4_fp16_gemm_sm80.h:88-226.

    Returns flat ``(packed_scales fp16, packed_zps uint8|None)`` in the buffer order the reference's
    quantize entry point returns (col-wise blocking: row-major ``[K/bs, N]``).
    """
    ps = np.empty(scales.size, np.float16)
    pz = np.empty(zps.size, np.uint8) if zps is not None else None
    err = lib().oracle_prepack_meta_sm80(block_size, int(column_wise), rows, columns,
                                         _p(np.ascontiguousarray(scales).view(np.uint16)),
                                         _p(None if zps is None else np.ascontiguousarray(zps)),
                                         _p(ps.view(np.uint16)), _p(pz))
    if err:
        raise ValueError("oracle_prepack_meta_sm80 failed")
    return ps, pz


def quant_sm80(block_size, column_wise, weights_nk, has_offsets, fused=True):
    """What the reference's ``blkq4_fp16_quant_sm80`` hands back (src/blkq4_f16_gemm_sm80.cu:205-314):
    ``(packed_w bytes, packed_scales, packed_zps|None)``."""
    n, k = weights_nk.shape
    cw, s, z = quantize(block_size, column_wise, weights_nk, has_offsets, fused)
    ps, pz = prepack_meta_sm80(block_size, column_wise, k, n, s, z)
    return prepack_weights_sm80(cw), ps, pz


def dequantize(block_size, column_wise, canon_w, scales, zps, bf16: bool = False) -> np.ndarray:
    """Reference: test/blkq4_fp16_gemm_sm80_test.cu:309-328.  Returns fp16 ``[N, K]`` (= col-major ``[K, N]``);
    ``bf16=True``: scales in and weights out are bf16 bit patterns (``uint16``)."""
    n, k2 = canon_w.shape
    assert scales.dtype == _elem_dtype(bf16)
    b = np.empty((n, k2 * 2), _elem_dtype(bf16))
    lib().oracle_dequantize_t(block_size, int(column_wise), k2 * 2, n, _p(np.ascontiguousarray(canon_w)),
                              _p(np.ascontiguousarray(scales).view(np.uint16)),
                              _p(None if zps is None else np.ascontiguousarray(zps)), _p(b.view(np.uint16)),
                              int(bf16))
    return b


def gemm(a_mk: np.ndarray, b_nk: np.ndarray, strict_order: bool = False, bf16: bool = False) -> np.ndarray:
    """fp16 ``C[M,N] = A[M,K] . B[K,N]`` with fp32 accumulation and one rounding to fp16 (``bf16=True``:
    all three matrices are bf16 bit patterns in ``uint16`` arrays).

    Reference: test/blkq4_fp16_gemm_sm80_test.cu:54-107,445-459.  ``b_nk`` is the ``[N, K]`` array
    :func:`dequantize` returns.
    """
    assert a_mk.dtype == _elem_dtype(bf16) and b_nk.dtype == _elem_dtype(bf16)
    m, k = a_mk.shape
    n, k2 = b_nk.shape
    assert k == k2
    c = np.empty((m, n), _elem_dtype(bf16))
    err = lib().oracle_gemm_t(m, n, k, _p(np.ascontiguousarray(a_mk).view(np.uint16)),
                              _p(np.ascontiguousarray(b_nk).view(np.uint16)), _p(c.view(np.uint16)),
                              int(strict_order), int(bf16))
    if err:
        raise MemoryError("oracle_gemm")
    return c


# -------------------------------------------------------------------------------------------------
# The library's own gfx950 weight layout, restated independently of the HIP code (numpy, from the
# layout's definition) so the kernels' packing can be checked:
#
#   native_w : uint8[K/32][N][16].  The 16-byte unit (ks, n) holds the 32 weights k = 32*ks .. +31 of
#   column n as four little-endian 32-bit words; word j holds k0 = 32*ks + 8*j .. +7 with weight
#   k0 + t stored in nibble position p(t) = (t >> 1) + 4 * (t & 1)   (so the nibbles of a word read
#   k0, k0+2, k0+4, k0+6, k0+1, k0+3, k0+5, k0+7 from the least significant end).
# -------------------------------------------------------------------------------------------------

_NIBBLE_POS = [(t >> 1) + 4 * (t & 1) for t in range(8)]


def nibbles_from_canonical(canon_w: np.ndarray) -> np.ndarray:
    """uint8 ``[N, K/2]`` -> uint8 ``[N, K]`` of values 0..15 (low nibble is the even k, f16_quant_sm80.cuh:312)."""
    n, k2 = canon_w.shape
    q = np.empty((n, k2 * 2), np.uint8)
    q[:, 0::2] = canon_w & 0x0F
    q[:, 1::2] = canon_w >> 4
    return q


def canonical_from_nibbles(q_nk: np.ndarray) -> np.ndarray:
    return (q_nk[:, 0::2] | (q_nk[:, 1::2] << 4)).astype(np.uint8)


def native_from_canonical(canon_w: np.ndarray) -> np.ndarray:
    """Canonical uint8 ``[N, K/2]`` -> flat native buffer (``K*N/2`` bytes)."""
    q = nibbles_from_canonical(canon_w).astype(np.uint32)  # [N, K]
    n, k = q.shape
    q = q.reshape(n, k // 32, 4, 8)
    words = np.zeros((n, k // 32, 4), np.uint32)
    for t in range(8):
        words |= q[..., t] << np.uint32(4 * _NIBBLE_POS[t])
    words = np.ascontiguousarray(words.transpose(1, 0, 2))  # [K/32, N, 4]
    return words.astype("<u4").view(np.uint8).reshape(-1)


def canonical_from_native(native_w: np.ndarray, rows: int, columns: int) -> np.ndarray:
    words = native_w.view("<u4").reshape(rows // 32, columns, 4).astype(np.uint32)
    q = np.empty((rows // 32, columns, 4, 8), np.uint8)
    for t in range(8):
        q[..., t] = (words >> np.uint32(4 * _NIBBLE_POS[t])) & 0xF
    q = q.transpose(1, 0, 2, 3).reshape(columns, rows)
    return canonical_from_nibbles(q)


# -------------------------------------------------------------------------------------------------
# The reference's deterministic known-answer generator.
# Reference: test/blkq4_fp16_quant_sm80_test.cu:72-112,165-186 and
# test/blkq4_fp16_gemm_sm80_test.cu:225-256,309-328 (the same construction in both).
# -------------------------------------------------------------------------------------------------

def _next_i4(v: int) -> int:
    v = (v + 5) % 16
    if v in (11, 7, 3):
        v = (v + 5) % 16
    return v


def kat_generate(block_size: int, column_wise: bool, rows: int, columns: int, has_offsets: bool):
    """Quantized data first, dequantized weights second (quant test :53-68).

    Returns a dict with ``canon_w`` uint8 ``[N, K/2]``, ``scales`` fp16 / ``zps`` uint8 in the
    canonical col-major meta order ``[N/kCol, K/kRow]`` (``zps`` always generated, as the reference
    does, but dequantization uses 8 when ``has_offsets`` is false), and ``weights`` fp16 ``[N, K]``.
    """
    krow, kcol = (block_size, 1) if column_wise else (1, block_size)
    k2 = rows // 2
    total = k2 * columns * 2
    # nibble stream: seed 7, then the 13-cycle the update rule falls into
    stream = np.empty(total + 1, np.uint8)
    v = 7
    # the rule is a pure function of v: walk until the cycle closes, then tile
    seq = []
    for _ in range(32):
        seq.append(v)
        v = _next_i4(v)
    # seq[0] = 7 is transient; seq[1:14] is the cycle
    cyc = np.array(seq[1:14], np.uint8)
    assert _next_i4(int(cyc[-1])) == int(cyc[0])
    stream[0] = 7
    reps = (total + 13) // 13 + 1
    stream[1:] = np.tile(cyc, reps)[:total]
    nib = stream[:total].reshape(columns, k2, 2)  # c outer, r inner, (v0, v1)
    canon_w = (nib[..., 0] | (nib[..., 1] << 4)).astype(np.uint8)
    v = int(stream[total])  # generator state after the weights

    meta_rows, meta_cols = rows // krow, columns // kcol
    scales = np.empty((meta_cols, meta_rows), np.float16)
    zps = np.empty((meta_cols, meta_rows), np.uint8)
    for col in range(meta_cols):
        for row in range(meta_rows):
            f = ((col * v + row + v // 3) % 63) + 1
            v += 41
            m = col * v + row + v * 3
            scales[col, row] = np.float16(f / float(1 << (4 + (m % 2))))
            zps[col, row] = ((f + m + v) % 8) + 4

    # dequantize: fp16(scale * float(w - offset)); every value is exact in fp16 by construction
    q = nibbles_from_canonical(canon_w).astype(np.int32)  # [N, K]
    s_full = np.repeat(np.repeat(scales.astype(np.float32), kcol, axis=0), krow, axis=1)
    z_full = np.repeat(np.repeat(zps.astype(np.int32), kcol, axis=0), krow, axis=1) if has_offsets else 8
    wf = s_full * (q - z_full).astype(np.float32)
    weights = wf.astype(np.float16)
    assert np.array_equal(weights.astype(np.float32), wf), "known-answer weights must be exact in fp16"
    return {"canon_w": canon_w, "scales": scales, "zps": zps, "weights": np.ascontiguousarray(weights)}
