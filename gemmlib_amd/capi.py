"""ctypes binding of the C ABI declared in ``include/ms_blkq4gemm.h``.

This is the thinnest possible host-side view of the library: plain pointers and byte sizes, exactly
what a C caller passes.  Device buffers come in as ``torch`` tensors only because torch is how this
repository allocates HBM; nothing here computes with torch.  There is no CPU fallback: if the
library is not built the import of the shared object fails loudly.
"""

from __future__ import annotations

import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libms_blkq4gemm.so")

EXPORTED_SYMBOLS = (
    "blkq4_fp16_gemm_sm80",
    "blkq4_fp16_gemm_bias_sm80",
    "blkq4_fp16_quant_sm80",
    "blkq4_fp16_quant_size_sm80",
    "blkq4_fp16_quant_selfcheck_sm80",
    "blkq4_fp16_repack_sm80",
    "blkq4_bf16_quant_sm80",
    "blkq4_bf16_gemm_sm80",
    "blkq4_gemm_plan_sm80",
    "blkq4_gemm_with_plan_sm80",
    "blkq4_fp16_gemm_noalloc_sm80",
    "blkq4_fp16_gemm_noalloc_init_sm80",
    "blkq4_gemm_workspace_info_sm80",
    "blkq4_gemm_workspace_release_sm80",
    "blkq4_fp16_gemv_valu_sm80",
    "blkq4_error_message_create",
    "blkq4_error_message_cstr",
    "blkq4_error_message_destroy",
)

_lib = None


class Blkq4Error(RuntimeError):
    """A C entry point returned -1; the message is the library's error string."""


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m gemmlib_amd.build` (there is no CPU fallback)")
    try:
        # torch ships its own HIP runtime with the same SONAME; loading torch first makes this library
        # bind to that copy instead of bringing a second runtime into the process.
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    vp, i, sz, b = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_bool
    i64p = ctypes.POINTER(ctypes.c_int64)
    L.blkq4_fp16_gemm_sm80.argtypes = [i, b, i, i, i, vp, vp, sz, vp, sz, vp, sz, vp, sz, vp, sz, vp]
    L.blkq4_fp16_gemm_sm80.restype = i
    L.blkq4_fp16_gemm_noalloc_sm80.argtypes = L.blkq4_fp16_gemm_sm80.argtypes
    L.blkq4_fp16_gemm_noalloc_sm80.restype = i
    L.blkq4_fp16_gemv_valu_sm80.argtypes = L.blkq4_fp16_gemm_sm80.argtypes
    L.blkq4_fp16_gemv_valu_sm80.restype = i
    L.blkq4_fp16_gemm_bias_sm80.argtypes = [i, b, i, i, i, vp, vp, sz, vp, sz, vp, sz, vp, sz, vp, sz, vp, sz, vp]
    L.blkq4_fp16_gemm_bias_sm80.restype = i
    L.blkq4_fp16_quant_sm80.argtypes = [i, b, i, i, i, vp, vp, sz, vp, sz, vp, sz, vp, sz, vp]
    L.blkq4_fp16_quant_sm80.restype = i
    # `int64_t&` is a pointer at the ABI level
    L.blkq4_fp16_quant_size_sm80.argtypes = [i, b, i, i, i64p, i64p, vp]
    L.blkq4_fp16_quant_size_sm80.restype = i
    L.blkq4_fp16_quant_selfcheck_sm80.argtypes = [vp, vp, sz, vp]
    L.blkq4_fp16_quant_selfcheck_sm80.restype = i
    L.blkq4_fp16_repack_sm80.argtypes = [i, i, i, vp, vp, sz, vp, sz, vp]
    L.blkq4_fp16_repack_sm80.restype = i
    L.blkq4_bf16_quant_sm80.argtypes = L.blkq4_fp16_quant_sm80.argtypes
    L.blkq4_bf16_quant_sm80.restype = i
    L.blkq4_bf16_gemm_sm80.argtypes = L.blkq4_fp16_gemm_bias_sm80.argtypes
    L.blkq4_bf16_gemm_sm80.restype = i
    u64p = ctypes.POINTER(ctypes.c_uint64)
    L.blkq4_gemm_plan_sm80.argtypes = [i, b, b, b, i, i, i, u64p, u64p, ctypes.c_char_p, sz, vp]
    L.blkq4_gemm_plan_sm80.restype = i
    L.blkq4_fp16_gemm_noalloc_init_sm80.argtypes = [vp]
    L.blkq4_fp16_gemm_noalloc_init_sm80.restype = i
    ip = ctypes.POINTER(ctypes.c_int)
    L.blkq4_gemm_workspace_info_sm80.argtypes = [vp, ip, ip, ip, ctypes.POINTER(sz), vp]
    L.blkq4_gemm_workspace_info_sm80.restype = i
    L.blkq4_gemm_workspace_release_sm80.argtypes = [vp]
    L.blkq4_gemm_workspace_release_sm80.restype = i
    L.blkq4_gemm_with_plan_sm80.argtypes = [ctypes.c_char_p, i, b, b, i, i, i, vp, vp, sz, vp, sz, vp, sz, vp, sz, vp, sz, vp]
    L.blkq4_gemm_with_plan_sm80.restype = i
    L.blkq4_error_message_create.restype = vp
    L.blkq4_error_message_cstr.argtypes = [vp]
    L.blkq4_error_message_cstr.restype = ctypes.c_char_p
    L.blkq4_error_message_destroy.argtypes = [vp]
    _lib = L
    return L


class _ErrMsg:
    def __init__(self, L):
        self.L = L
        self.h = L.blkq4_error_message_create()

    def text(self) -> str:
        return self.L.blkq4_error_message_cstr(self.h).decode()

    def __del__(self):
        self.L.blkq4_error_message_destroy(self.h)


def _check(rc: int, err: _ErrMsg):
    if rc != 0:
        raise Blkq4Error(err.text())


def quant_size(block_size: int, column_wise: bool, rows: int, columns: int):
    """-> (quant_weights_elems, quant_meta_elems); raises :class:`Blkq4Error` on -1."""
    L = load()
    err = _ErrMsg(L)
    w, m = ctypes.c_int64(-1), ctypes.c_int64(-1)
    rc = L.blkq4_fp16_quant_size_sm80(block_size, column_wise, rows, columns, ctypes.byref(w), ctypes.byref(m), err.h)
    _check(rc, err)
    return w.value, m.value


class RawBuffer:
    """A bare (address, byte size) pair for callers that do not hold a torch tensor."""

    def __init__(self, address: int, nbytes: int):
        self.address, self.nbytes = address, nbytes


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, RawBuffer):
        return ctypes.c_void_p(t.address)
    return ctypes.c_void_p(t.data_ptr())


def _nbytes(t):
    if t is None:
        return 0
    if isinstance(t, RawBuffer):
        return t.nbytes
    return t.numel() * t.element_size()


def _stream_ptr(stream):
    """torch stream / raw hipStream_t integer / None (= torch's current stream when a GPU is present)."""
    if stream is None:
        import torch
        if not torch.cuda.is_available():
            return ctypes.c_void_p(0)
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(getattr(stream, "cuda_stream", stream))


def quant(block_size: int, column_wise: bool, weights_nk, q_weights, q_scales, q_zp=None, stream=None,
          rows=None, columns=None, ld=None, bf16=False):
    """``blkq4_fp16_quant_sm80`` on device tensors (``bf16=True``: ``blkq4_bf16_quant_sm80``).  ``weights_nk``
    is the torch ``[out, in]`` tensor (rows = in_features = ``weights_nk.shape[1]``)."""
    L = load()
    err = _ErrMsg(L)
    columns = weights_nk.shape[0] if columns is None else columns
    rows = weights_nk.shape[1] if rows is None else rows
    ld = weights_nk.stride(0) if ld is None else ld
    entry = L.blkq4_bf16_quant_sm80 if bf16 else L.blkq4_fp16_quant_sm80
    rc = entry(block_size, column_wise, rows, columns, ld, _stream_ptr(stream),
                                 _ptr(weights_nk), _nbytes(weights_nk), _ptr(q_weights), _nbytes(q_weights),
                                 _ptr(q_scales), _nbytes(q_scales), _ptr(q_zp), _nbytes(q_zp), err.h)
    _check(rc, err)


def gemm(block_size: int, column_wise: bool, m: int, n: int, k: int, a, q_weights, q_scales, q_zp, out,
         stream=None, bias=None, bf16=False, noalloc=False, valu=False):
    """``blkq4_fp16_gemm_sm80`` on device tensors; with ``bias`` (fp16 ``[n]``) ``blkq4_fp16_gemm_bias_sm80``;
    ``bf16=True``: ``blkq4_bf16_gemm_sm80`` (bias optional); ``noalloc=True``: ``blkq4_fp16_gemm_noalloc_sm80``;
    ``valu=True``: ``blkq4_fp16_gemv_valu_sm80``."""
    L = load()
    err = _ErrMsg(L)
    if noalloc or valu:
        assert bias is None and not bf16
        entry = L.blkq4_fp16_gemv_valu_sm80 if valu else L.blkq4_fp16_gemm_noalloc_sm80
        rc = entry(block_size, column_wise, m, n, k, _stream_ptr(stream), _ptr(a), _nbytes(a),
                                            _ptr(q_weights), _nbytes(q_weights), _ptr(q_scales), _nbytes(q_scales),
                                            _ptr(q_zp), _nbytes(q_zp), _ptr(out), _nbytes(out), err.h)
    elif bf16:
        rc = L.blkq4_bf16_gemm_sm80(block_size, column_wise, m, n, k, _stream_ptr(stream), _ptr(a), _nbytes(a),
                                    _ptr(q_weights), _nbytes(q_weights), _ptr(q_scales), _nbytes(q_scales),
                                    _ptr(q_zp), _nbytes(q_zp), _ptr(bias), _nbytes(bias), _ptr(out),
                                    _nbytes(out), err.h)
    elif bias is None:
        rc = L.blkq4_fp16_gemm_sm80(block_size, column_wise, m, n, k, _stream_ptr(stream), _ptr(a), _nbytes(a),
                                    _ptr(q_weights), _nbytes(q_weights), _ptr(q_scales), _nbytes(q_scales),
                                    _ptr(q_zp), _nbytes(q_zp), _ptr(out), _nbytes(out), err.h)
    else:
        rc = L.blkq4_fp16_gemm_bias_sm80(block_size, column_wise, m, n, k, _stream_ptr(stream), _ptr(a), _nbytes(a),
                                         _ptr(q_weights), _nbytes(q_weights), _ptr(q_scales), _nbytes(q_scales),
                                         _ptr(q_zp), _nbytes(q_zp), _ptr(bias), _nbytes(bias), _ptr(out),
                                         _nbytes(out), err.h)
    _check(rc, err)


def repack(to_sm80: bool, rows: int, columns: int, src, dst, stream=None):
    """``blkq4_fp16_repack_sm80`` on device tensors."""
    L = load()
    err = _ErrMsg(L)
    rc = L.blkq4_fp16_repack_sm80(int(to_sm80), rows, columns, _stream_ptr(stream), _ptr(src), _nbytes(src),
                                  _ptr(dst), _nbytes(dst), err.h)
    _check(rc, err)


def gemm_plan(block_size: int, column_wise: bool, m: int, n: int, k: int, has_offsets: bool = True, bf16: bool = False):
    """``blkq4_gemm_plan_sm80``: which kernel a GEMM of this shape runs, without running it (host-only).
    -> (chosen_id, launched_id, description)."""
    L = load()
    err = _ErrMsg(L)
    chosen, launched = ctypes.c_uint64(0), ctypes.c_uint64(0)
    text = ctypes.create_string_buffer(256)
    rc = L.blkq4_gemm_plan_sm80(block_size, column_wise, bf16, has_offsets, m, n, k, ctypes.byref(chosen),
                                ctypes.byref(launched), text, len(text), err.h)
    _check(rc, err)
    return chosen.value, launched.value, text.value.decode()


def noalloc_init():
    """``blkq4_fp16_gemm_noalloc_init_sm80`` on the current device."""
    L = load()
    err = _ErrMsg(L)
    _check(L.blkq4_fp16_gemm_noalloc_init_sm80(err.h), err)


def workspace_info(stream=None):
    """``blkq4_gemm_workspace_info_sm80`` -> (state, buffers_in_use, buffers_max, buffer_bytes); state 1: a GEMM
    with a split plan issued on ``stream`` now has a workspace, 0: it would allocate one, -1: it would run the plan
    that needs none."""
    L = load()
    err = _ErrMsg(L)
    state, in_use, most = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    nbytes = ctypes.c_size_t(0)
    rc = L.blkq4_gemm_workspace_info_sm80(_stream_ptr(stream), ctypes.byref(state), ctypes.byref(in_use),
                                          ctypes.byref(most), ctypes.byref(nbytes), err.h)
    _check(rc, err)
    return state.value, in_use.value, most.value, nbytes.value


def workspace_release():
    """``blkq4_gemm_workspace_release_sm80``: frees every workspace (nothing that uses one may be running, queued or
    replayed later)."""
    L = load()
    err = _ErrMsg(L)
    _check(L.blkq4_gemm_workspace_release_sm80(err.h), err)


def quant_selfcheck(counts, stream=None):
    """``blkq4_fp16_quant_selfcheck_sm80``: ``counts`` is a device tensor of four int64 (disagreements for asymmetric
    blocks, symmetric blocks, the rounding; cases looked at)."""
    L = load()
    err = _ErrMsg(L)
    _check(L.blkq4_fp16_quant_selfcheck_sm80(_stream_ptr(stream), _ptr(counts), _nbytes(counts), err.h), err)


def gemm_with_plan(plan: str, block_size: int, column_wise: bool, m: int, n: int, k: int, a, q_weights, q_scales, q_zp, out,
                   stream=None, bf16=False):
    """``blkq4_gemm_with_plan_sm80``: the GEMM with the kernel and its shape given as text (``"auto"``, ``"tile ..."``,
    ``"streaming ..."``, ``"decode ..."``) instead of the cost model's choice."""
    L = load()
    err = _ErrMsg(L)
    rc = L.blkq4_gemm_with_plan_sm80(plan.encode(), block_size, column_wise, bf16, m, n, k, _stream_ptr(stream), _ptr(a),
                                     _nbytes(a), _ptr(q_weights), _nbytes(q_weights), _ptr(q_scales), _nbytes(q_scales),
                                     _ptr(q_zp), _nbytes(q_zp), _ptr(out), _nbytes(out), err.h)
    _check(rc, err)
