"""Host-side behaviour of the C ABI that needs no GPU: exported symbols, the size query and every
validation message (reference: src/blkq4_f16_gemm_sm80.cu:77-134,164-198,251-280,425-428,459-462).
No call here reaches a kernel launch: each one fails in validation first."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(capi):
    header = open(os.path.join(ROOT, "include", "ms_blkq4gemm.h")).read()
    body = re.sub(r"/\*.*?\*/", "", header, flags=re.S)  # declarations only, comments dropped
    declared = set(re.findall(r"\b(blkq4_\w+)\s*\(", body))
    assert declared == set(capi.EXPORTED_SYMBOLS)
    lib = capi.load()
    for sym in declared:
        assert getattr(lib, sym) is not None


def test_reference_entry_points_keep_their_signatures():
    """the three reference entry points, token for token (reference: include/ms_blkq4gemm.h:41-50,71-80,94-100)."""
    norm = lambda s: re.sub(r"\s+", " ", s)
    header = norm(open(os.path.join(ROOT, "include", "ms_blkq4gemm.h")).read())
    assert norm("""int blkq4_fp16_gemm_sm80( int block_size, bool column_wise_blocking, int m, int n, int k, void* stream,
        void const* act_ptr, size_t a_size, void const* weights_ptr, size_t weights_size, void const* scales_ptr,
        size_t scales_size, void const* offsets_ptr, size_t offsets_size, void* output_ptr, size_t output_size,
        void* error_message);""") in header
    assert norm("""int blkq4_fp16_quant_sm80( int block_size, bool column_wise_blocking, int rows, int columns,
        int leadingDimension, void* stream, void const* weights, size_t weights_size, void* quant_weights,
        size_t quant_weights_size, void* quant_scales, size_t quant_scales_size, void* offsets, size_t offsets_size,
        void* error_message);""") in header
    assert norm("""int blkq4_fp16_quant_size_sm80( int block_size, bool column_wise_blocking, int rows, int columns,
        int64_t& quant_weights_size, int64_t& quant_meta_size, void* error_message);""") in header


@pytest.mark.parametrize("bs,col,rows,cols,w,meta", [
    (32, True, 1024, 1024, 524288, 32768),        # C1
    (64, True, 4096, 4096, 8388608, 262144),      # C2 / C4
    (32, True, 4096, 11008, 22544384, 1409024),   # C3
    (16, True, 8192, 28672, 117440512, 14680064), # C5
    (32, False, 64, 32, 1024, 64),                # row-wise: meta [K, N/bs]
    (16, False, 256, 256, 32768, 4096),
])
def test_quant_size_closed_form(capi, oracle, bs, col, rows, cols, w, meta):
    assert capi.quant_size(bs, col, rows, cols) == (w, meta)
    assert oracle.quant_size(bs, col, rows, cols) == (0, w, meta)


@pytest.mark.parametrize("args,message", [
    ((48, True, 64, 32), "Unsupported block size: 48"),
    ((0, True, 64, 32), "Unsupported block size: 0"),
    ((32, True, 0, 32), "Empty problem size: 0x32"),
    ((32, True, 64, 0), "Empty problem size: 64x0"),
    ((32, True, 96, 32), "Cannot block quantize matrix with rows: 96"),
    ((64, True, 32, 32), "Cannot block quantize matrix with rows: 32"),
    ((32, True, 64, 48), "Cannot block quantize matrix with columns: 48"),
    ((64, False, 64, 32), "Cannot block quantize matrix with columns: 32"),  # fewer columns than one block
    # a multiple of 32 that is no whole number of blocks (the reference's `columns % meta columns` lets it through)
    ((64, False, 64, 96), "Cannot block quantize matrix with columns: 96"),
    ((64, False, 128, 160), "Cannot block quantize matrix with columns: 160"),
])
def test_quant_size_errors(capi, args, message):
    with pytest.raises(capi.Blkq4Error) as e:
        capi.quant_size(*args)
    assert str(e.value) == message


def test_quant_size_zeroes_outputs_and_accepts_null_message(capi):
    lib = capi.load()
    w, m = ctypes.c_int64(123), ctypes.c_int64(456)
    assert lib.blkq4_fp16_quant_size_sm80(32, True, 96, 32, ctypes.byref(w), ctypes.byref(m), None) == -1
    assert (w.value, m.value) == (0, 0)


def _buf(nbytes, address=0x1000):
    from gemmlib_amd.capi import RawBuffer
    return RawBuffer(address, nbytes)


def _gemm(capi, bs=32, col=True, m=4, n=64, k=64, a=None, w=None, s=None, z=None, c=None, bias=None):
    a = _buf(m * k * 2) if a is None else a
    w = _buf(k * n // 2) if w is None else w
    s = _buf((k // bs) * n * 2) if s is None else s
    c = _buf(m * n * 2) if c is None else c
    capi.gemm(bs, col, m, n, k, a, w, s, z, c, stream=0, bias=bias)


@pytest.mark.parametrize("kwargs,message", [
    (dict(bs=8), "Unsupported block size: 8"),
    (dict(m=0), "Empty problem size: 0x64x64"),
    (dict(n=0), "Empty problem size: 4x0x64"),
    (dict(a=_buf(10)), "Unexpected activation tensor size: 10 expected: 512"),
    (dict(w=_buf(2047)), "Unexpected weight tensor size: 2047 expected: 2048"),
    (dict(s=_buf(100)), "Unexpected scale tensor size: 100 expected: 256"),
    (dict(c=_buf(8)), "Unexpected output tensor size: 8 expected: 512"),
    (dict(z=_buf(127)), "Unexpected offsets tensor size: 127 expected: 128"),
    (dict(k=96, a=_buf(4 * 96 * 2), w=_buf(96 * 64 // 2), s=_buf(3 * 64 * 2)),
     "Kernel execution failed: Error Invalid Problem"),
    (dict(a=_buf(512, address=0x1002)), "Kernel execution failed: Error Misaligned Operand"),
    (dict(c=_buf(512, address=0x1008)), "Kernel execution failed: Error Misaligned Operand"),
    # scales and zero-points are copied four bytes at a time by the tile kernel: one rule for every m
    (dict(s=_buf(256, address=0x1002)), "Kernel execution failed: Error Misaligned Operand"),
    (dict(z=_buf(128, address=0x1001)), "Kernel execution failed: Error Misaligned Operand"),
    (dict(m=2048, z=_buf(128, address=0x1002)), "Kernel execution failed: Error Misaligned Operand"),
    # the entry point with a bias: its size and alignment, and the checks of the plain one in the same order
    (dict(bias=_buf(126)), "Unexpected bias tensor size: 126 expected: 128"),
    (dict(bias=_buf(128, address=0x1008)), "Kernel execution failed: Error Misaligned Operand"),
    (dict(bias=_buf(128), c=_buf(8)), "Unexpected output tensor size: 8 expected: 512"),
    (dict(bias=_buf(128), bs=8), "Unsupported block size: 8"),
    # blocks along N: the scales are fetched 16 bytes at a time; n must be a multiple of the block size
    (dict(col=False, s=_buf(64 * 2 * 2, address=0x1004)), "Kernel execution failed: Error Misaligned Operand"),
    (dict(col=False, bs=64, n=96, w=_buf(64 * 96 // 2), s=_buf(64 * 1 * 2), c=_buf(4 * 96 * 2)),
     "Kernel execution failed: Error Invalid Problem"),
])
def test_gemm_validation_messages(capi, kwargs, message):
    with pytest.raises(capi.Blkq4Error) as e:
        _gemm(capi, **kwargs)
    assert str(e.value) == message


def _quant(capi, bs=32, col=True, rows=64, cols=32, ld=None, src=None, qw=None, qs=None, qz=None):
    lib = capi.load()
    ld = rows if ld is None else ld
    src = _buf(cols * ld * 2) if src is None else src
    qw = _buf(rows * cols // 2) if qw is None else qw
    qs = _buf((rows // bs) * cols * 2) if qs is None else qs
    err = lib.blkq4_error_message_create()
    try:
        rc = lib.blkq4_fp16_quant_sm80(bs, col, rows, cols, ld, None, src.address, src.nbytes, qw.address, qw.nbytes,
                                       qs.address, qs.nbytes, None if qz is None else qz.address,
                                       0 if qz is None else qz.nbytes, err)
        return rc, lib.blkq4_error_message_cstr(err).decode()
    finally:
        lib.blkq4_error_message_destroy(err)


@pytest.mark.parametrize("kwargs,message", [
    (dict(bs=128), "Unsupported block size: 128"),
    (dict(rows=0), "Empty problem size: 0x32"),
    (dict(rows=100), "Cannot block quantize matrix with rows: 100"),
    (dict(cols=40), "Cannot block quantize matrix with columns: 40"),
    (dict(qw=_buf(1000)), "Unexpected quantized weight tensor size: 1000 expected: 1024"),
    (dict(qs=_buf(100)), "Unexpected scale tensor size: 50 expected: 64"),
    (dict(qz=_buf(63)), "Unexpected offset tensor size: 63 expected: 64"),
    (dict(src=_buf(64 * 32 * 2 - 2)), "Unexpected weight tensor size: 2047 expected: 2048"),
    (dict(ld=80, src=_buf(64 * 32 * 2)), "Unexpected weight tensor size: 2048 expected: 2560"),
    (dict(col=False, qs=_buf(60 * 2)), "Unexpected scale tensor size: 60 expected: 64"),   # row-wise meta is [K, N/bs]
])
def test_quant_validation_messages(capi, kwargs, message):
    rc, text = _quant(capi, **kwargs)
    assert rc == -1 and text == message


def test_repack_validation_messages(capi):
    cases = [
        (dict(rows=0, columns=32, src=_buf(0), dst=_buf(0, 0x9000)), "Empty problem size: 0x32"),
        (dict(rows=96, columns=32, src=_buf(1536), dst=_buf(1536, 0x9000)), "Cannot block quantize matrix with rows: 96"),
        (dict(rows=64, columns=32, src=_buf(1000), dst=_buf(1024, 0x9000)),
         "Unexpected quantized weight tensor size: 1000 expected: 1024"),
        (dict(rows=64, columns=32, src=_buf(1024), dst=_buf(1024, 0x1200)), "Source and destination buffers overlap"),
    ]
    for kwargs, message in cases:
        with pytest.raises(capi.Blkq4Error) as e:
            capi.repack(True, kwargs["rows"], kwargs["columns"], kwargs["src"], kwargs["dst"], stream=0)
        assert str(e.value) == message


def test_error_message_may_be_null(capi):
    lib = capi.load()
    assert lib.blkq4_fp16_gemm_sm80(32, True, 0, 64, 64, None, None, 0, None, 0, None, 0, None, 0, None, 0, None) == -1


@pytest.mark.parametrize("plan,message", [
    ("spiral 3", "Unknown plan: a plan is"),
    ("tile 4 2 1 4", "Unknown plan: a plan is"),
    ("tile 0 2 1 4 4 1 1", "Unknown plan: tile RT NT WM WN PW KW PARTS"),
    ("streaming 2 1 3 8 1 8", "Unknown plan: streaming DEPTH NT MT WAVES ROWS SPLIT"),
    ("streaming 2 1 1 8 1 4", "Unknown plan: streaming DEPTH NT MT WAVES ROWS SPLIT"),
    ("decode 32 1 8 4", "Unknown plan: decode ROWS NT WAVES DEPTH"),
    # plans that parse but name no kernel, or a kernel that does not fit the problem: refused by the launchers,
    # before anything is launched
    ("tile 3 3 1 4 4 1 1", "Kernel execution failed: invalid argument"),
    ("tile 4 1 1 1 4 2 1", "Kernel execution failed: invalid argument"),
    ("streaming 3 1 1 8 1 8", "Kernel execution failed: invalid argument"),
    ("decode 1 1 8 4", "Kernel execution failed: invalid argument"),     # 4 rows do not fit a kernel that keeps 1
    ("decode 4 1 8 4", "Kernel execution failed: invalid argument"),     # K = 512 is 4 slices, not 32
])
def test_plans_given_as_text_are_checked(capi, plan, message):
    """blkq4_gemm_with_plan_sm80: what is no plan is refused by the parser, what is no kernel by the launchers."""
    m, n, k, bs = 4, 64, 512, 32
    with pytest.raises(capi.Blkq4Error) as e:
        capi.gemm_with_plan(plan, bs, True, m, n, k, _buf(m * k * 2), _buf(k * n // 2), _buf((k // bs) * n * 2), None,
                            _buf(m * n * 2), stream=0)
    assert str(e.value).startswith(message), str(e.value)


def test_plan_entry_point_validates_like_the_gemm(capi):
    with pytest.raises(capi.Blkq4Error, match="Unexpected activation tensor size: 10 expected: 4096"):
        capi.gemm_with_plan("auto", 32, True, 4, 64, 512, _buf(10), _buf(512 * 32), _buf(16 * 64 * 2), None, _buf(512), stream=0)
