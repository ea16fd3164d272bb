"""The tile kernel with split tiles (fp32 partial tiles in the library's workspace, summed in a fixed order by the
workgroup that arrives last), through the C ABI, against the oracle: the reference's exact construction bit for
bit (test/blkq4_fp16_gemm_sm80_test.cu:194-256,469-472), Gaussian data within 1e-2, every call of a shape the
same bits, and the same bits when the call is recorded into a graph on a stream of its own."""

import numpy as np
import pytest
import torch

from gpu_util import gemm_on_gpu, max_rel_err, quantize_on_gpu, to_dev, to_np
from test_gpu_gemm import grid_activations, gaussian_problem

pytestmark = pytest.mark.gpu

# (block_size, column_wise, has_offsets, m, n, k, tile the plan must name, parts)
SPLIT_CASES = [
    (64, True, True, 100, 5120, 5120, "64 x 128", 3),
    (32, True, False, 256, 3072, 4096, "64 x 128", 2),
    (64, True, True, 200, 5120, 8192, "128 x 128", 3),
    (16, True, True, 65, 8192, 8192, "128 x 128", 4),
    (64, True, False, 300, 28672, 8192, "128 x 256", 3),
    (64, True, True, 1280, 14336, 8192, "128 x 256", 4),
    (64, False, True, 200, 5120, 8192, "128 x 128", 3),
    (32, False, False, 100, 5120, 5120, "64 x 128", 3),
    # 33 to 64 rows: every 64 x 128 tile in parts, where the kernel would otherwise stream the weights
    (64, True, True, 64, 5120, 5120, "64 x 128", 4),
    (32, True, False, 40, 13824, 5120, "64 x 128", 2),
]


def _assert_split_plan(capi, bs, col, m, n, k, tile, parts, bf16=False):
    text = capi.gemm_plan(bs, col, m, n, k, bf16=bf16)[2]
    assert text.startswith(f"tile: {tile},") and f" in {parts} parts" in text, text


@pytest.mark.parametrize("bs,col,has_offsets,m,n,k,tile,parts", SPLIT_CASES)
def test_split_tiles_exact_on_reference_construction(oracle, capi, device, bs, col, has_offsets, m, n, k, tile, parts):
    _assert_split_plan(capi, bs, col, m, n, k, tile, parts)
    rng = np.random.default_rng(m + n + k)
    kat = oracle.kat_generate(bs, col, k, n, has_offsets)
    a = grid_activations(rng, m, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, kat["weights"], has_offsets, column_wise=col)
    assert np.array_equal(to_np(q_w), oracle.native_from_canonical(kat["canon_w"]))
    ref = oracle.gemm(a, kat["weights"])
    for call in range(3):  # the workspace and its counters are used again by every call
        got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=col)
        bad = np.argwhere(got.view(np.uint16) != ref.view(np.uint16))
        assert bad.shape[0] == 0, f"call {call}: {bad.shape[0]} of {m * n} outputs differ, first {bad[:5].tolist()}"


@pytest.mark.parametrize("bs,col,has_offsets,m,n,k,tile,parts", SPLIT_CASES[:6:2] + SPLIT_CASES[6:7] + SPLIT_CASES[8:9])
def test_split_tiles_gaussian_deterministic_and_with_bias(oracle, capi, device, bs, col, has_offsets, m, n, k, tile, parts):
    a, w = gaussian_problem(7 * m + n + k, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, has_offsets, column_wise=col)
    canon, s, z = oracle.quantize(bs, col, w, has_offsets)
    b = oracle.dequantize(bs, col, canon, s, z)
    rows = np.unique(np.linspace(0, m - 1, 24).astype(np.int64))
    ref = oracle.gemm(np.ascontiguousarray(a[rows]), b)
    got = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=col)
    assert max_rel_err(got[rows], ref) <= 1e-2
    # the parts are added in a fixed order, whichever workgroup arrives last: every call gives the same bits
    for _ in range(4):
        again = gemm_on_gpu(capi, device, bs, a, q_w, q_s, q_zp, n, column_wise=col)
        assert np.array_equal(again.view(np.uint16), got.view(np.uint16))
    # bias in the epilogue of the workgroup that finishes the tile: fp16 result + fp16 bias, rounded again
    bias = torch.randn(n, generator=torch.Generator().manual_seed(3)).to(torch.float16)
    out = torch.empty(m, n, dtype=torch.float16, device=device)
    capi.gemm(bs, col, m, n, k, to_dev(a, device), q_w, q_s, q_zp, out, bias=bias.to(device))
    torch.cuda.synchronize()
    want = (torch.from_numpy(got.view(np.int16).copy()).view(torch.float16) + bias).view(torch.int16).numpy()
    assert np.array_equal(out.cpu().view(torch.int16).numpy(), want)


def test_split_tiles_bf16(oracle, capi, device):
    def bf16_bits(t):
        return t.contiguous().view(torch.int16).numpy().view(np.uint16)

    bs, m, n, k = 64, 200, 5120, 8192
    _assert_split_plan(capi, bs, True, m, n, k, "128 x 128", 3, bf16=True)
    g = torch.Generator(device="cpu").manual_seed(21)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
    w_elems, meta = capi.quant_size(bs, True, k, n)
    q_w = torch.empty(w_elems, dtype=torch.uint8, device=device)
    q_s = torch.empty(meta, dtype=torch.bfloat16, device=device)
    q_z = torch.empty(meta, dtype=torch.uint8, device=device)
    capi.quant(bs, True, w.to(device), q_w, q_s, q_z, bf16=True)
    out = torch.empty(m, n, dtype=torch.bfloat16, device=device)
    capi.gemm(bs, True, m, n, k, a.to(device), q_w, q_s, q_z, out, bf16=True)
    torch.cuda.synchronize()
    canon, s, z = oracle.quantize(bs, True, bf16_bits(w), True, bf16=True)
    b = oracle.dequantize(bs, True, canon, s, z, bf16=True)
    rows = np.arange(0, m, 9)
    ref = oracle.bf16_to_f32(oracle.gemm(np.ascontiguousarray(bf16_bits(a)[rows]), b, bf16=True))
    got = oracle.bf16_to_f32(bf16_bits(out.cpu())[rows])
    assert max_rel_err(got, ref) <= 1e-2


def test_split_tiles_recorded_on_a_stream_of_their_own_and_on_two_streams_at_once(capi, device):
    """a call recorded into a graph on a fresh stream gets that stream's workspace and gives the eager call's bits;
    two streams working at the same time do not share a workspace"""
    bs, m, n, k = 64, 200, 5120, 8192
    _assert_split_plan(capi, bs, True, m, n, k, "128 x 128", 3)
    a, w = gaussian_problem(99, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True)
    a_dev = to_dev(a, device)
    eager = torch.empty(m, n, dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, eager)
    torch.cuda.synchronize()
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {replay}"
    # two streams, many calls in flight on both
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    o1 = torch.empty_like(eager)
    o2 = torch.empty_like(eager)
    torch.cuda.synchronize()
    for _ in range(10):
        with torch.cuda.stream(s1):
            capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, o1)
        with torch.cuda.stream(s2):
            capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, o2)
    torch.cuda.synchronize()
    assert torch.equal(o1.view(torch.int16), eager.view(torch.int16))
    assert torch.equal(o2.view(torch.int16), eager.view(torch.int16))


def test_a_recording_has_a_workspace_of_its_own_and_the_thread_stream_has_none(oracle, capi, device):
    """Which calls share a workspace (the promises of the public header): eager calls on a stream share one; a
    recording on that same stream gets another, so the graph may run on any stream while the recording stream
    works eagerly; a second recording gets a third; hipStreamPerThread gets none and runs the unsplit plan."""
    bs, m, n, k = 64, 200, 5120, 8192
    _assert_split_plan(capi, bs, True, m, n, k, "128 x 128", 3)
    a, w = gaussian_problem(123, m, n, k)
    a2, _ = gaussian_problem(124, m, n, k)
    q_w, q_s, q_zp = quantize_on_gpu(capi, device, bs, w, True)
    a_dev, a2_dev = to_dev(a, device), to_dev(a2, device)
    want = torch.empty(m, n, dtype=torch.float16, device=device)
    want2 = torch.empty_like(want)
    s, t = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(s):
        capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, want)
        capi.gemm(bs, True, m, n, k, a2_dev, q_w, q_s, q_zp, want2)
    torch.cuda.synchronize()
    state, in_use, most, nbytes = capi.workspace_info(s)
    assert state == 1 and 1 <= in_use <= most == 32 and nbytes == (32 << 20) + (16 << 10)
    graphs, outs = [], []
    for i in range(2):
        out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(s):
            with torch.cuda.graph(g, stream=s):
                before = capi.workspace_info(s)
                capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out)
                after = capi.workspace_info(s)
        assert before[0] == 0 and after[0] == 1 and after[1] == before[1] + 1, (before, after)
        graphs.append(g)
        outs.append(out)
    assert capi.workspace_info(s)[:2] == (1, in_use + 2)   # eager calls on s still have theirs
    # both graphs on t and on the legacy stream while s works eagerly on other data
    eager_out = torch.empty_like(want)
    for rep in range(5):
        with torch.cuda.stream(t):
            graphs[0].replay()
        graphs[1].replay()
        with torch.cuda.stream(s):
            capi.gemm(bs, True, m, n, k, a2_dev, q_w, q_s, q_zp, eager_out)
        torch.cuda.synchronize()
        for out in outs:
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), rep
            out.fill_(float("nan"))
        assert torch.equal(eager_out.view(torch.int16), want2.view(torch.int16)), rep
    # hipStreamPerThread (the handle 2): no workspace, the plan that needs none, same result within tolerance
    assert capi.workspace_info(2)[0] == -1
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(bs, True, m, n, k, a_dev, q_w, q_s, q_zp, out, stream=2)
    torch.cuda.synchronize()
    assert capi.workspace_info(2)[:2] == (-1, in_use + 2)
    assert max_rel_err(to_np(out), to_np(want)) <= 1e-2 and not torch.isnan(out).any()
    canon, sc, z = oracle.quantize(bs, True, w, True)
    rows = np.arange(0, m, 25)
    ref = oracle.gemm(np.ascontiguousarray(a[rows]), oracle.dequantize(bs, True, canon, sc, z))
    assert max_rel_err(to_np(out)[rows], ref) <= 1e-2
