"""The Python drop-in surface (ms_blkq4linear_ext + BlkQ4Linear) on the GPU, against the oracle.
Mirrors what the reference's usage script does (reference: python/blkq4linear_test.py:10-85) and then
goes further: it actually calls forward()."""

import numpy as np
import pytest
import torch

from gpu_util import max_rel_err, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mod():
    import ms_blkq4linear  # top-level, as a user of the reference imports it; fails loudly if the extension is not built
    return ms_blkq4linear


def test_quant_matches_known_answer(oracle, device, mod):
    """the reference script's construction: in=64, out=32, block 32 (here column-wise)."""
    import ms_blkq4linear_ext as ext
    kat = oracle.kat_generate(32, True, 64, 32, True)
    q_w, q_s, q_zp = ext.quant(32, True, True, to_dev(kat["weights"], device))
    assert q_w.dtype == torch.uint8 and q_w.dim() == 1 and q_w.numel() == 64 * 32 // 2
    assert q_s.dtype == torch.float16 and q_s.numel() == 2 * 32 and q_zp.dtype == torch.uint8
    assert np.array_equal(to_np(q_w), oracle.native_from_canonical(kat["canon_w"]))
    assert np.array_equal(to_np(q_s).reshape(2, 32).view(np.uint16), kat["scales"].T.view(np.uint16))
    assert np.array_equal(to_np(q_zp).reshape(2, 32), kat["zps"].T)


@pytest.mark.parametrize("scale_only", [False, True])
@pytest.mark.parametrize("m", [1, 16, 80])
def test_module_forward_with_bias(oracle, device, mod, scale_only, m):
    g = torch.Generator(device="cpu").manual_seed(3 + m)
    k, n, bs = 512, 384, 64
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.float16)
    bias = torch.randn(n, generator=g).to(torch.float16)
    x = torch.randn(m, k, generator=g).to(torch.float16)
    layer = mod.BlkQ4Linear(bs, True, scale_only, w.to(device), bias.to(device))
    assert layer.in_features == k and layer.out_features == n and layer.has_offsets == (not scale_only)
    if scale_only:
        assert layer.q_zp.numel() == 0 and layer.q_zp.device.type == "cuda"
    y = layer(x.to(device))
    assert y.shape == (m, n) and y.dtype == torch.float16
    w_np = w.view(torch.int16).numpy().view(np.float16)
    canon, s, z = oracle.quantize(bs, True, w_np, not scale_only)
    ref = oracle.gemm(x.view(torch.int16).numpy().view(np.float16), oracle.dequantize(bs, True, canon, s, z))
    ref = (torch.from_numpy(ref.view(np.int16)).view(torch.float16) + bias).view(torch.int16).numpy().view(np.float16)
    assert max_rel_err(to_np(y), ref) <= 1e-2


def test_extension_argument_checks(device, mod):
    import ms_blkq4linear_ext as ext
    w = torch.zeros(32, 64, dtype=torch.float16, device=device)
    with pytest.raises(RuntimeError, match="only supports float16 weights"):
        ext.quant(32, True, True, w.float())
    with pytest.raises(RuntimeError, match="only supports 2D tensors"):
        ext.quant(32, True, True, w.reshape(2, 16, 64))
    with pytest.raises(RuntimeError, match="only supports contiguous tensors"):
        ext.quant(32, True, True, torch.zeros(64, 64, dtype=torch.float16, device=device)[:, ::2])
    with pytest.raises(RuntimeError, match="only supports CUDA tensors"):
        ext.quant(32, True, True, w.cpu())
    with pytest.raises(RuntimeError, match="Unsupported block size: 48"):
        ext.quant(48, True, True, w)
    with pytest.raises(RuntimeError, match="Cannot block quantize matrix with rows: 96"):
        ext.quant(32, True, True, torch.zeros(32, 96, dtype=torch.float16, device=device))
    q_w, q_s, q_zp = ext.quant(32, True, True, w)
    with pytest.raises(RuntimeError, match="Activation shape is not compatible"):
        ext.forward(32, True, 64, 32, torch.zeros(4, 32, dtype=torch.float16, device=device), q_w, q_s, q_zp)
    with pytest.raises(RuntimeError, match="only supports float16 inputs"):
        ext.forward(32, True, 64, 32, torch.zeros(4, 64, device=device), q_w, q_s, q_zp)


@pytest.mark.parametrize("col_wise", [True, False])
def test_module_leading_dimensions_and_row_wise_blocks(oracle, device, mod, col_wise):
    """[batch, seq, in_features] inputs, and the layer with quantization blocks along out_features."""
    g = torch.Generator(device="cpu").manual_seed(11)
    k, n, bs = 256, 192, 32
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.float16)
    x = torch.randn(3, 5, k, generator=g).to(torch.float16)
    layer = mod.BlkQ4Linear(bs, col_wise, False, w.to(device))
    y = layer(x.to(device))
    assert y.shape == (3, 5, n)
    w_np = w.view(torch.int16).numpy().view(np.float16)
    canon, s, z = oracle.quantize(bs, col_wise, w_np, True)
    ref = oracle.gemm(x.reshape(15, k).view(torch.int16).numpy().view(np.float16), oracle.dequantize(bs, col_wise, canon, s, z))
    assert max_rel_err(to_np(y.reshape(15, n)), ref) <= 1e-2
    assert torch.equal(layer(x.to(device).reshape(15, k)), y.reshape(15, n))


def test_state_dict_round_trip_and_from_packed(device, mod):
    g = torch.Generator(device="cpu").manual_seed(12)
    k, n, bs = 128, 64, 64
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.float16).to(device)
    bias = torch.randn(n, generator=g).to(torch.float16).to(device)
    x = torch.randn(7, k, generator=g).to(torch.float16).to(device)
    layer = mod.BlkQ4Linear(bs, True, False, w, bias)
    state = layer.state_dict()
    assert {"q_weights", "q_scales", "q_zp", "bias"} <= set(state)
    # a layer quantized from different weights takes over the saved tensors
    other = mod.BlkQ4Linear(bs, True, False, torch.zeros_like(w), torch.zeros_like(bias))
    other.load_state_dict(state)
    assert torch.equal(other(x), layer(x))
    # the quantization parameters are part of the state: a mismatching layer refuses it
    with pytest.raises((ValueError, RuntimeError)):
        mod.BlkQ4Linear(32, True, False, torch.zeros_like(w)).load_state_dict(state)
    packed = mod.BlkQ4Linear.from_packed(bs, True, k, n, layer.q_weights, layer.q_scales, layer.q_zp, bias)
    assert torch.equal(packed(x), layer(x))
    with pytest.raises(ValueError):
        mod.BlkQ4Linear.from_packed(bs, True, k, n + 32, layer.q_weights, layer.q_scales, layer.q_zp)


def test_reference_usage_script_steps_with_plain_imports_then_forward(oracle, device):
    """What a user of the reference runs (reference: python/blkq4linear_test.py:5-85): plain ``import
    ms_blkq4linear``, in_features 64, out_features 32, blocks of 32 along out_features, weights built from the
    known-answer quantized data, ``BlkQ4Linear(block_size, col_wise, scale_only, weights)``; then the packed
    tensors are what the construction started from, and ``forward`` (which that script never calls) is exact."""
    import importlib
    ms_blkq4linear = importlib.import_module("ms_blkq4linear")
    ext = importlib.import_module("ms_blkq4linear_ext")
    assert "gemmlib_amd" not in ms_blkq4linear.__name__ and ext.__name__ == "ms_blkq4linear_ext"
    in_features, out_features, block_size, col_wise, scale_only = 64, 32, 32, False, False
    kat = oracle.kat_generate(block_size, col_wise, in_features, out_features, not scale_only)
    weights = to_dev(kat["weights"], device)
    layer = ms_blkq4linear.BlkQ4Linear(block_size, col_wise, scale_only, weights)
    assert np.array_equal(to_np(layer.q_weights), oracle.native_from_canonical(kat["canon_w"]))
    ps, pz = oracle.prepack_meta_sm80(block_size, col_wise, in_features, out_features, kat["scales"], kat["zps"])
    assert np.array_equal(to_np(layer.q_scales).view(np.uint16), ps.view(np.uint16).reshape(-1))
    assert np.array_equal(to_np(layer.q_zp), pz.reshape(-1))
    # activations on the 0.25 grid in [-4, 4]: every product and partial sum is exact, any summation order agrees
    g = torch.Generator(device="cpu").manual_seed(5)
    x = (torch.randint(-16, 17, (9, in_features), generator=g).to(torch.float32) * 0.25).to(torch.float16)
    y = layer(x.to(device))
    ref = oracle.gemm(x.view(torch.int16).numpy().view(np.float16), kat["weights"])
    assert np.array_equal(to_np(y).view(np.uint16), ref.view(np.uint16))
