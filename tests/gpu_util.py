"""Helpers shared by the GPU parity tests: every call goes through the C ABI (gemmlib_amd.capi)."""

import numpy as np
import torch


def to_dev(a: np.ndarray, device):
    """numpy (fp16 / uint8) -> device tensor holding the same bits."""
    if a.dtype == np.float16:
        return torch.from_numpy(a.view(np.int16).copy()).to(device).view(torch.float16)
    return torch.from_numpy(a.copy()).to(device)


def to_np(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.float16:
        return t.view(torch.int16).cpu().numpy().view(np.float16)
    return t.cpu().numpy()


def quantize_on_gpu(capi, device, block_size, weights_nk: np.ndarray, has_offsets: bool, w_dev=None,
                    column_wise: bool = True):
    """blkq4_fp16_quant_size_sm80 + blkq4_fp16_quant_sm80 -> (q_w, q_s, q_zp|None) device tensors."""
    n, k = weights_nk.shape
    w_elems, meta_elems = capi.quant_size(block_size, column_wise, k, n)
    if w_dev is None:
        w_dev = to_dev(weights_nk, device)
    # poison the outputs so that an element the kernel fails to write cannot pass by luck
    q_w = torch.full((w_elems,), 0xA5, dtype=torch.uint8, device=device)
    q_s = torch.full((meta_elems,), float("nan"), dtype=torch.float16, device=device)
    q_zp = torch.full((meta_elems,), 0xEE, dtype=torch.uint8, device=device) if has_offsets else None
    capi.quant(block_size, column_wise, w_dev, q_w, q_s, q_zp)
    torch.cuda.synchronize()
    return q_w, q_s, q_zp


def gemm_on_gpu(capi, device, block_size, a_mk: np.ndarray, q_w, q_s, q_zp, n: int, column_wise: bool = True):
    m, k = a_mk.shape
    a_dev = to_dev(a_mk, device)
    out = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    capi.gemm(block_size, column_wise, m, n, k, a_dev, q_w, q_s, q_zp, out)
    torch.cuda.synchronize()
    return to_np(out)


def max_rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / max(|ref|, floor) with floor = 1e-3 * max|ref| (outputs whose exact value
    is nearly zero are measured against the scale of the matrix, not against themselves)."""
    g = got.astype(np.float64)
    r = ref.astype(np.float64)
    floor = 1e-3 * np.max(np.abs(r)) + 1e-30
    return float(np.max(np.abs(g - r) / np.maximum(np.abs(r), floor)))
