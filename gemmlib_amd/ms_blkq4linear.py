"""``BlkQ4Linear``: a linear layer whose weights are blockwise-quantized to 4 bits at construction.

Same constructor, attributes and ``forward`` as the reference module
(reference: python/ms_blkq4linear.py:10-28): ``weights`` is the fp16 ``[out_features, in_features]``
tensor on the GPU, ``scale_only`` selects the symmetric quantizer (no zero-points), the packed
tensors are reachable as ``q_weights`` / ``q_scales`` / ``q_zp``.  The bias is added by the GEMM's epilogue
with the same two roundings as the reference's in-place ``output += self.bias`` (python/ms_blkq4linear.py:26-27),
so the result is bit for bit the same without a second kernel.
All device work happens in the HIP library behind ``ms_blkq4linear_ext``; there is no fallback.

Beyond the reference (which keeps the packed tensors as plain attributes, so ``state_dict()`` loses
them, and takes 2-D inputs only):

* the packed tensors and the bias are registered buffers, and the quantization parameters travel as
  the module's extra state, so ``state_dict()`` / ``load_state_dict()`` round-trip a quantized layer;
  ``BlkQ4Linear.from_packed`` builds a layer straight from packed tensors, without the fp16 weights;
* ``forward`` accepts any number of leading dimensions (``[..., in_features]``);
* bfloat16 weights make a bfloat16 layer (bfloat16 scales, inputs, bias and outputs).
"""

import torch
from torch import nn

import ms_blkq4linear_ext  # top-level, as in the reference (python/ms_blkq4linear.py:7)


class BlkQ4Linear(nn.Module):
    def __init__(self, block_size, col_wise, scale_only, weights, bias_tensor=None):
        super().__init__()
        self.block_size = block_size
        self.col_wise = col_wise
        self.has_offsets = not scale_only
        self.in_features = weights.size(1)
        self.out_features = weights.size(0)
        q_weights, q_scales, q_zp = ms_blkq4linear_ext.quant(block_size, col_wise, self.has_offsets, weights)
        self.register_buffer("q_weights", q_weights)
        self.register_buffer("q_scales", q_scales)
        self.register_buffer("q_zp", q_zp)
        self.register_buffer("bias", bias_tensor)

    @classmethod
    def from_packed(cls, block_size, col_wise, in_features, out_features, q_weights, q_scales, q_zp=None,
                    bias_tensor=None):
        """A layer around tensors that ``ms_blkq4linear_ext.quant`` (or ``blkq4_fp16_quant_sm80``) produced
        earlier.  ``q_zp`` None or empty means the symmetric quantizer."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.block_size = block_size
        self.col_wise = col_wise
        self.has_offsets = q_zp is not None and q_zp.numel() > 0
        self.in_features = in_features
        self.out_features = out_features
        if q_zp is None:
            q_zp = torch.empty(0, dtype=torch.uint8, device=q_weights.device)
        blocks = (in_features // block_size) * out_features if col_wise else in_features * (out_features // block_size)
        if q_weights.numel() != in_features * out_features // 2 or q_scales.numel() != blocks or (
                self.has_offsets and q_zp.numel() != blocks):
            raise ValueError("packed tensor sizes do not match the layer shape and block size")
        self.register_buffer("q_weights", q_weights)
        self.register_buffer("q_scales", q_scales)
        self.register_buffer("q_zp", q_zp)
        self.register_buffer("bias", bias_tensor)
        return self

    def get_extra_state(self):
        return {"block_size": self.block_size, "col_wise": self.col_wise, "has_offsets": self.has_offsets,
                "in_features": self.in_features, "out_features": self.out_features,
                "dtype": str(self.q_scales.dtype)}

    def set_extra_state(self, state):
        for key in ("block_size", "col_wise", "has_offsets", "in_features", "out_features"):
            if getattr(self, key) != state[key]:
                raise ValueError(f"state dict was saved with {key}={state[key]}, this layer has {getattr(self, key)}")
        # the scales of a float16 and of a bfloat16 layer are not interchangeable (copying one into the other
        # would convert them silently); state dicts saved before the element type was recorded are float16
        saved = state.get("dtype", "torch.float16")
        if saved != str(self.q_scales.dtype):
            raise ValueError(f"state dict was saved with dtype={saved}, this layer has {self.q_scales.dtype}")

    def forward(self, input):
        lead = input.shape[:-1]
        x = input if input.dim() == 2 else input.reshape(-1, input.shape[-1])
        output = ms_blkq4linear_ext.forward(self.block_size, self.col_wise, self.in_features, self.out_features,
                                            x, self.q_weights, self.q_scales, self.q_zp, self.bias)
        return output if input.dim() == 2 else output.reshape(*lead, self.out_features)

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, block_size={self.block_size}, "
                f"col_wise={self.col_wise}, has_offsets={self.has_offsets}, bias={self.bias is not None}")
