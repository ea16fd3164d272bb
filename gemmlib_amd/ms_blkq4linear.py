"""``BlkQ4Linear``: a linear layer whose weights are blockwise-quantized to 4 bits at construction.

Same constructor, attributes and ``forward`` as the reference module
(reference: python/ms_blkq4linear.py:10-28): ``weights`` is the fp16 ``[out_features, in_features]``
tensor on the GPU, ``scale_only`` selects the symmetric quantizer (no zero-points), the packed
tensors are plain attributes ``q_weights`` / ``q_scales`` / ``q_zp`` and the bias is added in place.
All device work happens in the HIP library behind ``ms_blkq4linear_ext``; there is no fallback.
"""

from torch import nn

from . import ms_blkq4linear_ext


class BlkQ4Linear(nn.Module):
    def __init__(self, block_size, col_wise, scale_only, weights, bias_tensor=None):
        super().__init__()
        self.block_size = block_size
        self.col_wise = col_wise
        self.has_offsets = not scale_only
        self.in_features = weights.size(1)
        self.out_features = weights.size(0)
        self.q_weights, self.q_scales, self.q_zp = ms_blkq4linear_ext.quant(
            block_size, col_wise, self.has_offsets, weights)
        self.bias = bias_tensor

    def forward(self, input):
        output = ms_blkq4linear_ext.forward(self.block_size, self.col_wise, self.in_features, self.out_features,
                                            input, self.q_weights, self.q_scales, self.q_zp)
        if self.bias is not None:
            output += self.bias
        return output
