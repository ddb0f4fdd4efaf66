"""A short causal convolution over time on every channel, in front of a sub-layer.

What the sub-layer reads of the stream x is h_t = x_t + sum_j w[:, j] * x_(t - taps + 1 + j), with zeros before the
sequence's first token; w is [channels, taps] and there is no bias.  The sum is formed in fp32 from the fp32 stream
and rounded once to the activation dtype.  The last taps - 1 rows of x are the sequence's state: a step reads them
for its first rows and leaves its own last rows there, so that a sequence may be cut into steps anywhere.
"""
from ..cache.store import StateSpec
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Conv


class CausalConv(Conv):
    def __init__(self, size, taps, residual=True, tensor="weight"):
        if taps < 1:
            raise ValueError(f"a convolution needs at least one tap, found {taps}")
        self.size, self.taps, self.residual, self.tensor = int(size), int(taps), bool(residual), tensor

    def tensor_specs(self):
        return {self.tensor: TensorSpec((self.size, self.taps), init="norm")}

    def state_spec(self):
        return StateSpec((self.taps - 1, self.size), "float32") if self.taps > 1 else None

    def bind(self, tensors, rt):
        self.rt = rt
        self.w = tensors[self.tensor].float().contiguous()
        self.w_t = self.w.t().contiguous()               # [taps, channels]: neighbouring channels' taps side by side

    def forward(self, ctx, stream, state):
        return ctx.ops.causal_conv(stream, self.w, state, ctx.slot_ids, ctx.cu_rows, ctx.row_seq, ctx.dtype,
                                   residual=self.residual, one_row_each=ctx.mode == "decode", w_t=self.w_t)


register_part("conv", "causal_conv", CausalConv)
