"""RMSNorm with the weight used as (offset + w), over the whole row or over equal consecutive groups of it.

y = x * rsqrt(mean(x^2) + eps) * gain, statistics and products in fp32, one
rounding at the end (runtime/cuda/codebook_gemv.cu:192-202).  The reference
bakes Gemma's (1 + w) into the stored weight (model/export_gemma.py:25-26); here
the offset is a parameter and the sum is formed once, in fp32, when the weight
is bound.  With `groups` = g the row is cut into g equal consecutive parts and each
is divided by its own root mean square; the gain spans the whole row.  `tensor` is
the local name of the weight in the checkpoint ("" when the prefix is the whole name).
"""
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Norm


class RMSNorm(Norm):
    def __init__(self, size, eps, weight_offset=0.0, groups=1, tensor="weight", init="norm"):
        if groups <= 0 or size % groups:
            raise ValueError(f"a norm over {size} elements cannot be cut into {groups} equal groups")
        self.size = size
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)
        self.groups = int(groups)
        self.tensor = tensor
        self.init = init                    # how a random model draws the weight: "norm" around zero, "gain" around one

    def tensor_specs(self):
        return {self.tensor: TensorSpec((self.size,), init=self.init)}

    def bind(self, tensors, rt):
        self.rt = rt
        self.gain = (tensors[self.tensor].float() + self.weight_offset).contiguous()

    def forward(self, ctx, x, out_dtype=None):
        return ctx.ops.rms_norm(x, self.gain, self.eps, out_dtype or ctx.dtype, groups=self.groups)


register_part("norm", "rms_norm", RMSNorm)
