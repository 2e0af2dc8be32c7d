"""RMSNorm with the weight used as (offset + w).

y = x * rsqrt(mean(x^2) + eps) * gain, statistics and products in fp32, one
rounding at the end (runtime/cuda/codebook_gemv.cu:192-202).  The reference
bakes Gemma's (1 + w) into the stored weight (model/export_gemma.py:25-26); here
the offset is a parameter and the sum is formed once, in fp32, when the weight
is bound.
"""
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Norm


class RMSNorm(Norm):
    def __init__(self, size, eps, weight_offset=0.0):
        self.size = size
        self.eps = float(eps)
        self.weight_offset = float(weight_offset)

    def tensor_specs(self):
        return {"weight": TensorSpec((self.size,), init="norm")}

    def bind(self, tensors, rt):
        self.rt = rt
        self.gain = (tensors["weight"].float() + self.weight_offset).contiguous()

    def forward(self, ctx, x, out_dtype=None):
        return ctx.ops.rms_norm(x, self.gain, self.eps, out_dtype or ctx.dtype)


register_part("norm", "rms_norm", RMSNorm)
