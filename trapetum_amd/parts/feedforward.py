"""Gated feed-forward: down(act(gate x) * up x).

The reference computes gate and up as two fp32 vectors, applies
0.5 g (1 + tanh(0.7978845608 (g + 0.044715 g^3))) * u in fp32 and rounds once
(runtime/src/lib.rs:4511-4516, runtime/cuda/codebook_gemv.cu:531-537).  Here gate
and up are one matrix product whose epilogue applies the activation on the fp32
accumulators, so g and u never reach memory.
"""
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import FeedForward


class GatedMLP(FeedForward):
    def __init__(self, hidden_size, intermediate_size, activation):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation

    def tensor_specs(self):
        d, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": TensorSpec((i, d)), "up_proj.weight": TensorSpec((i, d)),
                "down_proj.weight": TensorSpec((d, i))}

    def bind(self, tensors, rt):
        self.rt = rt
        self.w_gate_up = rt.ops.pack_gate_up(rt.matrix(tensors["gate_proj.weight"]), rt.matrix(tensors["up_proj.weight"]))
        self.w_down = rt.matrix(tensors["down_proj.weight"])

    def forward(self, ctx, x):
        act = ctx.ops.gated_linear(x, self.w_gate_up, self.intermediate_size, self.activation, ctx.dtype)
        return ctx.ops.linear(act, self.w_down, ctx.dtype, defer=True)


register_part("feed_forward", "gated_mlp", GatedMLP)
