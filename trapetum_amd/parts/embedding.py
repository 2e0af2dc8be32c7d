"""Token embedding and the head that turns rows into logits.

Embedding: table[token] * scale in fp32 (the reference bakes Gemma's sqrt(hidden)
into an fp16 table at export, model/export_gemma.py:59-61; here the table stays
as stored so that a tied head can use it unscaled, :73).  Head: logits = rows @
table^T with fp32 accumulation and fp32 output, then c * tanh(z / c) when a cap is
set (runtime/src/lib.rs:4558-4560, on the host there; in the product's epilogue here).
"""
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Embedding, Head


class ScaledEmbedding(Embedding):
    def __init__(self, vocab_size, hidden_size, scale):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)

    def tensor_specs(self):
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size), init="embedding")}

    def bind(self, tensors, rt):
        self.rt = rt
        self.table = rt.matrix(tensors["weight"])

    def forward(self, ctx, tokens):
        return ctx.ops.embed_rows(tokens, self.table, self.scale)


class LinearHead(Head):
    def __init__(self, vocab_size, hidden_size, softcap=None):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.softcap = softcap

    def tensor_specs(self):
        return {"weight": TensorSpec((self.vocab_size, self.hidden_size), init="embedding")}

    def bind(self, tensors, rt):
        self.rt = rt
        self.weight = rt.matrix(tensors["weight"])

    def forward(self, ctx, rows):
        import torch
        return ctx.ops.linear(rows, self.weight, torch.float32, softcap=self.softcap)


register_part("embedding", "scaled_embedding", ScaledEmbedding)
register_part("head", "linear_head", LinearHead)
