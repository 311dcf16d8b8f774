"""Token embedding and the head that turns rows into logits.

Embedding: table[token] * scale in fp32, then (optionally) a norm of the row (the reference bakes Gemma's sqrt(hidden)
into an fp16 table at export, model/export_gemma.py:59-61; here the table stays
as stored so that a tied head can use it unscaled, :73).  Head: logits = rows @
table^T with fp32 accumulation and fp32 output, then c * tanh(z / c) when a cap is
set (runtime/src/lib.rs:4558-4560, on the host there; in the product's epilogue here).
"""
from ..models.spec import TensorSpec
from ..registry import build_part, register_part
from .base import Embedding, Head


class ScaledEmbedding(Embedding):
    def __init__(self, vocab_size, hidden_size, scale, tensor="weight", norm=None):
        """norm: (registered norm, parameters) applied to every embedded row, in fp32; its tensors stand beside the
        table under the names its parameters give."""
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.tensor = tensor             # the table's local name ("" when the prefix is the whole name)
        self.norm = build_part("norm", norm) if norm is not None else None

    def tensor_specs(self):
        specs = {self.tensor: TensorSpec((self.vocab_size, self.hidden_size), init="embedding")}
        if self.norm is not None:
            specs.update(self.norm.tensor_specs())
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        self.table = rt.matrix(tensors[self.tensor])
        if self.norm is not None:
            self.norm.bind({k: tensors[k] for k in self.norm.tensor_specs()}, rt)

    def forward(self, ctx, tokens):
        import torch
        rows = ctx.ops.embed_rows(tokens, self.table, self.scale)
        return rows if self.norm is None else self.norm.forward(ctx, rows, torch.float32)


class LinearHead(Head):
    def __init__(self, vocab_size, hidden_size, softcap=None, scale=None, tensor="weight"):
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.softcap = softcap
        self.scale = None if scale is None or float(scale) == 1.0 else float(scale)     # logits = (rows @ table^T) * scale
        self.tensor = tensor

    def tensor_specs(self):
        return {self.tensor: TensorSpec((self.vocab_size, self.hidden_size), init="embedding")}

    def bind(self, tensors, rt):
        self.rt = rt
        self.weight = rt.matrix(tensors[self.tensor])

    def forward(self, ctx, rows):
        import torch
        logits = ctx.ops.linear(rows, self.weight, torch.float32, softcap=self.softcap)
        if self.scale is not None:
            ctx.ops.scale_rows(logits, self.scale)
        return logits


register_part("embedding", "scaled_embedding", ScaledEmbedding)
register_part("head", "linear_head", LinearHead)
