"""Gated feed-forward: down(act(gate x) * up x), or with a limit L and a shift c: g = min(gate x, L),
u = clamp(up x, -L, L), down(act(g) * (u + c)).

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
    def __init__(self, hidden_size, intermediate_size, activation,
                 tensors=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), limit=None, up_shift=0.0):
        """activation: gelu_tanh, silu, relu or quick_gelu (g sigmoid(1.702 g)).  limit None: no clamps."""
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation
        self.limit = None if limit is None else float(limit)
        self.up_shift = float(up_shift)
        self.names = tuple(tensors)      # local names of the gate, up and down matrices

    def tensor_specs(self):
        d, i = self.hidden_size, self.intermediate_size
        g, u, dn = self.names
        return {g: TensorSpec((i, d)), u: TensorSpec((i, d)), dn: TensorSpec((d, i))}

    def bind(self, tensors, rt):
        self.rt = rt
        g, u, dn = self.names
        self.w_gate_up = rt.ops.pack_gate_up(rt.matrix(tensors[g]), rt.matrix(tensors[u]))
        self.w_down = rt.matrix(tensors[dn])

    def forward(self, ctx, x, out=None):
        """out: a contiguous float32 [M, hidden] to fill (a caller that adds this layer's output to another's)."""
        if self.limit is None and self.up_shift == 0.0:
            act = ctx.ops.gated_linear(x, self.w_gate_up, self.intermediate_size, self.activation, ctx.dtype)
        else:
            act = ctx.ops.gated_linear(x, self.w_gate_up, self.intermediate_size, self.activation, ctx.dtype,
                                       limit=self.limit, up_shift=self.up_shift)
        if out is not None:
            return ctx.ops.linear(act, self.w_down, out.dtype, out=out)
        return ctx.ops.linear(act, self.w_down, ctx.dtype, defer=True)


class BiasedMLP(FeedForward):
    """down(act(up x + b_up)) + b_down: one product up, one down, both with a bias, no gate.  The first product's
    float32 sums take the bias and the activation before they are rounded.  The second product carries its bias as a
    further column of its matrix, met by a column of ones in the activations (where the bias is exact in the matrix's
    width: a bfloat16 checkpoint's always is), so it is left to the block's add like any other product, in K slices where
    it has them; otherwise the bias is added by a launch of its own."""

    PAD = 64       # columns added to the second product's K: the bias and zeros (K stays a whole number of k steps)

    def __init__(self, hidden_size, intermediate_size, activation="gelu_erf", tensors=("up", "down"), bias_suffix=".b"):
        """activation: gelu_erf, the exact x Phi(x).  tensors: local names of the two matrices; a bias is named like its
        matrix with bias_suffix."""
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.names = tuple(tensors)
        self.bias_suffix = bias_suffix

    def tensor_specs(self):
        d, i, (up, dn), b = self.hidden_size, self.intermediate_size, self.names, self.bias_suffix
        return {up: TensorSpec((i, d)), up + b: TensorSpec((i,), init="norm"),
                dn: TensorSpec((d, i)), dn + b: TensorSpec((d,), init="norm")}

    def bind(self, tensors, rt):
        self.rt = rt
        (up, dn), b = self.names, self.bias_suffix
        import torch
        self.w_up = rt.matrix(tensors[up])
        self.b_up, self.b_down = tensors[up + b].float().contiguous(), tensors[dn + b].float().contiguous()
        w_down, bias = tensors[dn], tensors[dn + b]
        self.folded = bool(torch.equal(bias.to(w_down.dtype).float(), bias.float()))
        if self.folded:
            wide = torch.cat([w_down, bias.to(w_down.dtype).reshape(-1, 1), w_down.new_zeros((w_down.shape[0], self.PAD - 1))], dim=1)
            self.w_down = rt.matrix(wide.contiguous())
        else:
            self.w_down = rt.matrix(w_down)

    def forward(self, ctx, x, out=None):
        import torch
        up = ctx.ops.linear(x, self.w_up, torch.float32)
        if self.folded:
            act = ctx.ops.bias_act(up, self.b_up, self.activation, ctx.dtype, pad=self.PAD)
            return ctx.ops.linear(act, self.w_down, ctx.dtype, defer=True)
        act = ctx.ops.bias_act(up, self.b_up, self.activation, ctx.dtype)
        return ctx.ops.linear(act, self.w_down, torch.float32, bias=self.b_down)


register_part("feed_forward", "gated_mlp", GatedMLP)
register_part("feed_forward", "biased_mlp", BiasedMLP)
