"""A matrix memory per head with exponential gates (the mLSTM cell of xLSTM).

From the mixer's input x: q = W_q x * key_dim^(-1/2), k = W_k x (heads x key_dim), v = W_v x (heads x value_dim), and
per head the logarithms of an input and a forget gate, both capped by a tanh:

    i_t = cap tanh((W_i x + b_i) / cap),   f_t = logsigmoid(cap tanh((W_f x + b_f) / cap))
    m_t = max(f_t + m_(t-1), i_t)                                    (m starts at 0)
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t likewise with k_t alone
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)

Every head's o is divided by its root mean square, multiplied by a gain and by sigmoid(W_g x), and projected back.  The
gates (their sums too), m, S, n, o and the norm are float32; q, k, v and the output gate come from one product in the
activation dtype.  A sequence keeps S, n and m between steps, float32 states by name; there is nothing per token.
"""
from ..cache.store import StateSpec
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Mixer


class MatrixMemory(Mixer):
    output_dtype = None          # a mixer that holds this one may ask for its last product in another dtype

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, gate_cap, norm_eps,
                 tensors=("q", "k", "v", "g", "o", "norm", "i", "f"), bias_suffix=".b"):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.names = dict(zip(("q", "k", "v", "g", "o", "norm", "i", "f"), tensors))
        self.bias_suffix = bias_suffix

    def tensor_specs(self):
        n, d, H = self.names, self.hidden_size, self.num_heads
        qk, vv = H * self.key_dim, H * self.value_dim
        specs = {n["q"]: TensorSpec((qk, d)), n["k"]: TensorSpec((qk, d)), n["v"]: TensorSpec((vv, d)), n["g"]: TensorSpec((vv, d)),
                 n["o"]: TensorSpec((d, vv)), n["norm"]: TensorSpec((vv,), init="gain")}
        for s in ("i", "f"):
            specs[n[s]] = TensorSpec((H, d))
            specs[n[s] + self.bias_suffix] = TensorSpec((H,), init="norm")
        return specs

    def state_specs(self):
        H = self.num_heads
        return {"memory": StateSpec((H, self.key_dim, self.value_dim), "float32"),
                "normalizer": StateSpec((H, self.key_dim), "float32"), "maximum": StateSpec((H,), "float32")}

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        n = self.names
        w = torch.cat([tensors[n[s]] for s in ("q", "k", "v", "g")], dim=0)
        spare = -w.shape[0] % 8                  # zero rows: a row of the product is whole 16-byte pieces
        if spare:
            w = torch.cat([w, w.new_zeros((spare, w.shape[1]))], dim=0)
        self.w_in = rt.matrix(w.contiguous())
        self.w_gates = rt.matrix(torch.cat([tensors[n["i"]], tensors[n["f"]]], dim=0).contiguous())
        self.b_gates = torch.cat([tensors[n["i"] + self.bias_suffix].float(), tensors[n["f"] + self.bias_suffix].float()]).contiguous()
        self.norm_gain = tensors[n["norm"]].float().contiguous()
        self.w_o = rt.matrix(tensors[n["o"]])

    def forward(self, ctx, x, site):
        import torch
        ops, H = ctx.ops, self.num_heads
        qk, vv = H * self.key_dim, H * self.value_dim
        u = ops.linear(x, self.w_in, ctx.dtype)                                                   # [M, q | k | v | g]
        gates = ops.linear(x, self.w_gates, torch.float32, bias=self.b_gates)                     # [M, i | f] before the caps
        y = ops.matrix_memory_scan(u[:, :qk], u[:, qk:2 * qk], u[:, 2 * qk:2 * qk + vv], gates, self.gate_cap, self.key_dim ** -0.5,
                                   self.state(ctx, "memory"), self.state(ctx, "normalizer"), self.state(ctx, "maximum"),
                                   ctx.slot_ids, ctx.cu_rows, ctx.max_count, H, self.key_dim, self.value_dim)
        y = ops.head_norm_gate(y, self.norm_gain, u[:, 2 * qk + vv:2 * qk + 2 * vv], self.norm_eps, H, "sigmoid", ctx.dtype)
        if self.output_dtype is not None:
            return ops.linear(y, self.w_o, self.output_dtype)
        return ops.linear(y, self.w_o, ctx.dtype, defer=True)


register_part("mixer", "matrix_memory", MatrixMemory)
