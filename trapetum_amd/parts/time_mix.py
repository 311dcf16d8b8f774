"""A time-mixing recurrence: a matrix state per head that decays channel by channel, the decay computed from the input.

With x_t the mixer's input at a token and x_(t-1) the input of the token before (zeros before the sequence), each of
five branches s in (r, k, v, g, w) reads a mix of the two, x_t + (x_(t-1) - x_t) * mu_s.  r, k and v (heads x head_dim)
are products of their mixes; the gate is silu(W_g mix_g); the decay of key channel i of a head is

    w_t = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))           (W_w1 maps to a few channels, W_w2 back: the checkpoint's
                                                           shapes give their number)
    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t             (the bonus u counts for the present token only)
    S_t = diag(w_t) S_(t-1) + k_t v_t^T                   (S is head_dim x head_dim, zero before the sequence)

Every head's o is divided by its root mean square, multiplied by a gain and the gate, and projected back.  The decay
from the second small product on, the state, o and the norm are float32; the products and the mixes are in the
activation dtype.  What a sequence keeps between steps is S and the last token's input, both float32 states by name;
there is nothing per token.
"""
from ..cache.store import StateSpec
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import Mixer

BRANCHES = ("r", "k", "v", "g", "w")


class TimeMix(Mixer):
    output_dtype = None          # a mixer that holds this one may ask for its last product in another dtype

    def __init__(self, hidden_size, num_heads, head_dim, norm_eps, decay_rank=None,
                 tensors=("mu.", "r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o")):
        """decay_rank: the channels between the decay's two products when a random model is drawn (a checkpoint's
        shapes decide otherwise).  tensors: the prefix of the five mixing vectors, then the local names of W_r, W_k, W_v,
        W_g, W_w1, W_w2, w0, u, the norm's gain and W_o."""
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.norm_eps = float(norm_eps)
        self.decay_rank = int(decay_rank) if decay_rank else max(4, self.hidden_size // 16)
        self.names = dict(zip(("mu", "r", "k", "v", "g", "w1", "w2", "w0", "u", "norm", "o"), tensors))

    @property
    def inner(self):
        return self.num_heads * self.head_dim

    def tensor_specs(self):
        n, d, inner, rank = self.names, self.hidden_size, self.inner, self.decay_rank
        specs = {n["mu"] + s: TensorSpec((d,), init="norm") for s in BRANCHES}
        specs.update({n[s]: TensorSpec((inner, d)) for s in ("r", "k", "v", "g")})
        specs.update({n["w1"]: TensorSpec((rank, d), free=(0,)), n["w2"]: TensorSpec((inner, rank), free=(1,)),
                      n["w0"]: TensorSpec((inner,), init="norm"), n["u"]: TensorSpec((self.num_heads, self.head_dim), init="norm"),
                      n["norm"]: TensorSpec((inner,), init="gain"), n["o"]: TensorSpec((d, inner))})
        return specs

    def state_specs(self):
        return {"memory": StateSpec((self.num_heads, self.head_dim, self.head_dim), "float32"),
                "shift": StateSpec((self.hidden_size,), "float32")}

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        n = self.names
        if tensors[n["w1"]].shape[0] != tensors[n["w2"]].shape[1]:
            raise ValueError(f"the decay's two matrices do not meet: {tuple(tensors[n['w1']].shape)} and {tuple(tensors[n['w2']].shape)}")
        self.mu = torch.stack([tensors[n["mu"] + s].float() for s in BRANCHES]).contiguous()      # [5, D]
        self.w = {s: rt.matrix(tensors[n[s]]) for s in ("r", "k", "v", "g", "w1", "w2", "o")}
        self.w0 = tensors[n["w0"]].float().contiguous()
        self.bonus = tensors[n["u"]].float().contiguous()
        self.norm_gain = tensors[n["norm"]].float().contiguous()

    def forward(self, ctx, x, site):
        import torch
        ops, w = ctx.ops, self.w
        mixes = ops.shift_mix(x, self.mu, self.state(ctx, "shift"), ctx.slot_ids, ctx.cu_rows, ctx.row_seq,
                              one_row_each=ctx.mode == "decode")                                  # [5, M, D]
        r, k, v, g = (ops.linear(mixes[i], w[s], ctx.dtype) for i, s in enumerate(("r", "k", "v", "g")))
        low = ops.unary_(ops.linear(mixes[4], w["w1"], ctx.dtype), "tanh")
        log_rate = ops.linear(low, w["w2"], torch.float32)                                        # w0 is added in the scan
        y = ops.time_mix_scan(r, k, v, log_rate, self.w0, self.bonus, self.state(ctx, "memory"), ctx.slot_ids, ctx.cu_rows,
                              ctx.max_count, self.num_heads, self.head_dim)
        y = ops.head_norm_gate(y, self.norm_gain, g, self.norm_eps, self.num_heads, "silu", ctx.dtype)
        if self.output_dtype is not None:
            return ops.linear(y, w["o"], self.output_dtype)
        return ops.linear(y, w["o"], ctx.dtype, defer=True)


register_part("mixer", "time_mix", TimeMix)
