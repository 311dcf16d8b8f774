"""A mixture of experts: a router picks `top` of `n_experts` small gated feed-forward layers for every token.

Router: z = W_router h (+ a bias) in fp32, s = softmax(z) over all experts; the `top` largest scores choose the experts and
weigh their outputs as they are (renormalize=True divides them by their sum, which is the softmax over the chosen
logits alone).  A shared layer that every token passes may be added, optionally times sigmoid(w_sg . h), one number
per token.  Expert (no biases):
g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), y = g * sigmoid(alpha g) * (u + 1), output W_down y.
The step's (token, expert) pairs are sorted by expert on the device, so that each expert's matrices are read by one
run of row tiles, and the weighted sum over a token's experts is formed in fp32 in a fixed order.
"""
from ..models.spec import TensorSpec
from ..registry import register_part
from .base import FeedForward


class RoutedExperts(FeedForward):
    def __init__(self, hidden_size, intermediate_size, n_experts, top, limit, gate_alpha=1.702, up_shift=1.0,
                 renormalize=False, router="router", expert="e{}.", tensors=("gate", "up", "down"),
                 score="softmax", weight_input=False, shared=None, router_bias=None, shared_gate=None):
        """limit None: gate and up sums are not clamped (with gate_alpha 1 and up_shift 0 the expert is SiLU-gated).
        score: "softmax" over all experts or the "sigmoid" of each logit.  weight_input: a chosen expert's score
        multiplies its input, expert(s h), instead of its output.  shared: (registered feed-forward, parameters) of a
        layer that every token passes as well; its output is added.  router_bias: local name of a vector [experts] added
        to the router's logits.  shared_gate: local name of a matrix [1, hidden]; the shared layer's output is multiplied
        by the sigmoid of its product with the token's input."""
        if not 0 < top <= n_experts:
            raise ValueError(f"{top} of {n_experts} experts cannot be chosen")
        if score not in ("softmax", "sigmoid"):
            raise ValueError(f"a router's scores are softmax or sigmoid, not '{score}'")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.n_experts, self.top = int(n_experts), int(top)
        self.limit = None if limit is None else float(limit)
        self.gate_alpha, self.up_shift = float(gate_alpha), float(up_shift)
        self.renormalize = bool(renormalize)
        self.score, self.weight_input = score, bool(weight_input)
        self.router_name, self.expert_name, self.names = router, expert, tuple(tensors)
        self.router_bias_name, self.shared_gate_name = router_bias, shared_gate
        if shared_gate is not None and shared is None:
            raise ValueError("a gate on the shared layer needs a shared layer")
        self.shared, self.shared_prefix = None, ""
        if shared is not None:
            from ..registry import build_part
            name, params = shared
            params = dict(params)
            self.shared_prefix = params.pop("prefix", "shared.")
            self.shared = build_part("feed_forward", (name, params))

    def tensor_specs(self):
        d, i = self.hidden_size, self.intermediate_size
        specs = {self.router_name: TensorSpec((self.n_experts, d))}
        g, u, dn = self.names
        for e in range(self.n_experts):
            p = self.expert_name.format(e)
            specs.update({p + g: TensorSpec((i, d)), p + u: TensorSpec((i, d)), p + dn: TensorSpec((d, i))})
        if self.shared is not None:
            specs.update({self.shared_prefix + k: v for k, v in self.shared.tensor_specs().items()})
        if self.router_bias_name:
            specs[self.router_bias_name] = TensorSpec((self.n_experts,), init="norm")
        if self.shared_gate_name:
            specs[self.shared_gate_name] = TensorSpec((1, d))
        return specs

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        g, u, dn = self.names
        ex = [self.expert_name.format(e) for e in range(self.n_experts)]
        self.w_router = rt.matrix(tensors[self.router_name])
        # [experts, 2 ff, width]: an expert's gate rows, then its up rows; [experts, width, ff]
        self.w_gate_up = rt.matrix(torch.stack([torch.cat([tensors[p + g], tensors[p + u]], dim=0) for p in ex]).contiguous())
        self.w_down = rt.matrix(torch.stack([tensors[p + dn] for p in ex]).contiguous())
        if self.shared is not None:
            self.shared.bind({k: tensors[self.shared_prefix + k] for k in self.shared.tensor_specs()}, rt)
        self.router_bias = tensors[self.router_bias_name].float().contiguous() if self.router_bias_name else None
        self.w_shared_gate = rt.matrix(tensors[self.shared_gate_name].contiguous()) if self.shared_gate_name else None

    def forward(self, ctx, x):
        import torch
        ops = ctx.ops
        logits = ops.linear(x, self.w_router, torch.float32, bias=self.router_bias)        # fp32 sums of exact products
        chosen, weights = ops.route_top(logits, self.top, self.renormalize, score=self.score)
        if self.shared is None:
            return ops.expert_ffn(x, chosen, weights, self.w_gate_up, self.w_down, self.limit, self.gate_alpha, self.up_shift,
                                  weight_input=self.weight_input)
        # the experts' sum and the shared layer's output as two slices that the block's add forms the sum of
        both = torch.empty((2, x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
        ops.expert_ffn(x, chosen, weights, self.w_gate_up, self.w_down, self.limit, self.gate_alpha, self.up_shift,
                       weight_input=self.weight_input, out=both[0])
        self.shared.forward(ctx, x, out=both[1])
        if self.w_shared_gate is not None:
            ops.mul_sigmoid_heads(both[1], ops.linear(x, self.w_shared_gate, torch.float32), 1)
        return ops.SplitRows(both)


register_part("feed_forward", "routed_experts", RoutedExperts)
