"""Two mixers side by side on the same input: out = (norm_l(left(x)) + norm_r(right(x))) / 2, or a_l left(x) + a_r right(x).

combine "norm_mean": each output is divided by its root mean square over the model width and multiplied by a gain of
its own (used as stored), in float32, before the two are averaged.  combine "weighted_sum": the outputs are added as
they are, in float32, each times a constant of the model (`weights`); there are no gains.  The two mixers are any registered mixers; at most one of them may
keep tensors per token (it becomes this mixer's cache, so that another layer's run can read it), and the states they
declare by name are kept under "left." and "right.".
"""
from ..cache.store import TokenSpec
from ..models.spec import TensorSpec
from ..registry import build_part, register_part
from .base import Mixer


class ParallelMixers(Mixer):
    def __init__(self, hidden_size, left, right, eps=0.0, prefixes=("left.", "right."), tensors=("left.out", "right.out"),
                 combine="norm_mean", weights=(1.0, 1.0)):
        if combine not in ("norm_mean", "weighted_sum"):
            raise ValueError(f"two mixers side by side are combined by norm_mean or weighted_sum, not '{combine}'")
        self.hidden_size, self.eps = int(hidden_size), float(eps)
        self.sides = [build_part("mixer", left), build_part("mixer", right)]
        self.prefixes = tuple(prefixes)
        self.combine, self.weights = combine, tuple(float(w) for w in weights)
        self.names = tuple(tensors) if combine == "norm_mean" else ()
        if combine == "weighted_sum":
            import torch
            for m in self.sides:                     # the sum is formed in float32 from float32 products where a side can give them
                if hasattr(m, "output_dtype"):
                    m.output_dtype = torch.float32
        caches = [m.cache_spec() for m in self.sides]
        if sum(c is not None for c in caches) > 1:
            raise ValueError("of two mixers side by side only one may keep a cache of its own kind; the other keeps named states")
        if any(c is not None and not isinstance(c, TokenSpec) for c in caches):
            raise ValueError("a mixer beside another declares its states by name (state_specs), not as its cache")
        self._cache = next((c for c in caches if c is not None), None)

    def tensor_specs(self):
        specs = {}
        for m, p in zip(self.sides, self.prefixes):
            specs.update({p + k: v for k, v in m.tensor_specs().items()})
        for name in self.names:
            specs[name] = TensorSpec((self.hidden_size,), init="gain")
        return specs

    def cache_spec(self):
        return self._cache

    def state_specs(self):
        specs = {}
        for m, p in zip(self.sides, self.prefixes):
            specs.update({p + k: v for k, v in m.state_specs().items()})
        return specs

    def bind(self, tensors, rt):
        self.rt = rt
        for m, p in zip(self.sides, self.prefixes):
            m.state_scope = self.state_scope + p
            m.bind({k: tensors[p + k] for k in m.tensor_specs()}, rt)
        self.gains = [tensors[name].float().contiguous() for name in self.names]

    def forward(self, ctx, x, site):
        ops = ctx.ops
        if self.combine == "weighted_sum":
            import torch
            a, b = (ops.rows(m.forward(ctx, x, site), torch.float32) for m in self.sides)
            return ops.weighted_sum(a, self.weights[0], b, self.weights[1])
        a, b = (ops.rows(m.forward(ctx, x, site), ctx.dtype) for m in self.sides)
        return ops.pair_norm_mean(a, b, self.gains[0], self.gains[1], self.eps)


register_part("mixer", "parallel", ParallelMixers)
