"""Besulix as data: layers in the order config.json lists them.

The embedded row passes an RMS norm of its own.  A layer is x += mixer(n1(x)), then (if it has one) x += ff(n2(x)), with
RMS norms whose weight is the gain as stored: the `pre_norm` block.  Mixers: `mlstm`, a matrix memory per head with
exponential gates, or `parallel`: a chunked grouped-query attention (biased projections, rotation of halves on the
first rot.dims elements, values rotated by their position, a temperature and a softmax sink per head) beside a
time-mixing recurrence, their outputs added with the configuration's two weights.  Feed-forward: gate and up sums
clamped at `limit`, the gate through g sigmoid(1.702 g), the up sum plus one.  The logits pass a tanh cap.
Tensor names: embed, embed.norm, head, final.norm, l<i>.norm1/.norm2, l<i>.mix.{q,k,v,g,o,norm,i,i.b,f,f.b} or
l<i>.mix.left.{q,q.b,k,k.b,v,v.b,temp,sink,o} and l<i>.mix.right.{mu.r,mu.k,mu.v,mu.g,mu.w,r,k,v,g,w1,w2,w0,u,norm,o},
l<i>.mlp.{gate,up,down}.
"""
from ..config.besulix import BesulixConfig
from ..registry import register_architecture
from .spec import LayerSpec, ModelSpec, ScheduleEntry


def build_spec(c: BesulixConfig) -> ModelSpec:
    D = c.hidden_size
    norm = ("rms_norm", {"size": D, "eps": c.norm_eps, "weight_offset": 0.0, "tensor": "", "init": "gain"})
    layers, schedule = [], []
    for i, l in enumerate(c.layers):
        p = f"l{i}."
        m = l.mixer
        if l.type == "mlstm":
            mixer = ("matrix_memory", {"hidden_size": D, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim,
                                       "gate_cap": m.gate_cap, "norm_eps": c.norm_eps})
        else:
            a, r = m.left, m.right
            position = ("rope", {"rotary_dim": a.rot.dims, "theta": a.rot.base}) if a.rot.dims else ("none", {})
            left = ("attention", {"hidden_size": D, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
                                  "value_dim": a.vdim, "query_scale": a.scale, "position": position,
                                  "tensors": ("q", "k", "v", "o"), "bias_suffix": ".b", "chunk": a.chunk,
                                  "head_temperature": "temp", "sink": "sink", "value_rotation": a.rot.base, "precise_weights": True})
            right = ("time_mix", {"hidden_size": D, "num_heads": r.heads, "head_dim": r.dim, "norm_eps": c.norm_eps})
            mixer = ("parallel", {"hidden_size": D, "left": left, "right": right, "combine": "weighted_sum",
                                  "weights": (m.left_scale, m.right_scale)})
        prefixes = {"mixer": p + "mix.", "pre_mixer_norm": p + "norm1"}
        ff = None
        if l.mlp is not None:
            ff = ("gated_mlp", {"hidden_size": D, "intermediate_size": l.mlp.ff, "activation": "quick_gelu",
                                "tensors": ("gate", "up", "down"), "limit": l.mlp.limit, "up_shift": 1.0})
            prefixes.update({"feed_forward": p + "mlp.", "pre_ff_norm": p + "norm2"})
        layers.append(LayerSpec(block=("pre_norm", {}), mixer=mixer, feed_forward=ff, norm=norm, prefixes=prefixes))
        schedule.append(ScheduleEntry(i))
    return ModelSpec(
        architecture=c.architecture, hidden_size=D, vocab_size=c.vocab_size,
        embedding=("scaled_embedding", {"vocab_size": c.vocab_size, "hidden_size": D, "scale": 1.0, "tensor": "",
                                        "norm": ("rms_norm", {"size": D, "eps": c.norm_eps, "tensor": ".norm", "init": "gain"})}),
        embedding_prefix="embed", layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=("linear_head", {"vocab_size": c.vocab_size, "hidden_size": D, "softcap": c.logit_softcap, "tensor": ""}),
        head_prefix="head", stop_ids=())


register_architecture(BesulixConfig.architecture, BesulixConfig, build_spec)
