"""Vogunex as data: layers in the order config.json lists them.

A layer is x += mixer(shift(n1(x))), x += ff(n2(x)) with plain RMS norms: the `pre_norm` block with a token shift
(the mixer reads h + (h' - h) * w, h' the normed row of the token before).  Mixers: grouped-query attention with
biases, a rotation of halves, queries and keys over their root mean square, a score cap, a window plus pooled blocks
before it, and heads whose softmax weights are mixed by a matrix; attention through a cached latent with a latent for
the queries too, a rotation of neighbouring pairs, a window and a sigmoid gate per head; or a state-space mixer.
Feed-forward: a biased layer with the exact gelu, a mixture of experts (clamped, quick-gelu gated) whose router has a
bias and weighs by the softmax over the chosen logits, with a gated shared expert; or none.  A layer with
`weights_of: j` is a second run of layer j's parts with a cache and states of its own: a schedule entry, no tensors.
Tensor names: embed, head, final.norm, l<i>.norm1/.norm2/.shift, l<i>.mix.{q,k,v}(.b), .talk, .o;
l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,g,o}; l<i>.mix.{in,conv,conv.b,dt_bias,A_log,D,norm,o};
l<i>.mlp.{up,down}(.b) or l<i>.mlp.router(.b), l<i>.mlp.e<k>.{gate,up,down}, l<i>.mlp.shared.{gate,up,down,sg}.
"""
from ..config.vogunex import VogunexConfig
from ..registry import register_architecture
from .spec import LayerSpec, ModelSpec, ScheduleEntry


def _mixer(c, l):
    D, m = c.hidden_size, l.mixer
    if l.type == "attention":
        position = ("rope", {"rotary_dim": m.rot_dims, "theta": m.rot_base, "pairing": "halves"}) if m.rot_dims else ("none", {})
        return ("attention", {"hidden_size": D, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                              "value_dim": m.vdim, "query_scale": m.scale, "softcap": m.softcap, "window": m.window,
                              "position": position, "tensors": ("q", "k", "v", "o"), "bias_suffix": ".b",
                              "unit_norm_eps": c.norm_eps, "pool": m.pool, "talk": "talk"})
    if l.type == "latent_attention":
        position = ("rope", {"rotary_dim": m.rot_dims, "theta": m.rot_base, "pairing": "neighbours"}) if m.rot_dims else ("none", {})
        return ("latent_attention", {"hidden_size": D, "num_heads": m.heads, "nope_dim": m.dim, "rope_dim": m.rot_dim,
                                     "value_dim": m.vdim, "latent_rank": m.kv_rank, "scale": m.scale, "latent_eps": c.norm_eps,
                                     "position": position, "query_rank": m.q_rank, "window": m.window, "output_gate": "g",
                                     "precise_weights": True})
    return ("state_space", {"hidden_size": D, "num_heads": m.heads, "head_dim": m.vdim, "state_size": m.state,
                            "groups": m.groups, "conv_taps": m.conv, "norm_groups": m.norm_groups, "norm_eps": c.norm_eps})


def _feed_forward(c, f):
    D = c.hidden_size
    if f is None:
        return None
    if f.kind == "dense":
        return ("biased_mlp", {"hidden_size": D, "intermediate_size": f.ff, "activation": "gelu_erf",
                               "tensors": ("up", "down"), "bias_suffix": ".b"})
    shared = None if f.shared_ff is None else (
        "gated_mlp", {"hidden_size": D, "intermediate_size": f.shared_ff, "activation": "quick_gelu", "limit": f.shared_limit,
                      "up_shift": 1.0, "tensors": ("gate", "up", "down"), "prefix": "shared."})
    return ("routed_experts", {"hidden_size": D, "intermediate_size": f.ff, "n_experts": f.experts, "top": f.top,
                               "limit": f.limit, "gate_alpha": 1.702, "up_shift": 1.0, "renormalize": True,
                               "router_bias": "router.b", "shared": shared,
                               "shared_gate": None if shared is None else "shared.sg"})


def build_spec(c: VogunexConfig) -> ModelSpec:
    D = c.hidden_size
    norm = ("rms_norm", {"size": D, "eps": c.norm_eps, "tensor": "", "init": "gain"})
    layers, place, schedule = [], {}, []
    for i, l in enumerate(c.layers):
        if l.weights_of is not None:
            continue
        p = f"l{i}."
        ff = _feed_forward(c, l.mlp)
        prefixes = {"mixer": p + "mix.", "pre_mixer_norm": p + "norm1", "block": p}
        if ff is not None:
            prefixes.update({"feed_forward": p + "mlp.", "pre_ff_norm": p + "norm2"})
        place[i] = len(layers)
        layers.append(LayerSpec(block=("pre_norm", {"token_shift": "shift"}), mixer=_mixer(c, l), feed_forward=ff, norm=norm,
                                prefixes=prefixes))
    for i, l in enumerate(c.layers):
        schedule.append(ScheduleEntry(place[i if l.weights_of is None else l.weights_of]))
    return ModelSpec(
        architecture=c.architecture, hidden_size=D, vocab_size=c.vocab_size,
        embedding=("scaled_embedding", {"vocab_size": c.vocab_size, "hidden_size": D, "scale": c.embedding_scale, "tensor": ""}),
        embedding_prefix="embed", layers=layers, schedule=schedule,
        final_norm=norm, final_norm_prefix="final.norm",
        head=("linear_head", {"vocab_size": c.vocab_size, "hidden_size": D, "softcap": None, "tensor": ""}),
        head_prefix="head", stop_ids=())


register_architecture(VogunexConfig.architecture, VogunexConfig, build_spec)
