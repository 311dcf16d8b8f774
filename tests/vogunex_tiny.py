"""The tests' own small Vogunex configurations.

P mixes everything: attention layers with values larger and smaller than keys, a rotation of part of a head and of all
of it, windows shorter than a cache page and windows that are no multiple of one, pooled blocks of 3 and 5 positions,
several and single kv heads; latent attentions with rotated parts that turn wholly and partly; a state-space layer with
groups and norm groups; dense layers, mixtures with and without a shared expert, layers without a feed-forward; layers
that run on another layer's weights, one of them on a later layer's.
Q takes the values that hide faults when they are 1 or equal: one head everywhere, equal key and value sizes, no
rotation, blocks of one position, a window of one, one expert of which one is chosen, a mixture's top equal to its
experts, a width that no matrix-core kernel takes, no score cap.
S is P's shape with the attentions' scores scaled up until a softmax picks single keys: a key that is lost, a window's
edge one place off or a block seen too early then changes the logits by far more than any tolerance.
"""
import json
import os

from trapetum_amd.config import VogunexConfig
from trapetum_amd.weights import write_model_folder


def att(heads, kv, dim, vdim, scale, cap, base, dims, size, pool):
    mask = {"size": size} if pool is None else {"pool": pool, "size": size}
    return {"dim": dim, "heads": heads, "kv_heads": kv, "mask": mask, "rot": {"base": base, "dims": dims}, "scale": scale,
            "softcap": cap, "vdim": vdim}


def lat(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, dims, size):
    return {"dim": dim, "heads": heads, "kv_rank": kv_rank, "mask": {"size": size}, "q_rank": q_rank,
            "rot": {"base": base, "dims": dims}, "rot_dim": rot_dim, "scale": scale, "vdim": vdim}


def ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def moe(ff, limit, experts, top, shared=None):
    d = {"expert": {"ff": ff, "limit": limit}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared is not None:
        d["shared"] = {"ff": shared[0], "limit": shared[1]}
    return d


def layer(kind, mixer, mlp, weights_of=None):
    d = {"mixer": mixer, "mlp": mlp, "type": kind}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def config_p(scale=1.0):
    a0 = att(4, 2, 16, 24, 0.3 * scale, 30.0, 500.0, 8, 11, 3)
    a1 = att(3, 3, 24, 8, 0.25 * scale, 12.0, 77.0, 24, 20, 5)
    l0 = lat(3, 16, 8, 12, 24, 20, 0.25 * scale, 1000.0, 8, 13)
    l1 = lat(2, 8, 16, 16, 16, 12, 0.3 * scale, 50.0, 12, 18)
    m0 = moe(40, 1.5, 5, 2, shared=(24, 0.8))
    return {"architecture": "Vogunex", "embedding": {"scale": 0.7},
            "layers": [layer("attention", a0, dense(72)),
                       layer("latent_attention", l0, m0),
                       layer("attention", a0, dense(72), weights_of=0),
                       layer("mamba2", ssm(4, 12, 16, 2, 4, 3), moe(33, 2.0, 3, 1)),
                       layer("attention", a1, None, weights_of=6),
                       layer("latent_attention", l1, None),
                       layer("attention", a1, None),
                       layer("latent_attention", l0, m0, weights_of=1)],
            "norm": {"eps": 1e-5}, "vocab": 211, "width": 96}


def config_q():
    return {"architecture": "Vogunex", "embedding": {"scale": 1.0},
            "layers": [layer("attention", att(1, 1, 12, 12, 0.3, None, 10000.0, 0, 1, 1), moe(20, 1.0, 1, 1)),
                       layer("latent_attention", lat(1, 10, 4, 10, 6, 6, 0.3, 100.0, 0, 1000), dense(30)),
                       layer("mamba2", ssm(1, 10, 4, 1, 1, 1), moe(18, 3.0, 2, 2, shared=(18, 3.0))),
                       layer("attention", att(2, 2, 10, 10, 0.3, 5.0, 10.0, 10, 1000, None), None)],
            "norm": {"eps": 1e-6}, "vocab": 97, "width": 50}


CONFIGS = {"P": (config_p(), dict(seed=41, sigma=0.12, sigma_norm=0.3)),
           "Q": (config_q(), dict(seed=42, sigma=0.15, sigma_norm=0.2)),
           "S": (config_p(scale=12.0), dict(seed=43, sigma=0.12, sigma_norm=0.3))}


def make_folder(tmp_path, which):
    cfg, init = CONFIGS[which]
    folder = os.path.join(str(tmp_path), f"vogunex_{which}")
    write_model_folder(VogunexConfig.from_dict(cfg), folder, **init)
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == cfg                     # the configuration writes back what it read
    return folder


def draw(rng):
    """A configuration drawn at random: sizes, head counts, windows, blocks, constants and the order of layers."""
    def attention():
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 12, 16, 20, 32])
        return att(kv * rng.choice([1, 2, 3]), kv, dim, rng.choice([8, 12, 16, 24, 40]), rng.choice([0.2, 0.35]),
                   rng.choice([None, 8.0, 25.0]), rng.choice([10.0, 3000.0]), rng.choice([0, dim // 2 // 2 * 2, dim // 4 * 4, dim]),
                   rng.choice([1, 2, 7, 16, 23, 64]), rng.choice([None, 1, 2, 4, 7]))

    def latent():
        rot_dim = rng.choice([2, 4, 8, 16])
        return lat(rng.choice([1, 2, 5]), rng.choice([4, 8, 16, 24]), rot_dim, rng.choice([4, 8, 20]), rng.choice([6, 14, 32]),
                   rng.choice([5, 16, 24]), rng.choice([0.2, 0.4]), rng.choice([20.0, 5000.0]), rng.choice([0, rot_dim // 4 * 2, rot_dim]),
                   rng.choice([1, 3, 16, 30, 500]))

    def state_space():
        groups = rng.choice([1, 2])
        heads = groups * rng.choice([1, 2, 3])
        vdim = rng.choice([4, 8, 12])
        parts = rng.choice([n for n in (1, 2, 3, 4) if (heads * vdim) % n == 0])
        return ssm(heads, vdim, rng.choice([4, 8, 16]), groups, rng.choice([1, 2, 4]), parts)

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return dense(rng.choice([16, 40, 72]))
        experts = rng.choice([1, 2, 4, 7])
        return moe(rng.choice([8, 24, 40]), rng.choice([0.5, 2.0, 7.0]), experts, rng.randint(1, min(experts, 3)),
                   rng.choice([None, (rng.choice([8, 32]), rng.choice([0.7, 3.0]))]))
    makers = {"attention": attention, "latent_attention": latent, "mamba2": state_space}
    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(list(makers))
        layers.append(layer(kind, makers[kind](), mlp()))
    own = len(layers)
    for _ in range(rng.randint(0, 2)):                  # runs on another layer's weights, anywhere in the order
        j = rng.randrange(own)
        layers.insert(rng.randint(0, len(layers)), dict(layers[[i for i, l in enumerate(layers) if "weights_of" not in l][j]], weights_of=None))
    # name the layers that lend their weights by their final places
    firsts = {}
    for i, l in enumerate(layers):
        if "weights_of" not in l:
            firsts[json.dumps({k: l[k] for k in ("mixer", "mlp", "type")}, sort_keys=True)] = i
    for l in layers:
        if "weights_of" in l:
            l["weights_of"] = firsts[json.dumps({k: l[k] for k in ("mixer", "mlp", "type")}, sort_keys=True)]
    return {"architecture": "Vogunex", "embedding": {"scale": rng.choice([0.5, 1.0, 2.0])}, "layers": layers,
            "norm": {"eps": rng.choice([1e-6, 1e-5])}, "vocab": rng.choice([64, 101, 300]), "width": rng.choice([24, 40, 64, 100])}
