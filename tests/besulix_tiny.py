"""The tests' own small Besulix configurations.

P mixes everything: parallel layers whose attention has values larger and smaller than keys, a rotation of part of a
head and of all of it, chunks shorter than a cache page and chunks that are no multiple of one, several and single kv
heads; time-mixing heads of a size that is no power of two and of more channels than a wave has lanes; matrix memories
whose keys and values differ in size, with more than 64 key rows and more than 64 value columns; layers with and
without a feed-forward, limits that cut often and seldom.
Q takes the values that hide faults when they are 1 or equal: one head everywhere, equal key and value sizes, no
rotation of queries and keys, chunks longer than any test sequence, both weights of the sum 1, no cap on the logits, a
width that no matrix-core kernel takes.
S is P's shape with the attentions' scores scaled up until a softmax picks single keys: a key that is lost, or a chunk's
edge one place off, then changes the logits by far more than any tolerance.
"""
import json
import os

from trapetum_amd.config import BesulixConfig
from trapetum_amd.weights import write_model_folder


def _left(heads, kv_heads, dim, vdim, scale, base, dims, chunk):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims},
            "mask": {"size": chunk}}


def _par(left, heads, dim, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": ls, "right": {"heads": heads, "dim": dim}, "right_scale": rs},
            "mlp": mlp}


def _mem(heads, dim, vdim, cap, mlp):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def _ff(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def config_p(scale=1.0):
    return {"architecture": "Besulix", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
            "layers": [_par(_left(4, 2, 16, 24, 0.2 * scale, 500.0, 8, 8), 3, 20, 0.7, 1.1, _ff(72, 0.8)),
                       _mem(2, 24, 40, 6.0, None),
                       _par(_left(3, 3, 24, 8, 0.25 * scale, 77.0, 24, 20), 1, 72, 1.2, 0.6, None),
                       _mem(3, 72, 70, 9.0, _ff(56, 2.0)),
                       _par(_left(2, 1, 32, 32, 0.15 * scale, 1000.0, 16, 16), 2, 32, 0.9, 0.8, _ff(40, 0.5))]}


def config_q():
    return {"architecture": "Besulix", "vocab": 97, "width": 50, "norm": {"eps": 1e-6}, "logit_softcap": None,
            "layers": [_mem(1, 16, 16, 15.0, _ff(30, 1.0)),
                       _par(_left(1, 1, 12, 12, 0.3, 10000.0, 0, 1000), 1, 16, 1.0, 1.0, None)]}


CONFIGS = {"P": (config_p(), dict(seed=31, sigma=0.12, sigma_norm=0.3)),
           "Q": (config_q(), dict(seed=32, sigma=0.15, sigma_norm=0.2)),
           "S": (config_p(scale=14.0), dict(seed=33, sigma=0.12, sigma_norm=0.3))}


def make_folder(tmp_path, which):
    cfg, init = CONFIGS[which]
    folder = os.path.join(str(tmp_path), f"besulix_{which}")
    write_model_folder(BesulixConfig.from_dict(cfg), folder, **init)
    with open(os.path.join(folder, "config.json")) as f:
        assert json.load(f) == cfg                     # the configuration writes back what it read
    return folder


def make_long_memory_folder(tmp_path):
    """P with time-mixing decays of exp(-exp(-6)) whatever the input, and forget gates of sigmoid(6) at least: the
    states keep what the first tokens wrote."""
    import torch
    from safetensors.torch import load_file, save_file
    folder = make_folder(tmp_path, "P")
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    for name in list(t):
        if name.endswith(".right.w0") or name.endswith(".mix.f.b"):
            t[name] = torch.full_like(t[name], -6.0 if name.endswith("w0") else 6.0)
        elif name.endswith(".right.w2") or name.endswith(".mix.f"):
            t[name] = torch.zeros_like(t[name])
    save_file(t, path)
    return folder


def early_token_decides(model, cfg, pcfg, pw, tol, n=45, first=30):
    import torch

    from .plain import besulix_plain as plain
    from .tiny import random_tokens
    a = random_tokens(n, cfg.vocab_size, 61)
    b = list(a)
    b[2] = (a[2] + 1) % cfg.vocab_size
    ra, rb = plain.forward(pcfg, pw, a)[-1], plain.forward(pcfg, pw, b)[-1]
    assert float((ra - rb).norm() / ra.norm()) > 1e-2           # the early token does decide
    cache = model.new_cache(max_tokens=4 * n, page_size=16)
    outs = []
    for toks in (a, b):
        s = cache.acquire()
        model.step(cache, [s], toks[:first], counts=[first], want=[])
        outs.append(torch.cat([model.step(cache, [s], [t]) for t in toks[first:]])[-1].double().cpu())
        cache.release(s)
    assert float(((outs[0] - outs[1]) - (ra - rb)).norm() / (ra - rb).norm()) < tol
