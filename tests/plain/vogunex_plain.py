"""Vogunex, plainly: every mechanism as one slow function in float64, written from the design's equations.

Nothing here is shared with the product path.  A sequence is a matrix [n, width] of inputs at positions 0 .. n - 1;
`W` maps tensor names to float64 tensors, `p` is a name prefix ("l3.mix.").
"""
import json
import math
import os

import torch
from safetensors import safe_open

F = torch.float64


def read_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    W = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            W[k] = f.get_tensor(k).to(F)
    return cfg, W


def over_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def turn(x, base, dims, neighbours):
    """x [n, heads, d]: the first `dims` elements of every head turn by the row's position; pair i is (i, i + dims / 2),
    or (2i, 2i + 1) with `neighbours`; angle = position * base^(-2i / dims)."""
    n = x.shape[0]
    out = x.clone()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if neighbours else (i, i + dims // 2)
        ang = torch.arange(n, dtype=F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        out[..., a] = x[..., a] * c - x[..., b] * s
        out[..., b] = x[..., b] * c + x[..., a] * s
    return out


def token_shift(h, w):
    """h_t + (h_(t-1) - h_t) * w, with zeros before the first token."""
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=F), h[:-1]])
    return h + (before - h) * w


def pooled_window_weights(q, k, scale, softcap, size, pool):
    """q [n, d], k [n, d] of one head.  Returns (weights on the pooled blocks [n, n // pool], weights on the tokens
    [n, n]) of one softmax, and the block keys are the means of the blocks' keys."""
    n = q.shape[0]
    nb = n // pool if pool else 0
    kb = k[:nb * pool].reshape(nb, pool, -1).mean(1) if nb else torch.zeros(0, k.shape[1], dtype=F)
    s = torch.cat([q @ kb.T, q @ k.T], dim=1) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    i, j, b = torch.arange(n)[:, None], torch.arange(n)[None], torch.arange(nb)[None]
    seen = torch.cat([b * pool + pool - 1 <= i - size, (i - j >= 0) & (i - j < size)], dim=1)       # blocks, then tokens
    w = torch.softmax(s.masked_fill(~seen, -math.inf), dim=1)
    return w[:, :nb], w[:, nb:]


def attention(h, W, p, m, eps):
    n, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(n, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(n, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(n, G, dv)
    q = over_rms(turn(q, m["rot"]["base"], m["rot"]["dims"], False), eps)
    k = over_rms(turn(k, m["rot"]["base"], m["rot"]["dims"], False), eps)
    size, pool = m["mask"]["size"], m["mask"].get("pool") or 0
    per_head = [pooled_window_weights(q[:, g], k[:, g // (H // G)], m["scale"], m.get("softcap"), size, pool) for g in range(H)]
    talk = W[p + "talk"]
    out = torch.zeros(n, H, dv, dtype=F)
    nb = n // pool if pool else 0
    for hh in range(H):
        c = hh // (H // G)
        wb = sum(talk[hh, g] * per_head[g][0] for g in range(H))
        wt = sum(talk[hh, g] * per_head[g][1] for g in range(H))
        vb = v[:nb * pool, c].reshape(nb, pool, dv).mean(1) if nb else torch.zeros(0, dv, dtype=F)
        out[:, hh] = wb @ vb + wt @ v[:, c]
    return out.reshape(n, H * dv) @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    n, H, d, dr, dv, R = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = over_rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).reshape(n, H, d + dr)
    down = h @ W[p + "dkv"].T
    c = over_rms(down[:, :R], eps) * W[p + "dkv.norm"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    qr = turn(q[..., d:], base, dims, True)
    kr = turn(down[:, None, R:], base, dims, True)[:, 0]
    kn = (c @ W[p + "uk"].T).reshape(n, H, d)
    v = (c @ W[p + "uv"].T).reshape(n, H, dv)
    gate = torch.sigmoid(h @ W[p + "g"].T)
    i, j = torch.arange(n)[:, None], torch.arange(n)[None]
    seen = (i - j >= 0) & (i - j < m["mask"]["size"])
    out = torch.zeros(n, H, dv, dtype=F)
    for hh in range(H):
        s = (q[:, hh, :d] @ kn[:, hh].T + qr[:, hh] @ kr.T) * m["scale"]
        out[:, hh] = (torch.softmax(s.masked_fill(~seen, -math.inf), dim=1) @ v[:, hh]) * gate[:, hh:hh + 1]
    return out.reshape(n, H * dv) @ W[p + "o"].T


def mamba2(h, W, p, m, eps):
    n, H, P, N, G, taps = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=F), xbc])
    conv = W[p + "conv.b"] + sum(padded[t:t + n] * W[p + "conv"][:, t] for t in range(taps))
    conv = conv * torch.sigmoid(conv)
    x, B, C = conv[:, :inner].reshape(n, H, P), conv[:, inner:inner + G * N].reshape(n, G, N), conv[:, inner + G * N:].reshape(n, G, N)
    step = torch.log1p(torch.exp(dt + W[p + "dt_bias"]))
    y = torch.zeros(n, H, P, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, P, dtype=F)
        for t in range(n):
            S = torch.exp(-torch.exp(W[p + "A_log"][hh]) * step[t, hh]) * S + step[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + W[p + "D"][hh] * x[t, hh]
    y = y.reshape(n, inner) * (z * torch.sigmoid(z))
    parts = m["norm_groups"]
    y = over_rms(y.reshape(n, parts, inner // parts), eps).reshape(n, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def clamped_expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def router_choice(h, W, p, top):
    """(chosen experts [n, top], their weights): the largest logits, softmax over those alone."""
    z = h @ W[p + "router"].T + W[p + "router.b"]
    order = torch.argsort(-z, dim=1, stable=True)[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), dim=1)


def feed_forward(h, W, p, f):
    if f["kind"] == "dense":
        a = h @ W[p + "up"].T + W[p + "up.b"]
        a = 0.5 * a * (1.0 + torch.erf(a / math.sqrt(2.0)))
        return a @ W[p + "down"].T + W[p + "down.b"]
    chosen, weight = router_choice(h, W, p, f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(chosen.shape[1]):
            out[t] += weight[t, j] * clamped_expert(h[t:t + 1], W, p + f"e{int(chosen[t, j])}.", f["expert"]["limit"])[0]
    if f.get("shared"):
        out = out + clamped_expert(h, W, p + "shared.", f["shared"]["limit"]) * torch.sigmoid(h @ W[p + "shared.sg"].T)
    return out


MIXERS = {"attention": attention, "latent_attention": latent_attention, "mamba2": mamba2}


def forward(cfg, W, tokens, layers_out=None):
    """Logits [n, vocab] of one sequence."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens))] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{layer.get('weights_of', i)}."
        h = token_shift(over_rms(x, eps) * W[p + "norm1"], W[p + "shift"])
        x = x + MIXERS[layer["type"]](h, W, p + "mix.", layer["mixer"], eps)
        if layer["mlp"] is not None:
            x = x + feed_forward(over_rms(x, eps) * W[p + "norm2"], W, p + "mlp.", layer["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return (over_rms(x, eps) * W["final.norm"]) @ W["head"].T


def greedy_generate(cfg, W, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        z = forward(cfg, W, toks)[-1]
        best = int(torch.argmax(z))                      # the smallest id among equals
        toks.append(best)
        out.append(best)
    return out
