"""Plain Besulix: whole sequences, no cache, one function per mechanism, float64 by default.

Written from the design's equations; it shares no code with the engine.  Every function takes its sizes and
constants as arguments.  A model is a config dict (the config.json object) and {tensor name: tensor}.

  embedding  x = unit_rms(E[token]) * w_e
  layer      x <- x + mixer(n1(x));  x <- x + ff(n2(x))  (the second only when the layer has a feed-forward),
             n(v) = v / sqrt(mean(v^2) + eps) * w
  mixers     "mlstm": a matrix memory per head with exponential input gate, sigmoid forget gate (both capped by a
             tanh) and a running maximum that keeps the exponentials in range;
             "parallel": grouped-query attention in chunks, with biased projections, a rotation of part of each query
             and key head, values rotated by their own position (the output rotated back by the query's), a
             temperature per head and a sink in the softmax, beside a time-mixing recurrence with a decay per channel
             computed from the input and a bonus for the present token; the two outputs are added with fixed weights
  ff         g = min(W_g x, L), u = clamp(W_u x, -L, L), W_d (g sigmoid(1.702 g) (u + 1))
  output     final norm, head, C tanh(z / C)
"""
import json
import math
import os
import struct

import torch

_DT = {"F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16, "F64": torch.float64,
       "I32": torch.int32, "I64": torch.int64}


def read_folder(folder, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    out = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        raw = f.read()
    n = struct.unpack("<Q", raw[:8])[0]
    hdr = json.loads(raw[8:8 + n])
    for name, meta in hdr.items():
        if name == "__metadata__":
            continue
        s, e = meta["data_offsets"]
        t = torch.frombuffer(bytearray(raw[8 + n + s:8 + n + e]), dtype=_DT[meta["dtype"]]).reshape(meta["shape"])
        out[name] = t.to(dtype) if t.dtype.is_floating_point else t
    return cfg, out


# ---- small functions ----------------------------------------------------------------------------------------------
def unit_rms(v, eps):
    """v [..., n] over its root mean square, eps inside the root."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def log_sigmoid(z):
    return -(torch.log1p(torch.exp(-z.abs())) + torch.clamp(-z, min=0.0))


# ---- rotation -------------------------------------------------------------------------------------------------------
def turn_halves(x, pos, base, dims, sign=1.0):
    """x [T, heads, n]: element i < dims / 2 turns with element i + dims / 2 by sign * pos * base^(-2i / dims); elements
    from dims on stay."""
    half = dims // 2
    out = x.clone()
    for i in range(half):
        f = float(base) ** (-2.0 * i / dims)
        a = sign * pos.to(x.dtype) * f                         # [T]
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


# ---- the chunked attention ("left") ----------------------------------------------------------------------------------
def chunk_sink_attention(h, w, p, m):
    """h [T, D] -> [T, D].  m: heads, kv_heads, dim, vdim, scale, rot {base, dims}, mask {size}."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    base, rd, C = m["rot"]["base"], m["rot"]["dims"], m["mask"]["size"]
    pos = torch.arange(T)
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, dk)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, dk)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, dv)
    q, k = turn_halves(q, pos, base, rd), turn_halves(k, pos, base, rd)
    v = turn_halves(v, pos, base, dv)                          # a value carries its own position
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        temp, sink = w[p + "temp"][hd], w[p + "sink"][hd]
        for i in range(T):
            first = (i // C) * C
            s = (k[first:i + 1, g] @ q[i, hd]) * m["scale"] * temp
            top = torch.maximum(s.max(), sink)
            e = torch.exp(s - top)
            out[i, hd] = (e[:, None] * v[first:i + 1, g]).sum(0) / (e.sum() + torch.exp(sink - top))
    out = turn_halves(out, pos, base, dv, sign=-1.0)           # and is read in the query's frame
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ---- the time-mixing recurrence ("right") ---------------------------------------------------------------------------
def time_mix(h, w, p, m, eps):
    """h [T, D] -> [T, D].  m: heads, dim."""
    T, D = h.shape
    H, d = m["heads"], m["dim"]
    before = torch.cat([torch.zeros((1, D), dtype=h.dtype), h[:-1]])
    mix = {s: h + (before - h) * w[p + "mu." + s] for s in "rkvgw"}
    r = (mix["r"] @ w[p + "r"].T).reshape(T, H, d)
    k = (mix["k"] @ w[p + "k"].T).reshape(T, H, d)
    v = (mix["v"] @ w[p + "v"].T).reshape(T, H, d)
    gate = silu(mix["g"] @ w[p + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).reshape(T, H, d)
    u = w[p + "u"]                                             # [H, d]
    S = torch.zeros((H, d, d), dtype=h.dtype)                  # [head, key channel, value channel]
    out = torch.zeros((T, H, d), dtype=h.dtype)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S + u[:, :, None] * kv, r[t])
        S = decay[t][:, :, None] * S + kv
    out = unit_rms(out, eps).reshape(T, H * d) * w[p + "norm"] * gate
    return out @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    return m["left_scale"] * chunk_sink_attention(h, w, p + "left.", m["left"]) + \
        m["right_scale"] * time_mix(h, w, p + "right.", m["right"], eps)


# ---- the matrix memory ("mlstm") ------------------------------------------------------------------------------------
def matrix_memory(h, w, p, m, eps):
    """h [T, D] -> [T, D].  m: heads, dim, vdim, gate_cap."""
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, dk)
    v = (h @ w[p + "v"].T).reshape(T, H, dv)
    gi = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)                      # [T, H], log of the input gate
    gf = log_sigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))         # log of the forget gate
    S = torch.zeros((H, dk, dv), dtype=h.dtype)
    n = torch.zeros((H, dk), dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    out = torch.zeros((T, H, dv), dtype=h.dtype)
    for t in range(T):
        new = torch.maximum(gf[t] + mx, gi[t])
        keep, take = torch.exp(gf[t] + mx - new), torch.exp(gi[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
    out = unit_rms(out, eps).reshape(T, H * dv) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


# ---- feed-forward ------------------------------------------------------------------------------------------------------
def clamped_ff(h, w, p, m):
    L = m["limit"]
    g = torch.clamp(h @ w[p + "gate"].T, max=L)
    u = torch.clamp(h @ w[p + "up"].T, min=-L, max=L)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


# ---- the model ---------------------------------------------------------------------------------------------------------
def forward(cfg, w, tokens, layers_out=None):
    """tokens: list of ids of one sequence -> logits [T, vocab].  layers_out: a list that receives the stream after
    every layer."""
    eps = cfg["norm"]["eps"]
    x = unit_rms(w["embed"][torch.tensor(tokens, dtype=torch.long)], eps) * w["embed.norm"]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = unit_rms(x, eps) * w[p + "norm1"]
        if layer["type"] == "mlstm":
            x = x + matrix_memory(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            x = x + parallel_mixer(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer["mlp"] is not None:
            x = x + clamped_ff(unit_rms(x, eps) * w[p + "norm2"], w, p + "mlp.", layer["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    x = unit_rms(x, eps) * w["final.norm"]
    z = x @ w["head"].T
    cap = cfg.get("logit_softcap")
    return z if cap is None else cap * torch.tanh(z / cap)


def greedy_generate(cfg, w, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        z = forward(cfg, w, toks)[-1]
        tok = int(torch.nonzero(z == z.max())[0])
        out.append(tok)
        toks.append(tok)
    return out
