"""Plain torch references of the kernel library, one function per kernel, same signatures.

Two uses: the GPU tests compare each HIP kernel with its function here, and the
CPU tests run the engine's host logic (cache, step, batching, generation) on
these instead of the HIP library.  fp32 arithmetic, rounded once to the output
dtype, like the kernels.  None of this is on the product path.
"""
import math

import torch

GROUP = 16          # rows of gate, then rows of up, alternate in groups of this many


def pack_gate_up(w_gate, w_up):
    i, k = w_gate.shape
    ip = -(-i // GROUP) * GROUP
    g = torch.zeros((ip, k), dtype=w_gate.dtype, device=w_gate.device)
    u = torch.zeros_like(g)
    g[:i], u[:i] = w_gate, w_up
    return torch.stack([g.reshape(-1, GROUP, k), u.reshape(-1, GROUP, k)], dim=1).reshape(2 * ip, k).contiguous()


def embed_rows(tokens, table, scale):
    return table[tokens.long()].float() * scale


def _norm(x, gain, eps, groups=1):
    x = x.float()
    parts = x.reshape(x.shape[0], groups, -1)
    parts = parts * torch.rsqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * gain


def rms_norm(x, gain, eps, out_dtype, groups=1):
    return _norm(x, gain, eps, groups).to(out_dtype)


def add_rms_norm(stream, rows, gain_post, eps_post, gain_next, eps_next, out_dtype, groups=1):
    if hasattr(rows, "slices"):
        rows = rows.slices.sum(0)
    t = rows.float() if gain_post is None else _norm(rows, gain_post, eps_post, groups)
    stream += t
    if gain_next is None:
        return None
    return _norm(stream, gain_next, eps_next, groups).to(out_dtype)


def scale_rows(x, scale):
    x *= scale


def causal_conv(stream, w, state, slot_ids, cu_rows, row_seq, out_dtype, residual=True, one_row_each=False, w_t=None):
    """out_t = (x_t) + sum_j w[:, j] x_(t - taps + 1 + j); rows before the step come from state[slot] ([taps - 1, D],
    oldest first), which then takes the last taps - 1 rows of (state, step)."""
    taps = w.shape[1]
    out = torch.empty(stream.shape, dtype=torch.float32, device=stream.device)
    for i in range(len(cu_rows) - 1):
        a, b, slot = int(cu_rows[i]), int(cu_rows[i + 1]), int(slot_ids[i])
        hist = stream[a:b] if taps == 1 else torch.cat([state[slot], stream[a:b]])
        acc = stream[a:b].clone() if residual else torch.zeros_like(stream[a:b])
        for j in range(taps):
            acc += w[:, j] * hist[j:j + (b - a)]
        out[a:b] = acc
        if taps > 1:
            state[slot] = hist[hist.shape[0] - (taps - 1):].clone()
    return out.to(out_dtype)


def latent_prepare(proj, H, dn, dr, R, gain, eps, inv_freq, rot, row_seq, row_pos, new_len, table, pool, rows_cap,
                   own=True, out_dtype=None, tail=None, write=True):
    """proj [M, H (dr + dn) (+ dr + R)]: per head [rotated | unrotated] query parts, then [key part | latent] (or these as
    rows of their own, `tail`).  write False: the step's rows are returned, not cached.
    Returns q [M, H (dr + R)] with every head's first dr elements set (the rotated query part; the rest is for
    `head_linear`), and the step's rows [rope(key part) | rmsnorm(latent) * gain] (None when own is false), which are
    also written into the cache."""
    m = proj.shape[0]
    out_dtype = out_dtype or proj.dtype
    q = torch.zeros((m, H, dr + R), dtype=out_dtype, device=proj.device)
    qr = proj[:, :H * (dr + dn)].float().reshape(m, H, dr + dn)[:, :, :dr]
    q[:, :, :dr] = _rotate(qr, row_pos, inv_freq, rot).to(out_dtype)
    mine = None
    if own:
        tail = proj[:, H * (dr + dn):].float() if tail is None else tail.float()
        r = _rotate(tail[:, None, :dr], row_pos, inv_freq, rot)[:, 0]
        c = tail[:, dr:]
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * gain
        mine = torch.cat([r, c], dim=-1).to(out_dtype)
        if write:
            _cache_rows(mine, mine, row_seq, row_pos, new_len, table, pool, pool, rows_cap)
    return q.reshape(m, H * (dr + R)), mine


def head_linear(x, w, out=None):
    """x [M, H, K] (any strides), w [H, N, K] -> out [M, H, N] (a view to fill, or a new tensor of x's dtype)."""
    y = torch.einsum("mhk,hnk->mhn", x.float(), w.float())
    if out is None:
        return y.to(x.dtype).contiguous()
    out.copy_(y.to(out.dtype))
    return out


def route_top(logits, top, renormalize=False, score="softmax"):
    s = torch.softmax(logits.float(), dim=-1) if score == "softmax" else torch.sigmoid(logits.float())
    order = torch.argsort(-s, dim=-1, stable=True)[:, :top]
    w = torch.gather(s, 1, order)
    if renormalize:
        w = w / w.sum(-1, keepdim=True)
    return order.to(torch.int32), w


def expert_ffn(x, chosen, weights, w_gate_up, w_down, limit, alpha, shift, weight_input=False, out=None):
    """fp32 [M, D]: sum over a token's chosen experts, in the order they were chosen, of weight * expert(x), or
    (weight_input) of expert(weight * x): gate and up sums times the weight, before the clamps."""
    m, ff = x.shape[0], w_gate_up.shape[1] // 2
    limit = float("inf") if limit is None else limit
    res = torch.zeros((m, w_down.shape[1]), dtype=torch.float32, device=x.device)
    for k in range(chosen.shape[1]):
        for r in range(m):
            e = int(chosen[r, k])
            gu = w_gate_up[e].float() @ x[r].float()
            if weight_input:
                gu = gu * weights[r, k]
            g, u = torch.clamp(gu[:ff], max=limit), torch.clamp(gu[ff:], -limit, limit)
            y = (g * torch.sigmoid(alpha * g) * (u + shift)).to(x.dtype).float()
            res[r] += (1.0 if weight_input else weights[r, k]) * (w_down[e].float() @ y)
    if out is None:
        return res
    out.copy_(res)
    return out


def linear(x, w, out_dtype, softcap=None, defer=False, bias=None, out=None):
    y = x.float() @ w.float().T
    if bias is not None:
        y = y + bias.float()
    if softcap:
        y = softcap * torch.tanh(y / softcap)
    if out is None:
        return y.to(out_dtype)
    out.copy_(y.to(out_dtype))
    return out


def _gelu_tanh(g):
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608 * (g + 0.044715 * g * g * g)))


def gated_linear(x, w_packed, inter, activation, out_dtype, limit=None, up_shift=0.0):
    """limit: the gate sum is cut at it from above and the up sum from both sides, before the activation."""
    act = {"gelu_tanh": _gelu_tanh, "silu": lambda g: g * torch.sigmoid(g), "relu": torch.relu,
           "quick_gelu": lambda g: g * torch.sigmoid(1.702 * g)}[activation]
    y = x.float() @ w_packed.float().T                     # [M, 2 * ip]
    y = y.reshape(x.shape[0], -1, 2, GROUP)
    g, u = y[:, :, 0, :].reshape(x.shape[0], -1), y[:, :, 1, :].reshape(x.shape[0], -1)
    if limit is not None:
        g, u = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
    return (act(g) * (u + up_shift))[:, :inter].to(out_dtype).contiguous()


def _rotate(x, pos, inv_freq, rotary_dim, pairing="halves"):
    """x [M, heads, hd] fp32, pos [M]."""
    if inv_freq is None or rotary_dim == 0:
        return x.clone()
    half = rotary_dim // 2
    ang = pos.float()[:, None] * inv_freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if pairing == "neighbours":                          # pair d: elements 2d and 2d + 1
        x0, x1 = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        turned = torch.stack([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1).reshape(*x.shape[:-1], rotary_dim)
        return torch.cat([turned, x[..., rotary_dim:]], dim=-1)
    x0, x1 = x[..., :half], x[..., half:rotary_dim]
    return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s, x[..., rotary_dim:]], dim=-1)


def _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
    KV, page, hd = k_pool.shape[1], k_pool.shape[2], k_pool.shape[3]
    for r in range(k.shape[0]):
        s, p = int(row_seq[r]), int(row_pos[r])
        row = p
        if rows_cap:
            if p + rows_cap < int(new_len[s]):
                continue                                  # a later row of this step lands on the same ring row
            row = p % rows_cap
        pg = int(table[s, row // page])
        assert pg >= 0
        k_pool[pg, :, row % page, :] = k[r].reshape(KV, hd)
        v_pool[pg, :, row % page, :] = v[r].reshape(KV, hd)


def rope_kv_write(q, k, v, H, KV, hd, inv_freq, rotary_dim, row_seq, row_pos, new_len, table,
                  k_pool, v_pool, rows_cap, pairing="halves", write=True):
    m = q.shape[0]
    q.copy_(_rotate(q.float().reshape(m, H, hd), row_pos, inv_freq, rotary_dim, pairing).reshape(m, H * hd).to(q.dtype))
    if k is None:
        return
    k.copy_(_rotate(k.float().reshape(m, KV, hd), row_pos, inv_freq, rotary_dim, pairing).reshape(m, KV * hd).to(k.dtype))
    if write:
        _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap)


def kv_write(k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap):
    _cache_rows(k, v, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap)


def _attend(qrow, keys, vals, scale, softcap, sink=None):
    """qrow [hd], keys/vals [n, hd], fp32.  sink: a score without key or value that joins the denominator."""
    s = (keys @ qrow) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    if sink is not None:
        return torch.softmax(torch.cat([s, sink.reshape(1).float()]), dim=0)[:-1] @ vals
    p = torch.softmax(s, dim=0)
    return p @ vals


def _first_seen(p, window, chunk):
    lo = 0 if not window else max(0, p - window + 1)
    return max(lo, (p // chunk) * chunk) if chunk else lo


def attention_prefill(q, k, v, H, KV, hd, cu_rows, max_count, scale, softcap, window, out_dtype, row_seq=None, row_pos=None,
                      cached=None, shape=0, wide_weights=False, chunk=0, head_scale=None, sink=None):
    """k, v: the step's own rows.  cached None: every sequence starts at position 0.  Else cached = (new_len, table,
    k_pool, v_pool, rows_cap): sequence i's first row stands at new_len[i] - its count, and the positions before it are
    read from the cache as it is."""
    m = q.shape[0]
    out = torch.zeros((m, H * hd), dtype=torch.float32, device=q.device)
    qf, kf, vf = q.float().reshape(m, H, hd), k.float().reshape(-1, KV, hd), v.float().reshape(-1, KV, hd)
    g = H // KV
    for i in range(len(cu_rows) - 1):
        a, b = int(cu_rows[i]), int(cu_rows[i + 1])
        start, keys, vals = 0, kf[a:b], vf[a:b]
        if cached is not None:
            new_len, table, k_pool, v_pool, rows_cap = cached
            page = k_pool.shape[2]
            start = int(new_len[i]) - (b - a)
            first = _first_seen(start, window, chunk)                    # the earliest position any query of the step sees
            pos = torch.arange(first, start)
            rows = pos % rows_cap if rows_cap else pos
            pages = table[i].long()[rows // page]
            assert (pages >= 0).all()
            keys = torch.cat([torch.zeros(first, KV, hd), k_pool[pages, :, rows % page, :].float().cpu(), kf[a:b].cpu()]).to(q.device)
            vals = torch.cat([torch.zeros(first, KV, hd), v_pool[pages, :, rows % page, :].float().cpu(), vf[a:b].cpu()]).to(q.device)
        for r in range(a, b):
            p = start + r - a
            lo = _first_seen(p, window, chunk)
            for h in range(H):
                out[r, h * hd:(h + 1) * hd] = _attend(qf[r, h], keys[lo:p + 1, h // g], vals[lo:p + 1, h // g],
                                                      scale * (float(head_scale[h]) if head_scale is not None else 1.0), softcap,
                                                      None if sink is None else sink[h])
    return out.to(out_dtype)


def decode_splits(n, KV, hd, keys):
    return 1


def attention_decode(q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window, out_dtype, max_keys=None, splits=None, head_groups=None,
                     chunk=0, head_scale=None, sink=None):
    n = q.shape[0]
    page = k_pool.shape[2]
    out = torch.zeros((n, H * hd), dtype=torch.float32, device=q.device)
    qf = q.float().reshape(n, H, hd)
    g = H // KV
    for i in range(n):
        p = int(new_len[i]) - 1
        lo = _first_seen(p, window, chunk)
        pos = torch.arange(lo, p + 1)
        rows = pos % rows_cap if rows_cap else pos
        pages = table[i].long()[rows // page]
        assert (pages >= 0).all()
        keys = k_pool[pages, :, rows % page, :].float()          # [n_keys, KV, hd]
        vals = v_pool[pages, :, rows % page, :].float()
        for h in range(H):
            out[i, h * hd:(h + 1) * hd] = _attend(qf[i, h], keys[:, h // g], vals[:, h // g],
                                                  scale * (float(head_scale[h]) if head_scale is not None else 1.0), softcap,
                                                  None if sink is None else sink[h])
    return out.to(out_dtype)


def fuses_decode_step(dtype, H, KV, hd, k_pool):
    return False


def attention_decode_step(qkv, H, KV, hd, inv_freq, rotary_dim, new_len, table, k_pool, v_pool, rows_cap, scale, softcap,
                          window, out_dtype, max_keys=None, write_kv=True, splits=None):
    """The fused decode step as its three parts: qkv float32 [n, (H + 2 KV) hd] (already summed over K slices),
    rotated in float32 and rounded once to the cache's dtype."""
    n = qkv.shape[0]
    pos = new_len.to(torch.int32) - 1
    q = _rotate(qkv[:, :H * hd].float().reshape(n, H, hd), pos, inv_freq, rotary_dim).reshape(n, H * hd).to(k_pool.dtype)
    if write_kv:
        k = _rotate(qkv[:, H * hd:(H + KV) * hd].float().reshape(n, KV, hd), pos, inv_freq, rotary_dim).to(k_pool.dtype)
        v = qkv[:, (H + KV) * hd:].reshape(n, KV, hd).to(k_pool.dtype)
        page = k_pool.shape[2]
        for i in range(n):
            row = int(pos[i]) % rows_cap if rows_cap else int(pos[i])
            pg = int(table[i, row // page])
            assert pg >= 0
            k_pool[pg, :, row % page, :] = k[i]
            v_pool[pg, :, row % page, :] = v[i]
    return attention_decode(q, H, KV, hd, new_len, table, k_pool, v_pool, rows_cap, scale, softcap, window, out_dtype)


class SplitRows:
    """The kernel library's rows in slices, fp32 [slices, M, N]: their sum is meant."""

    def __init__(self, slices):
        self.slices = slices
        self.shape = tuple(slices.shape[1:])
        self.dtype = torch.float32


def rows(r, dtype):
    if isinstance(r, SplitRows):
        return r.slices.sum(0).to(dtype)
    return r


def conv_act(x, w_t, bias, state, slot_ids, cu_rows, row_seq, activation=None, one_row_each=False):
    """out_t = act(bias + sum_j w_t[j] x_(t - taps + 1 + j)); rows before the step come from state[slot] ([taps - 1, C],
    oldest first), which then takes the last taps - 1 rows of (state, step)."""
    taps = w_t.shape[0]
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    xf = x.float()
    for i in range(len(cu_rows) - 1):
        a, b, slot = int(cu_rows[i]), int(cu_rows[i + 1]), int(slot_ids[i])
        hist = xf[a:b] if taps == 1 else torch.cat([state[slot], xf[a:b]])
        acc = torch.zeros_like(xf[a:b]) if bias is None else bias.float().expand(b - a, -1).clone()
        for j in range(taps):
            acc += w_t[j] * hist[j:j + (b - a)]
        out[a:b] = acc
        if taps > 1:
            state[slot] = hist[hist.shape[0] - (taps - 1):].clone()
    if activation == "silu":
        out = out * torch.sigmoid(out)
    return out.to(x.dtype)


def ssd_scan(xbc, z, dt, dt_bias, a_log, skip, state, slot_ids, cu_rows, max_count, heads, groups, n_state, head_dim):
    """S <- exp(-exp(a_log) d) S + d B x^T, y = (S^T C + skip x) * silu(z), d = softplus(dt + dt_bias), row after row of
    every sequence from state[slot] [heads, n_state, head_dim], which is left updated.  float32 [M, heads head_dim]."""
    m, inner, gn = xbc.shape[0], heads * head_dim, groups * n_state
    x = xbc[:, :inner].float().reshape(m, heads, head_dim)
    B = xbc[:, inner:inner + gn].float().reshape(m, groups, n_state).repeat_interleave(heads // groups, dim=1)
    C = xbc[:, inner + gn:].float().reshape(m, groups, n_state).repeat_interleave(heads // groups, dim=1)
    d = torch.nn.functional.softplus(dt.float() + dt_bias, threshold=1e9)
    decay = torch.exp(-torch.exp(a_log)[None, :] * d)
    y = torch.empty((m, heads, head_dim), dtype=torch.float32, device=xbc.device)
    for i in range(len(cu_rows) - 1):
        slot = int(slot_ids[i])
        S = state[slot].clone()
        for r in range(int(cu_rows[i]), int(cu_rows[i + 1])):
            S = decay[r][:, None, None] * S + (d[r][:, None] * B[r])[:, :, None] * x[r][:, None, :]
            y[r] = torch.einsum("hnp,hn->hp", S, C[r]) + skip[:, None] * x[r]
        state[slot] = S
    zf = z.float()
    return y.reshape(m, inner) * (zf * torch.sigmoid(zf))


def shift_mix(x, mu, state, slot_ids, cu_rows, row_seq, one_row_each=False, out_dtype=None):
    """out[s, r] = x[r] + (x[r - 1] - x[r]) * mu[s] within each sequence; the row before a sequence's first row of the
    step is state[slot] (float32 [slots, D]), which then takes the sequence's last row."""
    xf = x.float()
    before = torch.empty_like(xf)
    for i in range(len(cu_rows) - 1):
        a, b, slot = int(cu_rows[i]), int(cu_rows[i + 1]), int(slot_ids[i])
        before[a] = state[slot]
        before[a + 1:b] = xf[a:b - 1]
        state[slot] = xf[b - 1]
    return (xf[None] + (before - xf)[None] * mu[:, None, :]).to(out_dtype or x.dtype)


def unary_(x, name):
    """In place: x <- tanh(x)."""
    assert name == "tanh"
    x.copy_(torch.tanh(x.float()).to(x.dtype))
    return x


def time_mix_scan(r, k, v, log_rate, w0, bonus, state, slot_ids, cu_rows, max_count, heads, dim, chunk=None):
    """o = (S + diag(bonus) k v^T)^T r, then S <- diag(w) S + k v^T with w = exp(-exp(log_rate + w0)), row after row of
    every sequence from state[slot] [heads, dim, dim], which is left updated.  float32 [M, heads dim]."""
    m = r.shape[0]
    wide = state.dtype                                   # float64 states: the whole recurrence in float64
    rf, kf, vf = (t.to(wide).reshape(m, heads, dim) for t in (r, k, v))
    w = torch.exp(-torch.exp(log_rate.to(wide) + w0.to(wide))).reshape(m, heads, dim)
    bonus = bonus.to(wide)
    y = torch.empty((m, heads, dim), dtype=wide, device=r.device)
    for i in range(len(cu_rows) - 1):
        slot = int(slot_ids[i])
        S = state[slot].clone()
        for t in range(int(cu_rows[i]), int(cu_rows[i + 1])):
            kv = kf[t][:, :, None] * vf[t][:, None, :]
            y[t] = torch.einsum("hkv,hk->hv", S + bonus[:, :, None] * kv, rf[t])
            S = w[t][:, :, None] * S + kv
        state[slot] = S
    return y.reshape(m, heads * dim).float()


def matrix_memory_scan(q, k, v, gates, cap, q_scale, memory, normalizer, maximum, slot_ids, cu_rows, max_count, heads, dk, dv, chunk=None):
    """gates float32 [M, 2 heads]: the input and forget gates' sums.  i = cap tanh(. / cap), f = logsigmoid(cap tanh(. / cap)),
    m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k, o = S^T q' / (max(|n . q'|, e^(-m')) + 1e-6)
    with q' = q q_scale; the states [slots, heads, dk, dv], [slots, heads, dk], [slots, heads] are left updated."""
    M = q.shape[0]
    wide = memory.dtype                                  # float64 states: the whole recurrence in float64
    qf, kf, vf = q.to(wide).reshape(M, heads, dk) * q_scale, k.to(wide).reshape(M, heads, dk), v.to(wide).reshape(M, heads, dv)
    gi = cap * torch.tanh(gates[:, :heads].to(wide) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh(gates[:, heads:].to(wide) / cap))
    y = torch.empty((M, heads, dv), dtype=wide, device=q.device)
    for s in range(len(cu_rows) - 1):
        slot = int(slot_ids[s])
        S, n, mx = memory[slot].clone(), normalizer[slot].clone(), maximum[slot].clone()
        for t in range(int(cu_rows[s]), int(cu_rows[s + 1])):
            new = torch.maximum(gf[t] + mx, gi[t])
            keep, take = torch.exp(gf[t] + mx - new), torch.exp(gi[t] - new)
            S = keep[:, None, None] * S + take[:, None, None] * kf[t][:, :, None] * vf[t][:, None, :]
            n = keep[:, None] * n + take[:, None] * kf[t]
            mx = new
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
            y[t] = torch.einsum("hkv,hk->hv", S, qf[t]) / den[:, None]
        memory[slot], normalizer[slot], maximum[slot] = S, n, mx
    return y.reshape(M, heads * dv).float()


def head_norm_gate(y, gain, g, eps, heads, activation, out_dtype):
    """Every head's part of a row over its root mean square, times the gain, times act(g): sigmoid(g) or silu(g)."""
    gf = g.float()
    act = torch.sigmoid(gf) if activation == "sigmoid" else gf * torch.sigmoid(gf)
    return (_norm(y, gain, eps, heads) * act).to(out_dtype)


def weighted_sum(a, wa, b, wb):
    return wa * a.float() + wb * b.float()


def pair_norm_mean(a, b, gain_a, gain_b, eps):
    return 0.5 * (_norm(a, gain_a, eps) + _norm(b, gain_b, eps))


def mul_sigmoid(x, g):
    x.copy_((x.float() * torch.sigmoid(g.float())).to(x.dtype))
    return x


def mul_sigmoid_heads(x, g, heads):
    m = x.shape[0]
    x.copy_((x.float().reshape(m, heads, -1) * torch.sigmoid(g.float())[:, :, None]).reshape(m, -1).to(x.dtype))
    return x


def bias_act(rows, bias, activation, out_dtype, pad=0):
    y = rows.float() + (bias.float() if bias is not None else 0.0)
    if activation == "gelu_erf":
        y = 0.5 * y * (1.0 + torch.erf(y * 0.7071067811865476))
    else:
        assert activation is None
    if pad:
        tail = torch.zeros((y.shape[0], pad), dtype=y.dtype, device=y.device)
        tail[:, 0] = 1.0
        y = torch.cat([y, tail], dim=1)
    return y.to(out_dtype)


def qkv_prepare(x, bias, H, KV, row, dim, inv_freq, rotary_dim, row_pos, unit_eps, out_dtype, pairing="halves"):
    m = x.shape[0]
    y = x.float() + (bias.float() if bias is not None else 0.0)
    y = y.reshape(m, H + 2 * KV, row)
    qk = _rotate(y[:, :H + KV], row_pos, inv_freq, rotary_dim, pairing)
    if unit_eps is not None:
        qk = qk * torch.rsqrt((qk[..., :dim] ** 2).mean(-1, keepdim=True) + unit_eps)
    qk[..., dim:] = 0.0
    q = qk[:, :H].reshape(m, H * row).to(out_dtype)
    if not KV:
        return q, None, None
    return q, qk[:, H:].reshape(m, KV * row).to(out_dtype), y[:, H + KV:].reshape(m, KV * row).to(out_dtype)


def pool_write(k, v, KV, row, block, cu_rows, max_count, new_len, slot_ids, sums, table, k_blocks, v_blocks):
    page = k_blocks.shape[2]
    for i in range(len(cu_rows) - 1):
        a, b, slot = int(cu_rows[i]), int(cu_rows[i + 1]), int(slot_ids[i])
        start = int(new_len[i]) - (b - a)
        for r in range(a, b):
            p = start + r - a
            if p % block == 0:
                sums[slot].zero_()
            sums[slot, 0] += k[r].float()
            sums[slot, 1] += v[r].float()
            if p % block == block - 1:
                n = p // block
                pg = int(table[i, n // page])
                assert pg >= 0
                k_blocks[pg, :, n % page, :] = (sums[slot, 0] / block).reshape(KV, row).to(k_blocks.dtype)
                v_blocks[pg, :, n % page, :] = (sums[slot, 1] / block).reshape(KV, row).to(v_blocks.dtype)


def attention_pooled(q, k, v, H, KV, hd, cu_rows, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap, scale, softcap,
                     window, blocks=None, all_values=False, max_count=None):
    m, page = q.shape[0], k_pool.shape[2]
    VG = KV if all_values else 1
    out = torch.zeros((m, H, VG, hd), dtype=torch.float32, device=q.device)
    qf, kf, vf = q.float().reshape(m, H, hd), k.float().reshape(m, KV, hd), v.float().reshape(m, KV, hd)
    for i in range(len(cu_rows) - 1):
        a, b = int(cu_rows[i]), int(cu_rows[i + 1])
        start = int(new_len[i]) - (b - a)
        for r in range(a, b):
            p = start + r - a
            lo = max(0, p - window + 1) if window else 0
            keys, vals = [], []
            if blocks is not None:
                block, btable, kb, vb = blocks
                for n in range(max(0, p - window + 1) // block):
                    pg = int(btable[i, n // page])
                    keys.append(kb[pg, :, n % page, :].float())
                    vals.append(vb[pg, :, n % page, :].float())
            for t in range(lo, p + 1):
                if t < start:
                    rr = t % rows_cap if rows_cap else t
                    pg = int(table[i, rr // page])
                    keys.append(k_pool[pg, :, rr % page, :].float())
                    vals.append(v_pool[pg, :, rr % page, :].float())
                else:
                    keys.append(kf[a + t - start])
                    vals.append(vf[a + t - start])
            keys, vals = torch.stack(keys), torch.stack(vals)            # [n, KV, hd]
            for h in range(H):
                g = h // (H // KV)
                s_ = (keys[:, g] @ qf[r, h]) * scale
                if softcap:
                    s_ = softcap * torch.tanh(s_ / softcap)
                w = torch.softmax(s_, dim=0)
                for c in range(VG):
                    out[r, h, c] = w @ vals[:, c if all_values else g]
    return out


def talk_mix(a, talk, out_dtype):
    m, H, VG, hd = a.shape
    own = torch.arange(H) // (H // VG)
    picked = a[:, :, own, :]                              # [m, g, h, hd]: head g's weights on the values of h's kv head
    return torch.einsum("hg,mghd->mhd", talk.float(), picked).reshape(m, H * hd).to(out_dtype)


def gather_rows(x, rows):
    return x[rows.long()].contiguous()


def argmax(logits):
    """Smallest index among the largest values."""
    mx = logits.max(dim=-1, keepdim=True).values
    idx = torch.arange(logits.shape[-1], device=logits.device).expand_as(logits)
    big = torch.full_like(idx, logits.shape[-1])
    return torch.where(logits == mx, idx, big).min(dim=-1).values.to(torch.int32)


def apply_repetition_penalty(logits, recent, penalty):
    """recent int32 [B, R], -1 = empty; each distinct token once: z / penalty if z > 0 else z * penalty."""
    if penalty <= 1.0:
        return
    for b in range(logits.shape[0]):
        for t in set(int(x) for x in recent[b] if int(x) >= 0):
            z = logits[b, t]
            logits[b, t] = z / penalty if z > 0 else z * penalty


def sample(logits, temperature, top_k, top_p, uniforms):
    """Per row: the top_k largest (ties: smaller id first), p = softmax((z - max) / T) over them, the
    shortest prefix with mass >= top_p, walk with r = u * kept mass.  Returns int32 [B]."""
    out = []
    for b in range(logits.shape[0]):
        z = logits[b].double()
        k = min(top_k, z.numel()) if top_k > 0 else z.numel()
        if top_k > 0:
            order = sorted(range(z.numel()), key=lambda i: (-float(z[i]), i))[:k]
        else:
            order = list(range(z.numel()))            # the whole vocabulary, in id order, no nucleus
        zs = torch.tensor([float(z[i]) for i in order], dtype=torch.float64)
        p = torch.exp((zs - zs.max()) / temperature)
        p = p / p.sum()
        cum = torch.cumsum(p, 0)
        keep = k
        for j in range(k):
            if float(cum[j]) >= top_p:
                keep = j + 1
                break
        r = float(uniforms[b]) * float(p[:keep].sum())
        tok = order[0]
        for j in range(keep):
            if r < float(p[j]):
                tok = order[j]
                break
            r -= float(p[j])
        out.append(tok)
    return torch.tensor(out, dtype=torch.int32, device=logits.device)
