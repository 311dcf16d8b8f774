"""Two designs side by side at equal layer sizes: Golepel or Lutovik next to Gemma-2, Besulix or Vogunex next to Lutovik,
random weights, one MI355X.

    python bench.py --compare golepel|lutovik|besulix|vogunex [--sizes 2b|9b] [--layers L] [--steps K] [--warmup W]

For each design: tokens per second of a prefill of 2,048 tokens and of the generation loop's decode steps at batch 8
and 1 (HIP graphs, greedy choice on the device), and the time of the kernels a step spends its time in, one by one at
the same shapes, with their share of the HBM or matrix peak (`measure.time_kernels` for Gemma-2, `time_golepel_kernels`
here).  One JSON line.  The Golepel sizes follow the Gemma-2 size of the same name: its width, vocabulary and number
of layers; 16 heads of 128 unrotated and 64 rotated elements, values of 128, a latent of 192 (a cached row of 256
elements, against Gemma-2's 2 x 4 x 256 at 2B); every second layer reads the cache of the layer before it; the
feed-forward alternates in pairs between a dense layer of Gemma's width and 8 experts of half that width, 2 chosen,
so that a token passes through as many feed-forward weights in either.
The Lutovik sizes: Gemma-2's width, vocabulary, number of layers and attention geometry (8 heads on 4 kv heads of 256 at
2B, a rotation of 64 elements with scaled frequencies); of every four layers the first and the last are attention
layers with a dense feed-forward, the second runs an attention (keys of 128, values of 256, gated) beside a state-space
mixer (heads of 64 channels filling the width, a state of 128 rows, 4 groups, 4 taps), and the third is an attention
layer on the first one's cache; the second and third have 8 experts of half the dense width, 2 chosen, and a shared
expert of a quarter of it (`time_lutovik_kernels`).
The Besulix sizes: the same width, vocabulary and number of layers; layers alternate between a parallel layer with a
dense feed-forward of Gemma's width (left: 16 heads on 4 kv heads of 128, values of 128, a rotation of 64 elements,
chunks of 1,024 positions; right: time-mixing heads of 64 channels filling the width) and a matrix-memory layer without
a feed-forward (heads of 128 key and 256 value elements filling the width) (`time_besulix_kernels`).
The Vogunex sizes: the same width, vocabulary and number of layers; of every four layers the first is an attention layer
(Gemma-2's heads; a window of 1,024 positions, pooled blocks of 16, a score cap, talking heads) with a biased dense
feed-forward of Gemma's width, the second an attention through a latent (16 heads of 128 + 64, values of 128, a latent
of 192, a query latent of 768, a window of 1,024, gated heads), the third runs on the first one's weights, the fourth is
a state-space layer of Lutovik's sizes; the second and fourth have 8 experts of half the dense width, 2 chosen, and a
gated shared expert of a quarter of it (`time_vogunex_kernels`).
"""
import json
import sys
import time

from .measure import CONTEXT, OTHER_SIZES, PEAK_FLOPS, PEAK_HBM_GBS, PREFILL_TOKENS, SIZES, time_kernels


def golepel_config(which, layers=0):
    from .config import GolepelConfig
    g = dict(SIZES, **OTHER_SIZES[which])
    n = layers or g["num_hidden_layers"]
    D, I = g["hidden_size"], g["intermediate_size"]
    out = []
    for i in range(n):
        mixer = {"heads": 16, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 192, "scale": 192 ** -0.5,
                 "rot": {"base": 10000.0, "dims": 64}}
        if i % 2:
            mixer["kv_from"] = i - 1
        if i % 4 < 2:
            mlp = {"kind": "dense", "ff": I}
        else:
            mlp = {"kind": "moe", "expert": {"ff": I // 2, "limit": 7.0}, "router": {"experts": 8, "top": 2}}
        out.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    return GolepelConfig.from_dict({"architecture": "Golepel", "vocab": g["vocab_size"], "width": D, "logit_scale": 1.0,
                                    "norm": {"eps": 1e-6, "groups": 2}, "canon": {"taps": 4}, "layers": out})


def lutovik_config(which, layers=0):
    from .config import LutovikConfig
    g = dict(SIZES, **OTHER_SIZES[which])
    n = layers or g["num_hidden_layers"]
    D, I, H, KV, hd = g["hidden_size"], g["intermediate_size"], g["num_attention_heads"], g["num_key_value_heads"], g["head_dim"]
    rot = {"base": 10000.0, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}
    att = {"heads": H, "kv_heads": KV, "dim": hd, "vdim": hd, "scale": hd ** -0.5, "rot": rot}
    left = {"heads": H, "kv_heads": KV, "dim": hd // 2, "vdim": hd, "scale": (hd // 2) ** -0.5, "rot": {"base": 100000.0, "dims": hd // 2}}
    right = {"heads": D // 64, "vdim": 64, "state": 128, "groups": 4, "conv": 4, "norm_groups": 4}
    moe = {"kind": "moe", "expert": {"ff": I // 2}, "router": {"experts": 8, "top": 2}, "shared": {"ff": I // 4}}
    out = []
    for i in range(n):
        if i % 4 == 1:
            out.append({"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": moe})
        elif i % 4 == 2:
            out.append({"type": "attention", "mixer": dict(att, kv_from=i - 2), "mlp": moe})
        else:
            out.append({"type": "attention", "mixer": att, "mlp": {"kind": "dense", "ff": I}})
    return LutovikConfig.from_dict({"architecture": "Lutovik", "vocab": g["vocab_size"], "width": D, "embedding": {"scale": D ** 0.5},
                                    "norm": {"eps": 1e-6}, "layers": out})


def besulix_config(which, layers=0):
    from .config import BesulixConfig
    g = dict(SIZES, **OTHER_SIZES[which])
    n = layers or g["num_hidden_layers"]
    D, I = g["hidden_size"], g["intermediate_size"]
    left = {"heads": 16, "kv_heads": 4, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "rot": {"base": 250000.0, "dims": 64},
            "mask": {"size": 1024}}
    par = {"type": "parallel", "mixer": {"left": left, "left_scale": 0.8, "right": {"heads": D // 64, "dim": 64}, "right_scale": 0.9},
           "mlp": {"kind": "dense", "ff": I, "limit": 7.0}}
    mem = {"type": "mlstm", "mixer": {"heads": D // 256, "dim": 128, "vdim": 256, "gate_cap": 15.0}, "mlp": None}
    return BesulixConfig.from_dict({"architecture": "Besulix", "vocab": g["vocab_size"], "width": D, "norm": {"eps": 1e-6},
                                    "logit_softcap": 30.0, "layers": [par if i % 2 == 0 else mem for i in range(n)]})


def vogunex_config(which, layers=0):
    from .config import VogunexConfig
    g = dict(SIZES, **OTHER_SIZES[which])
    n = layers or g["num_hidden_layers"]
    D, I, H, KV, hd = g["hidden_size"], g["intermediate_size"], g["num_attention_heads"], g["num_key_value_heads"], g["head_dim"]
    att = {"heads": H, "kv_heads": KV, "dim": hd, "vdim": hd, "scale": hd ** -0.5, "softcap": 50.0, "rot": {"base": 10000.0, "dims": 64},
           "mask": {"size": 1024, "pool": 16}}
    lat = {"heads": 16, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 192, "q_rank": 768, "scale": 192 ** -0.5,
           "rot": {"base": 10000.0, "dims": 64}, "mask": {"size": 1024}}
    ssm = {"heads": D // 64, "vdim": 64, "state": 128, "groups": 4, "conv": 4, "norm_groups": 4}
    moe = {"kind": "moe", "expert": {"ff": I // 2, "limit": 7.0}, "router": {"experts": 8, "top": 2}, "shared": {"ff": I // 4, "limit": 7.0}}
    dense = {"kind": "dense", "ff": I}
    out = []
    for i in range(n):
        if i % 4 == 0:
            out.append({"type": "attention", "mixer": att, "mlp": dense})
        elif i % 4 == 1:
            out.append({"type": "latent_attention", "mixer": lat, "mlp": moe})
        elif i % 4 == 2:
            out.append({"type": "attention", "mixer": att, "mlp": dense, "weights_of": i - 2})
        else:
            out.append({"type": "mamba2", "mixer": ssm, "mlp": moe})
    return VogunexConfig.from_dict({"architecture": "Vogunex", "vocab": g["vocab_size"], "width": D, "embedding": {"scale": D ** 0.5},
                                    "norm": {"eps": 1e-6}, "layers": out})


def time_vogunex_kernels(engine, cfg, batch, context, prefill_tokens):
    """Microseconds of Vogunex's kernels at a decode step of `batch` sequences over `context` cached tokens and at a
    prefill of `prefill_tokens`, each called once per layer on that layer's own weights, replayed from a HIP graph.
    Products are priced by their weights' bytes (decode) or their flops against the bf16 matrix peak (prefill); the
    attention over a window and pooled blocks by the keys and values of all kv heads that a query's window and blocks
    hold (decode) or by the flops of every query head on its own kv head's keys and values (prefill: what it computes
    beyond that for the mix of the heads is not counted as work)."""
    import torch
    from .engine.batch import StepContext
    model, ops, dev = engine.model, engine.model.rt.ops, engine.model.rt.device
    bf, f32 = torch.bfloat16, torch.float32
    blocks = [l.block for l in model.layers]
    att = [b for b in blocks if hasattr(b.mixer, "talk")]
    lat = [b for b in blocks if hasattr(b.mixer, "w_absorb")]
    dense = [b for b in blocks if hasattr(b.feed_forward, "b_up")]
    moe = [b for b in blocks if hasattr(b.feed_forward, "w_router")]
    D = cfg.hidden_size
    out = {}
    timed = _timer(dev, out)
    cache = engine.cache
    entry = lambda group: next(i for i, e in enumerate(model.schedule) if model.layers[e.layer].block is group[0])
    elems = lambda w: float(w.numel())
    for rows, tag in ((batch, f"decode_b{batch}"), (prefill_tokens, f"prefill_{prefill_tokens}")):
        decode = rows == batch
        slots = [cache.acquire() for _ in range(batch if decode else 1)]
        try:
            for s in slots:
                cache.grow(s, context if decode else rows)
            counts = [1] * batch if decode else [rows]
            starts = [context - 1] * batch if decode else [0]
            ctx = StepContext(model.rt, cache, slots, counts, starts, [])
            x = torch.randn((rows, D), device=dev).to(bf)
            one = lambda f, **kw: timed(f"{tag}.{kw.pop('name')}", f, **kw)
            prod = (lambda name, calls, w, m=rows: one(calls, name=name, bytes_each=2.0 * elems(w)) if decode
                    else one(calls, name=name, flops_each=2.0 * m * elems(w)))
            stream = torch.randn((rows, D), device=dev)
            shift_state = cache.entry_state(0, "token_shift")
            one([lambda: ops.shift_mix(stream, blocks[0].shift_weight, shift_state, ctx.slot_ids, ctx.cu_rows, ctx.row_seq, one_row_each=decode,
                                       out_dtype=bf)] * 16, name="token_shift", bytes_each=rows * D * 6.0)
            if att:
                e = entry(att)
                ctx.entry = ctx.cache_owner = e
                a = att[0].mixer
                H, KV, row, W, P = a.num_heads, a.num_kv_heads, a.row, a.window, a.pool
                site, bsite = cache.site(e), cache.entry_site(e, "mixer.blocks")
                table, btable = ctx.page_table(site.group_index), ctx.page_table(bsite.group_index)
                kp, vp, cap = site.tensor("k"), site.tensor("v"), site.rows_cap or 0
                kb, vb, sums = bsite.tensor("k"), bsite.tensor("v"), cache.entry_state(e, "mixer.block_sums")
                prod("qkv_f32", [(lambda b=b: ops.linear(x, b.mixer.w_qkv, f32)) for b in att], a.w_qkv)
                qkv = torch.randn((rows, (H + 2 * KV) * row), device=dev)
                prep = lambda: ops.qkv_prepare(qkv, a.b_qkv, H, KV, row, a.head_dim, a.inv_freq, a.position.rotary_dim, ctx.row_pos,
                                               a.unit_norm_eps, bf)
                one([prep] * 16, name="qkv_prepare", bytes_each=rows * (H + 2 * KV) * row * 6.0)
                q, k, v = prep()
                one([lambda: ops.pool_write(k, v, KV, row, P, ctx.cu_rows, ctx.max_count, ctx.new_len, ctx.slot_ids, sums, btable, kb, vb)] * 16,
                    name="pool_write", bytes_each=rows * 2 * KV * row * (2.0 + 2.0 / P))
                att_call = lambda: ops.attention_pooled(q, k, v, H, KV, row, ctx.cu_rows, ctx.row_seq, ctx.row_pos, ctx.new_len, table, kp, vp, cap,
                                                        a.query_scale, a.softcap, W, blocks=(P, btable, kb, vb), all_values=True,
                                                        max_count=ctx.max_count)
                if decode:
                    keys = min(context, W) + max(0, context - W) // P
                    one([att_call] * 8, name=f"attention_{keys}_keys_of_{context}", bytes_each=2.0 * batch * keys * 2 * KV * row)
                else:
                    pairs = sum(min(p + 1, W) + max(0, p - W + 1) // P for p in range(rows))
                    one([att_call] * 4, name=f"attention_window_{W}_blocks_of_{P}", flops_each=4.0 * pairs * H * row)
                heads = att_call()
                one([lambda: ops.talk_mix(heads, a.talk, bf)] * 16, name="talk_mix", bytes_each=rows * H * row * (4.0 * KV + 2.0))
                one([lambda: ops.kv_write(k, v, KV, row, ctx.row_seq, ctx.row_pos, ctx.new_len, table, kp, vp, cap)] * 16, name="kv_write",
                    bytes_each=rows * 2 * KV * row * 4.0)
                xa = torch.randn((rows, H * row), device=dev).to(bf)
                prod("o", [(lambda b=b: ops.linear(xa, b.mixer.w_o, bf, defer=True)) for b in att], a.w_o)
            if lat:
                e = entry(lat)
                ctx.entry = ctx.cache_owner = e
                mx = lat[0].mixer
                H, dn, dr, dv, R, lrow = mx.num_heads, mx.nope_dim, mx.rope_dim, mx.value_dim, mx.rank, mx.row
                site = cache.site(e)
                table, pool, cap = ctx.page_table(site.group_index), site.tensor("latent"), site.rows_cap or 0
                prod("latent_dq_f32", [(lambda b=b: ops.linear(x, b.mixer.w_dq, f32)) for b in lat], mx.w_dq)
                cq = torch.randn((rows, mx.query_rank), device=dev).to(bf)
                prod("latent_uq", [(lambda b=b: ops.linear(cq, b.mixer.w_uq, bf)) for b in lat], mx.w_uq)
                prod("latent_dkv", [(lambda b=b: ops.linear(x, b.mixer.w_tail, bf)) for b in lat], mx.w_tail)
                proj, tail = ops.linear(cq, mx.w_uq, bf), ops.linear(x, mx.w_tail, bf)
                prep = lambda: ops.latent_prepare(proj, H, dn, dr, R, mx.latent_gain, 1e-6, mx.inv_freq, mx.position.rotary_dim, ctx.row_seq,
                                                  ctx.row_pos, ctx.new_len, table, pool, cap, own=True, out_dtype=bf, tail=tail)
                one([prep] * 16, name="latent_prepare", bytes_each=rows * (proj.shape[1] + H * dr + 3 * lrow) * 2.0)
                q, mine = prep()
                xq = proj.view(rows, H, dr + dn)[:, :, dr:]
                qv = q.view(rows, H, lrow)[:, :, dr:]
                one([(lambda b=b: ops.head_linear(xq, b.mixer.w_absorb, qv)) for b in lat], name="latent_absorb",
                    bytes_each=2.0 * (elems(mx.w_absorb) + rows * H * (dn + R)))
                if decode:
                    keys = min(context, mx.window)
                    per = next(g for g in (mx.DECODE_GROUP_LONG if keys >= mx.LONG_KEYS else mx.DECODE_GROUP, 4, 2, 1) if H % g == 0)
                    one([lambda: ops.attention_decode(q, H, 1, lrow, ctx.new_len, table, pool, pool, cap, mx.scale, 0.0, mx.window, bf,
                                                      max_keys=ctx.max_rows_visible(site), head_groups=H // per,
                                                      splits=ops.decode_splits(batch * (H // per), 1, lrow, keys))] * 8,
                        name=f"latent_attention_{keys}_keys", bytes_each=2.0 * batch * keys * lrow)
                else:
                    pairs = sum(min(p + 1, mx.window) for p in range(rows))
                    one([lambda: ops.attention_prefill(q, mine, mine, H, 1, lrow, ctx.cu_rows, rows, mx.scale, 0.0, mx.window, bf,
                                                       row_seq=ctx.row_seq, row_pos=ctx.row_pos, wide_weights=True)] * 4,
                        name=f"latent_attention_window_{mx.window}", flops_each=4.0 * pairs * H * lrow)
                o_lat = torch.randn((rows, H * lrow), device=dev).to(bf)
                ov = o_lat.view(rows, H, lrow)[:, :, dr:]
                one([(lambda b=b: ops.head_linear(ov, b.mixer.w_up, None)) for b in lat], name="latent_up",
                    bytes_each=2.0 * (elems(mx.w_up) + rows * H * (R + dv)))
                hv = torch.randn((rows, H * dv), device=dev).to(bf)
                gates = torch.randn((rows, H), device=dev)
                one([lambda: ops.mul_sigmoid_heads(hv, gates, H)] * 16, name="gate_heads", bytes_each=rows * H * dv * 4.0)
                prod("latent_o", [(lambda b=b: ops.linear(hv, b.mixer.w_o, bf, defer=True)) for b in lat], mx.w_o)
            if dense:
                ff = dense[0].feed_forward
                prod("up_f32", [(lambda b=b: ops.linear(x, b.feed_forward.w_up, f32)) for b in dense], ff.w_up)
                up = torch.randn((rows, ff.intermediate_size), device=dev)
                one([lambda: ops.bias_act(up, ff.b_up, "gelu_erf", bf)] * 16, name="bias_gelu", bytes_each=rows * ff.intermediate_size * 6.0)
                xi = torch.randn((rows, ff.w_down.shape[1]), device=dev).to(bf)
                prod("down_with_bias", [(lambda b=b: ops.linear(xi, b.feed_forward.w_down, bf, defer=True)) for b in dense], ff.w_down)
            if moe:
                ff = moe[0].feed_forward
                logits = torch.randn((rows, ff.n_experts), device=dev)
                chosen, weights = ops.route_top(logits, ff.top, True)
                one([lambda: ops.route_top(logits, ff.top, True)] * 16, name="route_top")
                used = len(set(chosen.reshape(-1).tolist()))
                per_expert = float(ff.w_gate_up[0].numel() + ff.w_down[0].numel())
                calls = [(lambda b=b: ops.expert_ffn(x, chosen, weights, b.feed_forward.w_gate_up, b.feed_forward.w_down, ff.limit, ff.gate_alpha,
                                                     ff.up_shift)) for b in moe]
                if decode:
                    one(calls, name=f"experts_{used}_used", bytes_each=2.0 * used * per_expert)
                else:
                    one(calls, name="experts", flops_each=2.0 * rows * ff.top * per_expert)
                sh = ff.shared
                prod("shared_gate_up", [(lambda b=b: ops.gated_linear(x, b.feed_forward.shared.w_gate_up, sh.intermediate_size, "quick_gelu", bf,
                                                                      limit=sh.limit, up_shift=sh.up_shift)) for b in moe],
                     sh.w_gate_up[:2 * sh.intermediate_size])
                both = torch.randn((rows, D), device=dev)
                sg = torch.randn((rows, 1), device=dev)
                one([lambda: ops.mul_sigmoid_heads(both, sg, 1)] * 16, name="gate_shared", bytes_each=rows * D * 8.0)
            rows_b = torch.randn((rows, D), device=dev).to(bf)
            g = torch.ones(D, device=dev)
            one([lambda: ops.add_rms_norm(stream, rows_b, None, 0.0, g, 1e-6, f32)] * 16, name="add_rms_norm_f32",
                bytes_each=rows * D * (4 + 4 + 2 + 4) + 4.0 * D)
        finally:
            for s in slots:
                cache.release(s)
    return out


def gemma_config(which, layers=0):
    from .config import Gemma2Config
    g = dict(SIZES, **OTHER_SIZES[which])
    return Gemma2Config.from_kwargs(**dict(g, num_hidden_layers=layers or g["num_hidden_layers"]))


class Run:
    """One design's engine and the two things timed on it."""

    def __init__(self, cfg, rows, most_tokens, name):
        import torch
        from .engine import Engine
        from .sampling import Sampler, SamplingParams
        t0 = time.time()
        self.cfg, self.name = cfg, name
        self.engine = Engine.from_config(cfg, seed=2, sigma=0.02, dtype="bfloat16", draw_on_device=True,
                                         max_tokens_in_cache=most_tokens, max_context=CONTEXT, max_batch=rows)
        self.model, self.cache = self.engine.model, self.engine.cache
        self.sampler = Sampler(self.model.rt, SamplingParams())
        self.gen = torch.Generator().manual_seed(2)
        torch.cuda.synchronize()
        import math
        self.weight_bytes = 2 * sum(math.prod(ts.shape) for ts in self.model.tensor_layout().values())
        print(f"[compare] {name} ready in {time.time() - t0:.1f}s, {self.weight_bytes / 1e9:.2f} GB of weights", file=sys.stderr, flush=True)

    def prompts(self, lengths):
        import torch
        return [torch.randint(0, self.cfg.vocab_size, (n,), generator=self.gen).tolist() for n in lengths]

    def prefill(self, tokens=PREFILL_TOKENS):
        import torch

        def once():
            s = self.cache.acquire()
            toks = self.prompts([tokens])[0]
            torch.cuda.synchronize()
            t = time.perf_counter()
            self.model.step(self.cache, [s], toks, counts=[tokens])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            self.cache.release(s)
            return dt
        once()
        return min(once() for _ in range(3))

    def decode(self, lengths, steps, warmup):
        import torch
        from .engine.generate import BatchRun
        items = [(i, p, i) for i, p in enumerate(self.prompts(lengths))]
        run = BatchRun(self.model, self.cache, items, 1 << 30, self.sampler, 0, set(), graphs=self.engine.graphed)
        try:
            run.prefill()
            for _ in range(warmup):
                run.advance()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(steps):
                run.advance()
            torch.cuda.synchronize()
            return time.perf_counter() - t
        finally:
            run.close()

    def close(self):
        import torch
        del self.engine, self.model, self.cache, self.sampler
        torch.cuda.empty_cache()


def time_golepel_kernels(engine, cfg, batch, context, prefill_tokens):
    """Microseconds of Golepel's kernels at a decode step of `batch` sequences over `context` cached tokens and at a
    prefill of `prefill_tokens`, each called once per layer on that layer's own weights, replayed from a HIP graph.
    {name: {"us", "GB/s" | "TFLOP/s", "frac"}}."""
    import torch
    from .engine.batch import StepContext
    model, ops, dev = engine.model, engine.model.rt.ops, engine.model.rt.device
    bf = torch.bfloat16
    blocks = [l.block for l in model.layers]
    own = [b for b in blocks if b.mixer.own_latent]
    moe = [b for b in blocks if hasattr(b.feed_forward, "w_router")]
    dense = [b for b in blocks if hasattr(b.feed_forward, "w_gate_up") and not hasattr(b.feed_forward, "w_router")]
    mx = own[0].mixer
    H, dn, dr, dv, R, row, D = mx.num_heads, mx.nope_dim, mx.rope_dim, mx.value_dim, mx.rank, mx.row, cfg.hidden_size
    out = {}

    def timed(name, calls, bytes_each=None, flops_each=None):
        calls = calls * max(1, -(-24 // len(calls)))
        calls[0]()
        torch.cuda.synchronize()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for f in calls:
                    f()
        torch.cuda.current_stream(dev).wait_stream(side)
        best = float("inf")
        for _ in range(4):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b) * 1e3 / len(calls))
        r = {"us": round(best, 2)}
        if bytes_each is not None:
            r["GB/s"] = round(bytes_each / best / 1e3, 1)
            r["frac"] = round(bytes_each / best / 1e3 / PEAK_HBM_GBS, 4)
        elif flops_each is not None:
            r["TFLOP/s"] = round(flops_each / best / 1e6, 1)
            r["frac"] = round(flops_each / (best * 1e-6) / PEAK_FLOPS["bfloat16"], 4)
        out[name] = r

    cache = engine.cache
    for rows, tag in ((batch, f"decode_b{batch}"), (prefill_tokens, f"prefill_{prefill_tokens}")):
        decode = rows == batch
        slots = [cache.acquire() for _ in range(batch if decode else 1)]
        try:
            for s in slots:
                cache.grow(s, context if decode else rows)
            counts = [1] * batch if decode else [rows]
            starts = [context - 1] * batch if decode else [0]
            ctx = StepContext(model.rt, cache, slots, counts, starts, [])
            site = cache.site(0)
            table, pool = ctx.page_table(site.group_index), site.tensor("latent")
            stream = torch.randn((rows, D), device=dev)
            x = torch.randn((rows, D), device=dev).to(bf)
            taps = cfg.canon_taps
            state = cache.entry_state(0, "mixer_conv") if taps > 1 else None
            conv = blocks[0].convs["mixer_conv"]
            one = lambda f, **kw: timed(f"{tag}.{kw.pop('name')}", f, **kw)
            one([lambda: ops.causal_conv(stream, conv.w, state, ctx.slot_ids, ctx.cu_rows, ctx.row_seq, bf, one_row_each=decode, w_t=conv.w_t)] * 16,
                name="conv", bytes_each=rows * D * 6.0 + (0 if not decode else rows * (taps - 1) * D * 8.0))
            elems = lambda w: float(w.numel())
            prod = (lambda name, calls, w, m=rows: one(calls, name=name, bytes_each=2.0 * elems(w)) if decode
                    else one(calls, name=name, flops_each=2.0 * m * elems(w)))
            prod("in_proj", [(lambda b=b: ops.linear(x, b.mixer.w_in, bf)) for b in own], mx.w_in)
            proj = ops.linear(x, mx.w_in, bf)
            prep = lambda b: ops.latent_prepare(proj, H, dn, dr, R, b.mixer.latent_gain, 1e-6, b.mixer.inv_freq, b.mixer.position.rotary_dim,
                                                ctx.row_seq, ctx.row_pos, ctx.new_len, table, pool, 0, own=True, out_dtype=bf)
            one([(lambda b=b: prep(b)) for b in own], name="latent_prepare", bytes_each=rows * (proj.shape[1] + H * dr + 2 * row) * 2.0)
            q, mine = prep(own[0])
            xq = proj[:, :H * (dr + dn)].view(rows, H, dr + dn)[:, :, dr:]
            qv = q.view(rows, H, row)[:, :, dr:]
            # the per-head products move rows in and out for some 70 flop a byte, far below the ridge: priced by bytes
            one([(lambda b=b: ops.head_linear(xq, b.mixer.w_absorb, qv)) for b in blocks], name="absorb",
                bytes_each=2.0 * (elems(mx.w_absorb) + rows * H * (dn + R)))
            if decode:
                # as the mixer calls it: the heads in groups that each read the shared cached rows
                per = next(g for g in (mx.DECODE_GROUP_LONG if context >= mx.LONG_KEYS else mx.DECODE_GROUP, 4, 2, 1) if H % g == 0)
                one([lambda: ops.attention_decode(q, H, 1, row, ctx.new_len, table, pool, pool, 0, mx.scale, 0.0, 0, bf, max_keys=context,
                                                  head_groups=H // per, splits=ops.decode_splits(batch * (H // per), 1, row, context))] * 8,
                    name=f"attention_ctx{context}", bytes_each=2.0 * batch * context * row)
            else:
                pairs = rows * (rows + 1) / 2.0
                one([lambda: ops.attention_prefill(q, mine, mine, H, 1, row, ctx.cu_rows, rows, mx.scale, 0.0, 0, bf)] * 4,
                    name="attention", flops_each=4.0 * pairs * H * row)
            o_lat = torch.randn((rows, H * row), device=dev).to(bf)
            ov = o_lat.view(rows, H, row)[:, :, dr:]
            one([(lambda b=b: ops.head_linear(ov, b.mixer.w_up, None)) for b in blocks], name="up",
                bytes_each=2.0 * (elems(mx.w_up) + rows * H * (R + dv)))
            heads = torch.randn((rows, H * dv), device=dev).to(bf)
            prod("o", [(lambda b=b: ops.linear(heads, b.mixer.w_o, bf, defer=True)) for b in blocks], mx.w_o)
            if dense:
                ff = dense[0].feed_forward
                prod("gate_up", [(lambda b=b: ops.gated_linear(x, b.feed_forward.w_gate_up, ff.intermediate_size, "silu", bf)) for b in dense],
                     ff.w_gate_up[:2 * ff.intermediate_size])
                xi = torch.randn((rows, ff.intermediate_size), device=dev).to(bf)
                prod("down", [(lambda b=b: ops.linear(xi, b.feed_forward.w_down, bf, defer=True)) for b in dense], ff.w_down)
            if moe:
                ff = moe[0].feed_forward
                logits = torch.randn((rows, ff.n_experts), device=dev)
                chosen, weights = ops.route_top(logits, ff.top)
                one([lambda: ops.route_top(logits, ff.top)] * 16, name="route_top")
                used = len(set(chosen.reshape(-1).tolist()))
                per_expert = float(ff.w_gate_up[0].numel() + ff.w_down[0].numel())
                calls = [(lambda b=b: ops.expert_ffn(x, chosen, weights, b.feed_forward.w_gate_up, b.feed_forward.w_down, ff.limit,
                                                     ff.gate_alpha, ff.up_shift)) for b in moe]
                if decode:
                    one(calls, name=f"experts_{used}_used", bytes_each=2.0 * used * per_expert)
                else:
                    one(calls, name="experts", flops_each=2.0 * rows * ff.top * per_expert)
            rows_b = torch.randn((rows, D), device=dev).to(bf)
            g = torch.ones(D, device=dev)
            one([lambda: ops.add_rms_norm(stream, rows_b, g, 1e-6, None, 0.0, bf, groups=cfg.norm_groups)] * 16, name="add_group_norm",
                bytes_each=rows * D * (4 + 4 + 2) + 4.0 * D)
        finally:
            for s in slots:
                cache.release(s)
    return out


def _timer(dev, out):
    """timed(name, calls, bytes_each=, flops_each=, peak=): the calls replayed from a HIP graph, microseconds a call."""
    import torch

    def timed(name, calls, bytes_each=None, flops_each=None, peak=PEAK_FLOPS["bfloat16"]):
        calls = calls * max(1, -(-24 // len(calls)))
        calls[0]()
        torch.cuda.synchronize()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for f in calls:
                    f()
        torch.cuda.current_stream(dev).wait_stream(side)
        best = float("inf")
        for _ in range(4):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            b.synchronize()
            best = min(best, a.elapsed_time(b) * 1e3 / len(calls))
        r = {"us": round(best, 2)}
        if bytes_each is not None:
            r["GB/s"] = round(bytes_each / best / 1e3, 1)
            r["frac"] = round(bytes_each / best / 1e3 / PEAK_HBM_GBS, 4)
        elif flops_each is not None:
            r["TFLOP/s"] = round(flops_each / best / 1e6, 1)
            r["frac"] = round(flops_each / (best * 1e-6) / peak, 4)
        out[name] = r
    return timed


def time_lutovik_kernels(engine, cfg, batch, context, prefill_tokens):
    """Microseconds of Lutovik's kernels at a decode step of `batch` sequences over `context` cached tokens and at a
    prefill of `prefill_tokens`, each called once per layer on that layer's own weights, replayed from a HIP graph.
    Products are priced by their weights' bytes (decode) or their flops against the bf16 matrix peak (prefill), the scan
    by its state's bytes (decode) or its multiply-adds against the float32 vector peak (prefill)."""
    import torch
    from .engine.batch import StepContext
    model, ops, dev = engine.model, engine.model.rt.ops, engine.model.rt.device
    bf = torch.bfloat16
    blocks = [l.block for l in model.layers]
    par = [b for b in blocks if hasattr(b.mixer, "sides")]
    own = [b for b in blocks if not hasattr(b.mixer, "sides") and b.mixer.own_kv]
    moe = [b for b in blocks if hasattr(b.feed_forward, "w_router")]
    dense = [b for b in blocks if b.feed_forward is not None and not hasattr(b.feed_forward, "w_router")]
    D = cfg.hidden_size
    out = {}
    timed = _timer(dev, out)
    cache = engine.cache
    par_entry = next(i for i, l in enumerate(model.layers) if hasattr(l.block.mixer, "sides"))
    elems = lambda w: float(w.numel())
    for rows, tag in ((batch, f"decode_b{batch}"), (prefill_tokens, f"prefill_{prefill_tokens}")):
        decode = rows == batch
        slots = [cache.acquire() for _ in range(batch if decode else 1)]
        try:
            for s in slots:
                cache.grow(s, context if decode else rows)
            counts = [1] * batch if decode else [rows]
            starts = [context - 1] * batch if decode else [0]
            ctx = StepContext(model.rt, cache, slots, counts, starts, [])
            ctx.entry = ctx.cache_owner = par_entry
            x = torch.randn((rows, D), device=dev).to(bf)
            one = lambda f, **kw: timed(f"{tag}.{kw.pop('name')}", f, **kw)
            prod = (lambda name, calls, w, m=rows: one(calls, name=name, bytes_each=2.0 * elems(w)) if decode
                    else one(calls, name=name, flops_each=2.0 * m * elems(w)))
            # ---- attention layers: the products; the attention itself runs on the kernels Gemma-2's does
            a = own[0].mixer
            H, KV, row = a.num_heads, a.num_kv_heads, a.row
            prod("qkv", [(lambda b=b: ops.linear(x, b.mixer.w_qkv, bf, defer=decode)) for b in own], a.w_qkv)
            xa = torch.randn((rows, H * row), device=dev).to(bf)
            prod("o", [(lambda b=b: ops.linear(xa, b.mixer.w_o, bf, defer=True)) for b in own], a.w_o)
            site = cache.site(next(i for i, l in enumerate(model.layers) if l.block is own[0]))
            table = ctx.page_table(site.group_index)
            if decode:
                qkv = torch.randn((rows, (H + 2 * KV) * row), device=dev).to(bf)
                one([lambda: ops.attention_decode_step(qkv, H, KV, row, a.inv_freq, a.position.rotary_dim, ctx.new_len, table,
                                                       site.tensor("k"), site.tensor("v"), 0, a.query_scale, 0.0, 0, bf, max_keys=context)] * 8,
                    name=f"attention_ctx{context}", bytes_each=2.0 * batch * context * 2 * KV * row)
            else:
                q, k, v = (torch.randn((rows, n * row), device=dev).to(bf) for n in (H, KV, KV))
                one([lambda: ops.attention_prefill(q, k, v, H, KV, row, ctx.cu_rows, rows, a.query_scale, 0.0, 0, bf,
                                                   wide_weights=a.precise_weights)] * 4,
                    name="attention", flops_each=4.0 * (rows * (rows + 1) / 2.0) * H * row)
            # ---- the parallel layers: the gated attention's extras, the state-space mixer, the average of the two
            if par:
                left, right = par[0].mixer.sides
                prod("left_gate_proj", [(lambda b=b: ops.linear(x, b.mixer.sides[0].w_g, bf)) for b in par], left.w_g)
                heads_out = torch.randn((rows, left.num_heads * left.row), device=dev).to(bf)
                gates = torch.randn((rows, left.num_heads * left.row), device=dev).to(bf)
                one([lambda: ops.mul_sigmoid(heads_out, gates)] * 16, name="mul_sigmoid", bytes_each=rows * left.num_heads * left.row * 6.0)
                prod("ssm_in_proj", [(lambda b=b: ops.linear(x, b.mixer.sides[1].w_in, bf)) for b in par], right.w_in)
                inner, ch, nh, N, P = right.inner, right.conv_channels, right.num_heads, right.state_size, right.head_dim
                u = (torch.randn((rows, right.w_in.shape[0]), device=dev) * 0.5).to(bf)     # the in-projection's rows, as the mixer gets them
                conv_state = cache.entry_state(par_entry, "mixer.right.conv") if right.taps > 1 else None
                ssm_state = cache.entry_state(par_entry, "mixer.right.ssm")
                conv = lambda: ops.conv_act(u[:, inner:inner + ch], right.conv_t, right.conv_b, conv_state, ctx.slot_ids, ctx.cu_rows, ctx.row_seq,
                                            activation="silu", one_row_each=decode)
                one([conv] * 16, name="conv_act", bytes_each=rows * ch * 4.0 + (rows * (right.taps - 1) * ch * 8.0 if decode else 0.0))
                xbc = conv()
                scan = lambda: ops.ssd_scan(xbc, u[:, :inner], u[:, inner + ch:inner + ch + nh], right.dt_bias, right.a_log, right.skip, ssm_state, ctx.slot_ids,
                                            ctx.cu_rows, rows if not decode else 1, nh, right.groups, N, P)
                if decode:
                    one([scan] * 8, name="ssd_scan", bytes_each=batch * nh * N * P * 8.0)
                else:                                    # every row: the state's update and its product with C, 4 N P flop a head
                    one([scan] * 4, name="ssd_scan", flops_each=4.0 * rows * nh * N * P, peak=PEAK_FLOPS["float32"])
                y = torch.randn((rows, inner), device=dev)
                one([lambda: ops.rms_norm(y, right.norm_gain, 1e-6, bf, groups=right.norm_groups)] * 16, name="ssm_group_norm",
                    bytes_each=rows * inner * 6.0)
                yn = torch.randn((rows, inner), device=dev).to(bf)
                prod("ssm_o", [(lambda b=b: ops.linear(yn, b.mixer.sides[1].w_o, bf, defer=True)) for b in par], right.w_o)
                oa, ob = torch.randn((rows, D), device=dev).to(bf), torch.randn((rows, D), device=dev).to(bf)
                gains = par[0].mixer.gains
                one([lambda: ops.pair_norm_mean(oa, ob, gains[0], gains[1], 1e-6)] * 16, name="pair_norm_mean", bytes_each=rows * D * 8.0)
            # ---- feed-forward
            if dense:
                ff = dense[0].feed_forward
                prod("gate_up_relu", [(lambda b=b: ops.gated_linear(x, b.feed_forward.w_gate_up, ff.intermediate_size, "relu", bf)) for b in dense],
                     ff.w_gate_up[:2 * ff.intermediate_size])
                xi = torch.randn((rows, ff.intermediate_size), device=dev).to(bf)
                prod("down", [(lambda b=b: ops.linear(xi, b.feed_forward.w_down, bf, defer=True)) for b in dense], ff.w_down)
            if moe:
                ff = moe[0].feed_forward
                logits = torch.randn((rows, ff.n_experts), device=dev)
                chosen, weights = ops.route_top(logits, ff.top, score="sigmoid")
                one([lambda: ops.route_top(logits, ff.top, score="sigmoid")] * 16, name="route_top")
                used = len(set(chosen.reshape(-1).tolist()))
                per_expert = float(ff.w_gate_up[0].numel() + ff.w_down[0].numel())
                calls = [(lambda b=b: ops.expert_ffn(x, chosen, weights, b.feed_forward.w_gate_up, b.feed_forward.w_down, None, 1.0, 0.0,
                                                     weight_input=True)) for b in moe]
                if decode:
                    one(calls, name=f"experts_{used}_used", bytes_each=2.0 * used * per_expert)
                else:
                    one(calls, name="experts", flops_each=2.0 * rows * ff.top * per_expert)
                sh = ff.shared
                if sh is not None:
                    prod("shared_gate_up", [(lambda b=b: ops.gated_linear(x, b.feed_forward.shared.w_gate_up, sh.intermediate_size, "silu", bf)) for b in moe],
                         sh.w_gate_up[:2 * sh.intermediate_size])
            stream = torch.randn((rows, D), device=dev)
            rows_b = torch.randn((rows, D), device=dev).to(bf)
            g = torch.ones(D, device=dev)
            one([lambda: ops.add_rms_norm(stream, rows_b, g, 1e-6, g, 1e-6, bf)] * 16, name="add_rms_norm",
                bytes_each=rows * D * (4 + 4 + 2 + 2) + 8.0 * D)
        finally:
            for s in slots:
                cache.release(s)
    return out


def time_besulix_kernels(engine, cfg, batch, context, prefill_tokens):
    """Microseconds of Besulix's kernels at a decode step of `batch` sequences over `context` cached tokens and at a
    prefill of `prefill_tokens`, each called once per layer on that layer's own weights, replayed from a HIP graph.
    Products are priced by their weights' bytes (decode) or their flops against the bf16 matrix peak (prefill), the two
    scans by their states' bytes (decode) or their multiply-adds against the float32 vector peak (prefill), the attention
    by the cached rows it reads (decode) or its flops (prefill)."""
    import torch
    from .engine.batch import StepContext
    model, ops, dev = engine.model, engine.model.rt.ops, engine.model.rt.device
    bf, f32 = torch.bfloat16, torch.float32
    blocks = [l.block for l in model.layers]
    par = [b for b in blocks if hasattr(b.mixer, "sides")]
    mem = [b for b in blocks if hasattr(b.mixer, "w_gates")]
    dense = [b for b in blocks if b.feed_forward is not None]
    D = cfg.hidden_size
    out = {}
    timed = _timer(dev, out)
    cache = engine.cache
    entry = lambda group: next(i for i, l in enumerate(model.layers) if l.block is group[0])
    elems = lambda w: float(w.numel())
    for rows, tag in ((batch, f"decode_b{batch}"), (prefill_tokens, f"prefill_{prefill_tokens}")):
        decode = rows == batch
        slots = [cache.acquire() for _ in range(batch if decode else 1)]
        try:
            for s in slots:
                cache.grow(s, context if decode else rows)
            counts = [1] * batch if decode else [rows]
            starts = [context - 1] * batch if decode else [0]
            ctx = StepContext(model.rt, cache, slots, counts, starts, [])
            x = torch.randn((rows, D), device=dev).to(bf)
            one = lambda f, **kw: timed(f"{tag}.{kw.pop('name')}", f, **kw)
            prod = (lambda name, calls, w, m=rows: one(calls, name=name, bytes_each=2.0 * elems(w)) if decode
                    else one(calls, name=name, flops_each=2.0 * m * elems(w)))
            if par:
                e = entry(par)
                ctx.entry = ctx.cache_owner = e
                left, right = par[0].mixer.sides
                H, KV, row = left.num_heads, left.num_kv_heads, left.row
                site = cache.site(e)
                table = ctx.page_table(site.group_index)
                kp, vp, cap = site.tensor("k"), site.tensor("v"), site.rows_cap or 0
                prod("left_qkv_bias", [(lambda b=b: ops.linear(x, b.mixer.sides[0].w_qkv, bf, bias=b.mixer.sides[0].b_qkv)) for b in par], left.w_qkv)
                qkv = torch.randn((rows, (H + 2 * KV) * row), device=dev).to(bf)
                q, k, v = qkv[:, :H * row], qkv[:, H * row:(H + KV) * row], qkv[:, (H + KV) * row:]
                one([lambda: left._turn(ctx, v, KV, left.value_freq)] * 16, name="turn_values", bytes_each=rows * KV * row * 4.0)
                one([lambda: ops.rope_kv_write(q, k, v, H, KV, row, left.inv_freq, left.position.rotary_dim, ctx.row_seq, ctx.row_pos,
                                               ctx.new_len, table, kp, vp, cap)] * 16, name="rope_kv_write", bytes_each=rows * (H + 3 * KV) * row * 4.0)
                more = dict(chunk=left.chunk, head_scale=left.temperature, sink=left.sink)
                seen = min(context, (context - 1) % left.chunk + 1) if left.chunk else context
                if decode:
                    one([lambda: ops.attention_decode(q, H, KV, row, ctx.new_len, table, kp, vp, cap, left.query_scale, 0.0, 0, bf,
                                                  max_keys=ctx.max_rows_visible(site), **more)] * 8, name=f"attention_{seen}_of_{context}_keys",
                        bytes_each=2.0 * batch * seen * 2 * KV * row)
                else:
                    C = left.chunk or rows
                    full, rest = divmod(rows, C)
                    pairs = full * C * (C + 1) / 2.0 + rest * (rest + 1) / 2.0
                    one([lambda: ops.attention_prefill(q, k, v, H, KV, row, ctx.cu_rows, rows, left.query_scale, 0.0, 0, bf, row_seq=ctx.row_seq,
                                                   row_pos=ctx.row_pos, wide_weights=left.precise_weights, **more)] * 4, name=f"attention_chunks_of_{C}", flops_each=4.0 * pairs * H * row)
                heads_out = torch.randn((rows, H * row), device=dev).to(bf)
                one([lambda: left._turn(ctx, heads_out, H, left.value_back)] * 16, name="turn_back", bytes_each=rows * H * row * 4.0)
                prod("left_o", [(lambda b=b: ops.linear(heads_out, b.mixer.sides[0].w_o, f32)) for b in par], left.w_o)
                # ---- the time-mixing side
                nh, d, inner = right.num_heads, right.head_dim, right.inner
                shift, memory = cache.entry_state(e, "mixer.right.shift"), cache.entry_state(e, "mixer.right.memory")
                one([lambda: ops.shift_mix(x, right.mu, shift, ctx.slot_ids, ctx.cu_rows, ctx.row_seq, one_row_each=decode)] * 16,
                    name="shift_mix", bytes_each=rows * D * 12.0)
                for s in ("r", "g"):
                    prod(f"right_{s}", [(lambda b=b, s=s: ops.linear(x, b.mixer.sides[1].w[s], bf)) for b in par], right.w[s])

                def decay_rates(b):
                    low = ops.unary_(ops.linear(x, b.mixer.sides[1].w["w1"], bf), "tanh")
                    return ops.linear(low, b.mixer.sides[1].w["w2"], f32)
                one([(lambda b=b: decay_rates(b)) for b in par], name="decay_w1_tanh_w2",
                    bytes_each=2.0 * (elems(right.w["w1"]) + elems(right.w["w2"])) + rows * (D * 2.0 + inner * 4.0))
                r_, k_, v_ = ((torch.randn((rows, inner), device=dev) * 0.3).to(bf) for _ in range(3))
                rate = torch.randn((rows, inner), device=dev)
                scan = lambda: ops.time_mix_scan(r_, k_, v_, rate, right.w0, right.bonus, memory, ctx.slot_ids, ctx.cu_rows,
                                                 1 if decode else rows, nh, d)
                if decode:
                    one([scan] * 8, name="time_mix_scan", bytes_each=batch * nh * d * d * 8.0)
                else:                                    # every row: the state's update and its product with r, 4 d d flop a head
                    one([scan] * 4, name="time_mix_scan", flops_each=4.0 * rows * nh * d * d, peak=PEAK_FLOPS["float32"])
                y = torch.randn((rows, inner), device=dev)
                one([lambda: ops.head_norm_gate(y, right.norm_gain, r_, 1e-6, nh, "silu", bf)] * 16, name="head_norm_gate",
                    bytes_each=rows * inner * 8.0)
                yn = torch.randn((rows, inner), device=dev).to(bf)
                prod("right_o", [(lambda b=b: ops.linear(yn, b.mixer.sides[1].w["o"], f32)) for b in par], right.w["o"])
                oa, ob = torch.randn((rows, D), device=dev), torch.randn((rows, D), device=dev)
                one([lambda: ops.weighted_sum(oa, 0.8, ob, 0.9)] * 16, name="weighted_sum", bytes_each=rows * D * 12.0)
            if mem:
                e = entry(mem)
                ctx.entry = ctx.cache_owner = e
                mm = mem[0].mixer
                nh, dk, dv = mm.num_heads, mm.key_dim, mm.value_dim
                prod("memory_in", [(lambda b=b: ops.linear(x, b.mixer.w_in, bf)) for b in mem], mm.w_in)
                one([(lambda b=b: ops.linear(x, b.mixer.w_gates, f32, bias=b.mixer.b_gates)) for b in mem], name="memory_gates",
                    bytes_each=2.0 * elems(mm.w_gates) + rows * D * 2.0)
                u = (torch.randn((rows, mm.w_in.shape[0]), device=dev) * 0.3).to(bf)
                gates = torch.randn((rows, 2 * nh), device=dev)
                S, nrm, mx = (cache.entry_state(e, "mixer." + s) for s in ("memory", "normalizer", "maximum"))
                qk, vv = nh * dk, nh * dv
                scan = lambda: ops.matrix_memory_scan(u[:, :qk], u[:, qk:2 * qk], u[:, 2 * qk:2 * qk + vv], gates, mm.gate_cap, dk ** -0.5,
                                                      S, nrm, mx, ctx.slot_ids, ctx.cu_rows, 1 if decode else rows, nh, dk, dv)
                if decode:
                    one([scan] * 8, name="matrix_memory_scan", bytes_each=batch * nh * dk * dv * 8.0)
                else:
                    one([scan] * 4, name="matrix_memory_scan", flops_each=4.0 * rows * nh * dk * dv, peak=PEAK_FLOPS["float32"])
                y = torch.randn((rows, vv), device=dev)
                one([lambda: ops.head_norm_gate(y, mm.norm_gain, u[:, 2 * qk + vv:2 * qk + 2 * vv], 1e-6, nh, "sigmoid", bf)] * 16,
                    name="memory_head_norm_gate", bytes_each=rows * vv * 8.0)
                yn = torch.randn((rows, vv), device=dev).to(bf)
                prod("memory_o", [(lambda b=b: ops.linear(yn, b.mixer.w_o, bf, defer=True)) for b in mem], mm.w_o)
            if dense:
                ff = dense[0].feed_forward
                prod("gate_up_clamped", [(lambda b=b: ops.gated_linear(x, b.feed_forward.w_gate_up, ff.intermediate_size, "quick_gelu", bf,
                                                                       limit=ff.limit, up_shift=ff.up_shift)) for b in dense],
                     ff.w_gate_up[:2 * ff.intermediate_size])
                xi = torch.randn((rows, ff.intermediate_size), device=dev).to(bf)
                prod("down", [(lambda b=b: ops.linear(xi, b.feed_forward.w_down, bf, defer=True)) for b in dense], ff.w_down)
            stream = torch.randn((rows, D), device=dev)
            rows_b = torch.randn((rows, D), device=dev).to(bf)
            g = torch.ones(D, device=dev)
            one([lambda: ops.add_rms_norm(stream, rows_b, None, 0.0, g, 1e-6, bf)] * 16, name="add_rms_norm",
                bytes_each=rows * D * (4 + 4 + 2 + 2) + 4.0 * D)
        finally:
            for s in slots:
                cache.release(s)
    return out


def main(args):
    import torch
    which = args.sizes
    steps, warmup = args.steps, max(2, args.warmup)
    prompt, batch = args.prompt, args.batch
    design = args.compare
    build, time_design = {"golepel": (golepel_config, time_golepel_kernels), "lutovik": (lutovik_config, time_lutovik_kernels),
                          "besulix": (besulix_config, time_besulix_kernels), "vogunex": (vogunex_config, time_vogunex_kernels)}[design]
    # the design it stands next to: the closest of the others
    beside_lutovik = ("lutovik", lutovik_config, time_lutovik_kernels, "Lutovik")
    other, build_other, time_other, title = {"besulix": beside_lutovik, "vogunex": beside_lutovik}.get(
        design, ("gemma2", gemma_config, time_kernels, "Gemma-2"))
    line = {"metric": f"{design.capitalize()} next to {title} at {which} layer sizes: prefill and decode tok/s", "unit": "tok/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "dtype": "bf16", "data": "synthetic: seeded random weights N(0, 0.02) and uniform-random token ids",
            "sizes": which, "designs": {}, "kernels": {}}
    most = max(PREFILL_TOKENS, batch * (prompt + steps + warmup + 128)) + 1024
    for name, cfg in ((design, build(which, args.layers)), (other, build_other(which, args.layers))):
        run = Run(cfg, max(batch, 8), most, name)
        pre = run.prefill()
        d = {"layers": len(cfg.layers) if hasattr(cfg, "layers") else cfg.num_hidden_layers, "weights_GB": round(run.weight_bytes / 1e9, 2),
             f"prefill_{PREFILL_TOKENS}_tok_s": round(PREFILL_TOKENS / pre, 1), f"prefill_{PREFILL_TOKENS}_ms": round(pre * 1e3, 2)}
        for b in (batch, 1):
            dt = run.decode([prompt] * b, steps, warmup)
            d[f"decode_b{b}_tok_s"] = round(b * steps / dt, 1)
            d[f"decode_b{b}_ms_per_step"] = round(dt / steps * 1e3, 4)
        print(f"[compare] {name}: {d}", file=sys.stderr, flush=True)
        if name == design:
            k = time_design(run.engine, cfg, batch, prompt + 40, PREFILL_TOKENS)
        else:
            k = time_other(run.engine, cfg, batch, prompt + 40, PREFILL_TOKENS)
        for kn, row in k.items():
            print(f"[compare] {name} kernel {kn}: {row}", file=sys.stderr, flush=True)
        line["designs"][name] = d
        line["kernels"][name] = k
        run.close()
    g, m = line["designs"][design], line["designs"][other]
    line["value"] = g[f"decode_b{batch}_tok_s"]
    line[f"ratio_to_{other}"] = {k: round(g[k] / m[k], 3) for k in g if k.endswith("tok_s")}
    print(json.dumps(line), flush=True)
    return 0
