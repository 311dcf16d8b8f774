"""Grouped-query attention over the cache, with optional score cap and window.

In the reference's order (runtime/src/lib.rs:4483-4496): q, k, v projections,
RoPE on q and k, append k (rotated) and v to the cache, attention, output
projection.  Scores: (q . k) * query_scale, then cap * tanh(s / cap) when a cap is
set, softmax in fp32 over the visible keys, weighted sum of v; query head h reads
kv head h // (heads / kv_heads) (runtime/cuda/codebook_gemv.cu:240-270).  The
reference fixes the scale to rsqrt(head_dim) (cu:249) and has no window
(lib.rs:4455); both are parameters here: the query at position p sees keys
t <= p, and with a window W only those with p - t < W.

The three projections are one product over the concatenated weight.  A run that
reads another run's cache projects and rotates its queries only (a layer may also have no key and value
projections at all, `own_kv=False`).  Values may have another size than keys (`value_dim`), the heads' outputs
may pass a sigmoid gate computed from the layer's input (`output_gate`), and a position scheme that turns
neighbouring elements is carried out as the rotation of halves on reordered projection rows.  In a decode step
rotation, cache write and attention are one kernel launch where the kernel library
has one for the geometry (`ops.fuses_decode_step`); the order of the arithmetic is
the same.  A step that continues sequences by several tokens, or mixes starting and running sequences, attends
over the cached positions its queries still see, read in place through the page table, plus its own rows (the
reference's multi-token step walks its cache from any position: runtime/src/lib.rs:676-720,
runtime/cuda/codebook_gemv.cu:410-440), and caches its own rows after the attention.

Further parameters, none of which the reference has: biases on the q, k and v projections; `chunk` C, with which the
query at position p sees only the keys t <= p of its own chunk, floor(t / C) = floor(p / C), chunks counted from the
sequence's first position (the cache then keeps a ring of C positions); a temperature per head that multiplies its
scores; a sink per head, a learned score without key or value whose exponential joins the softmax's denominator once;
and `value_rotation` theta: the value of position t is turned by t over all its elements like a key (pairs (d, d +
value_dim / 2), frequencies theta^(-2d / value_dim)) before it is cached, and a head's output at position p is turned
back by -p, so that the weighted sum is read in the query's frame.  Chunks, temperatures and sinks are arguments of
every attention kernel (a chunk is a window whose start does not move with the query; the sink is added to the sum
when a query's keys are done, in the kernel that normalises); the values' two rotations are launches of the rotation
kernel.  A decode step of such a layer is not the one fused launch: its projections carry biases and its values turn.

A third family of parameters makes the layer an attention over a window plus pooled blocks whose heads talk:
`unit_norm_eps` (every query and key head is divided by its root mean square after the rotation: a norm without a
gain), `pool` P (beside the `window` W positions back a query at p sees one key and value for every block of P
positions b P .. b P + P - 1 with b P + P - 1 <= p - W, the mean of the block's cached keys and of its values; the
positions between the last such block and the window are not seen at all) and `talk` (a matrix [heads, heads] that
mixes the heads' softmax weights, w_h <- sum_g T[h, g] w_g, before head h applies them to the values of its own kv
head).  Any of the three takes the layer to `ops.qkv_prepare` (bias, rotation and unit norm in float32 from the
product's float32 sums, one rounding), `ops.pool_write` (the block means go to a paged pool of their own that keeps
one row per P tokens; an unfinished block's sums wait in a float32 state), `ops.attention_pooled` and
`ops.talk_mix`.  The cache's ring keeps the window only; the step's rows are cached after the attention in every
kind of step, so one sequence of launches serves prompts, portions of prompts and decode steps.
"""
from ..cache.store import TokenSpec
from ..models.spec import TensorSpec
from ..registry import build_part, register_part
from .base import Mixer


class Attention(Mixer):
    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, query_scale,
                 softcap=None, window=None, position=("none", {}), value_dim=None, output_gate=False, own_kv=True,
                 precise_weights=False,
                 tensors=("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight", "g_proj.weight"),
                 bias_suffix=None, chunk=None, head_temperature=None, sink=None, value_rotation=None,
                 unit_norm_eps=None, pool=None, talk=None):
        """value_dim: elements of a value head when they differ from a key's head_dim.  output_gate: the heads' outputs
        are multiplied by sigmoid(W_g x) before the output projection.  own_kv False: the layer has no key and value
        projections; its schedule entry names the run whose cache it reads.  precise_weights: the softmax weights meet
        the values with 16 bits of mantissa or more in every kernel (the kernel of many queries rounds them to bfloat16
        otherwise; a decode step's are float32 anyway).  tensors: local names of W_q, W_k, W_v, W_o (and W_g).
        bias_suffix: q, k and v have biases, named like their matrices with this suffix.  chunk: positions per chunk.
        head_temperature, sink: local names of float vectors [heads].  value_rotation: the base theta of the values'
        rotation by their position.  unit_norm_eps: the eps of the norm without gain on every query and key head (None:
        no such norm).  pool: positions per pooled block before the window.  talk: local name of the matrix
        [heads, heads] that mixes the heads' softmax weights."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} kv heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.value_dim = int(value_dim) if value_dim else head_dim
        # The kernels know one head size: keys and values are kept in rows of the larger of the two, the shorter kind
        # filled up with zeros through zero rows of its projection (zeros add nothing to a score, and a value's zero
        # columns meet zero columns of W_o).
        self.row = max(self.head_dim, self.value_dim)
        self.query_scale = float(query_scale)
        self.softcap = float(softcap) if softcap else 0.0
        self.window = int(window) if window else 0
        self.output_gate = bool(output_gate)
        self.own_kv = bool(own_kv)
        self.precise_weights = bool(precise_weights)
        self.names = dict(zip(("q", "k", "v", "o", "g"), tuple(tensors) + ("g_proj.weight",) * (5 - len(tensors))))
        self.position = build_part("position", position)
        if self.position.rotary_dim > head_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head_dim {head_dim}")
        self.bias_suffix = bias_suffix
        self.chunk = int(chunk) if chunk else 0
        self.temperature_name, self.sink_name = head_temperature, sink
        self.value_position = None
        if value_rotation is not None:
            self.value_position = build_part("position", ("rope", {"rotary_dim": self.value_dim, "theta": value_rotation}))
        self.output_dtype = None         # a mixer that holds this one may ask for its last product in another dtype
        self.per_head = bool(self.chunk or head_temperature or sink)
        if (self.per_head or value_rotation is not None) and (self.output_gate or not self.own_kv):
            raise ValueError("chunks, temperatures, sinks and rotated values go with an ungated attention on its own cache")
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.pool = int(pool) if pool else 0
        self.talk_name = talk
        self.pooled = self.unit_norm_eps is not None or bool(self.pool) or talk is not None
        if self.pooled and (self.per_head or value_rotation is not None or not self.own_kv):
            raise ValueError("unit norms, pooled blocks and talking heads go with an attention on its own cache, without chunks, "
                             "temperatures, sinks or rotated values")
        if self.pool and not self.window:
            raise ValueError("pooled blocks stand before a window: the layer needs one")

    @property
    def reach(self):
        """Positions back (the query's own included) that a query can see: the window, the chunk, or 0 for all."""
        return min((n for n in (self.window, self.chunk) if n), default=0)

    def tensor_specs(self):
        n, d = self.names, self.hidden_size
        q, kv = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        specs = {n["q"]: TensorSpec((q, d)), n["o"]: TensorSpec((d, self.num_heads * self.value_dim))}
        if self.own_kv:
            specs[n["k"]] = TensorSpec((kv, d))
            specs[n["v"]] = TensorSpec((self.num_kv_heads * self.value_dim, d))
        if self.output_gate:
            specs[n["g"]] = TensorSpec((self.num_heads * self.value_dim, d))
        if self.bias_suffix:
            for s in ("q", "k", "v") if self.own_kv else ("q",):
                specs[n[s] + self.bias_suffix] = TensorSpec((specs[n[s]].shape[0],), init="norm")
        if self.temperature_name:
            specs[self.temperature_name] = TensorSpec((self.num_heads,), init="gain")
        if self.sink_name:
            specs[self.sink_name] = TensorSpec((self.num_heads,), init="norm")
        if self.talk_name:
            specs[self.talk_name] = TensorSpec((self.num_heads, self.num_heads), init="talk")
        return specs

    def cache_spec(self):
        per_token = (self.num_kv_heads, self.row)
        return TokenSpec.of(self.reach or None, k=per_token, v=per_token)

    def token_specs(self):
        """The pooled blocks: one mean key and value per `pool` tokens, of all tokens."""
        if not self.pool:
            return {}
        per_block = (self.num_kv_heads, self.row)
        return {"blocks": TokenSpec.of(None, every=self.pool, k=per_block, v=per_block)}

    def state_specs(self):
        """The sums of the keys and of the values of the block that is not finished yet."""
        if not self.pool:
            return {}
        from ..cache.store import StateSpec
        return {"block_sums": StateSpec((2, self.num_kv_heads * self.row), "float32")}

    def _heads(self, w, heads, size, turned=False):
        """[heads * size, d] -> [heads * row, d]: zero rows fill a head up to `row`.  turned: a rotation of neighbouring
        pairs (2f, 2f + 1) becomes the rotation of halves (f, f + rotary_dim / 2) that every kernel knows by taking
        a head's even rotated rows first, then its odd ones; queries and keys are reordered alike, so every score is
        the same sum in another order."""
        import torch
        w = w.reshape(heads, size, -1)
        rot = self.position.rotary_dim
        if turned and rot and self.position.pairing == "neighbours":
            order = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, size))
            w = w[:, order]
        if size < self.row:
            w = torch.cat([w, w.new_zeros((heads, self.row - size, w.shape[2]))], dim=1)
        return w.reshape(heads * self.row, -1)

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        n, H, KV = self.names, self.num_heads, self.num_kv_heads
        parts = [self._heads(tensors[n["q"]], H, self.head_dim, turned=True)]
        if self.own_kv:
            parts += [self._heads(tensors[n["k"]], KV, self.head_dim, turned=True), self._heads(tensors[n["v"]], KV, self.value_dim)]
        self.w_qkv = rt.matrix(torch.cat(parts, dim=0)).contiguous()
        self.w_g = rt.matrix(self._heads(tensors[n["g"]], H, self.value_dim).contiguous()) if self.output_gate else None
        w_o = tensors[n["o"]]
        if self.value_dim < self.row:
            w_o = torch.cat([w_o.reshape(-1, H, self.value_dim), w_o.new_zeros((w_o.shape[0], H, self.row - self.value_dim))], dim=2)
            w_o = w_o.reshape(-1, H * self.row).contiguous()
        self.w_o = rt.matrix(w_o)
        self.inv_freq = self.position.inv_freq(rt.device)
        self.b_qkv = None
        if self.bias_suffix:
            sides = [("q", H, self.head_dim, True)] + ([("k", KV, self.head_dim, True), ("v", KV, self.value_dim, False)] if self.own_kv else [])
            self.b_qkv = torch.cat([self._heads(tensors[n[s] + self.bias_suffix].reshape(-1, 1), heads, size, turned=t).reshape(-1)
                                    for s, heads, size, t in sides]).float().contiguous()
        self.temperature = tensors[self.temperature_name].float().contiguous() if self.temperature_name else None
        self.sink = tensors[self.sink_name].float().contiguous() if self.sink_name else None
        self.talk = None
        if self.pooled:            # heads that do not talk are mixed by the unit matrix, in the same launch that rounds
            self.talk = (tensors[self.talk_name].float() if self.talk_name else torch.eye(H, device=self.w_o.device)).contiguous()
        self.value_freq = self.value_back = None
        if self.value_position is not None:
            self.value_freq = self.value_position.inv_freq(rt.device)
            self.value_back = (-self.value_freq).contiguous()            # the same angles the other way round

    def _project_out(self, ctx, x, out):
        if self.output_gate:
            ctx.ops.mul_sigmoid(out, ctx.ops.linear(x, self.w_g, ctx.dtype))
        if self.output_dtype is not None:
            return ctx.ops.linear(out, self.w_o, self.output_dtype)
        return ctx.ops.linear(out, self.w_o, ctx.dtype, defer=True)

    def _turn(self, ctx, rows, heads, freq):
        """Turn every head of `rows` by its position, over the values' elements, in place."""
        ctx.ops.rope_kv_write(rows, None, None, heads, 0, self.row, freq, self.value_dim, ctx.row_seq, ctx.row_pos, ctx.new_len,
                              None, None, None, 0, write=False)

    def _forward_pooled(self, ctx, x, site):
        import torch
        ops = ctx.ops
        H, KV, hd = self.num_heads, self.num_kv_heads, self.row
        if ctx.cache_owner != ctx.entry:
            raise ValueError("an attention with unit norms, pooled blocks or talking heads runs on its own cache")
        if site.spec.window is not None and not 0 < self.reach <= site.spec.window:
            raise ValueError(f"this attention sees {self.reach or 'all'} keys back, the cache it reads keeps {site.spec.window}")
        table = ctx.page_table(site.group_index)
        k_pool, v_pool = site.tensor("k"), site.tensor("v")
        rows_cap = site.rows_cap or 0
        qkv = ops.linear(x, self.w_qkv, torch.float32)                # float32 sums: bias, rotation and norm before any rounding
        q, k, v = ops.qkv_prepare(qkv, self.b_qkv, H, KV, hd, self.head_dim, self.inv_freq, self.position.rotary_dim, ctx.row_pos,
                                  self.unit_norm_eps, ctx.dtype)
        blocks = None
        if self.pool:
            bsite = self.tokens(ctx, "blocks")
            btable = ctx.page_table(bsite.group_index)
            kb, vb = bsite.tensor("k"), bsite.tensor("v")
            # the blocks this step completes are seen by its own later queries: their means are written first (the
            # pool keeps every block, so nothing a query still needs is overwritten)
            ops.pool_write(k, v, KV, hd, self.pool, ctx.cu_rows, ctx.max_count, ctx.new_len, ctx.slot_ids,
                           self.state(ctx, "block_sums"), btable, kb, vb)
            blocks = (self.pool, btable, kb, vb)
        a = ops.attention_pooled(q, k, v, H, KV, hd, ctx.cu_rows, ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool,
                                 rows_cap, self.query_scale, self.softcap, self.window, blocks=blocks,
                                 all_values=self.talk_name is not None, max_count=ctx.max_count)
        out = ops.talk_mix(a, self.talk, ctx.dtype)
        ops.kv_write(k, v, KV, hd, ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool, rows_cap)
        return self._project_out(ctx, x, out)

    def forward(self, ctx, x, site):
        if self.pooled:
            return self._forward_pooled(ctx, x, site)
        ops = ctx.ops
        H, KV, hd = self.num_heads, self.num_kv_heads, self.row
        Q, KVD = H * hd, KV * hd
        owns_cache = ctx.cache_owner == ctx.entry
        if owns_cache and not self.own_kv:
            raise ValueError("an attention without key and value projections must read another run's cache")
        w_in = self.w_qkv if owns_cache else self.w_qkv[:Q]          # a run on another run's cache projects its queries only
        if site.spec.window is not None and not 0 < self.reach <= site.spec.window:
            raise ValueError(f"this attention sees {self.reach or 'all'} keys back, the cache it reads keeps {site.spec.window}")
        if site.spec.shape_of("k") != (KV, hd):
            raise ValueError(f"the cache read here keeps keys of {site.spec.shape_of('k')}, this layer needs {(KV, hd)}")
        table = ctx.page_table(site.group_index)
        k_pool, v_pool = site.tensor("k"), site.tensor("v")         # [pages, kv_heads, page, row]
        rows_cap = site.rows_cap or 0
        bias = None if self.b_qkv is None else (self.b_qkv if owns_cache else self.b_qkv[:Q])
        more = dict(chunk=self.chunk, head_scale=self.temperature, sink=self.sink) if self.per_head else {}
        if ctx.mode == "decode" and bias is None and not self.per_head and self.value_freq is None and ops.fuses_decode_step(ctx.dtype, H, KV, hd, k_pool):
            # one launch rotates, writes the cache and attends; the projections may stay in K slices until then
            qkv = ops.linear(x, w_in, ctx.dtype, defer=True)
            out = ops.attention_decode_step(qkv, H, KV, hd, self.inv_freq, self.position.rotary_dim, ctx.new_len,
                                            table, k_pool, v_pool, rows_cap, self.query_scale, self.softcap,
                                            self.window, ctx.dtype, max_keys=ctx.max_rows_visible(site), write_kv=owns_cache)
            return self._project_out(ctx, x, out)
        qkv = ops.linear(x, w_in, ctx.dtype, bias=bias) if bias is not None else ops.linear(x, w_in, ctx.dtype)
        if owns_cache:
            q, k, v = qkv[:, :Q], qkv[:, Q:Q + KVD], qkv[:, Q + KVD:]
        else:
            q, k, v = qkv, None, None
        if self.value_freq is not None:
            self._turn(ctx, v, KV, self.value_freq)
        if ctx.mode == "decode":
            ops.rope_kv_write(q, k, v, H, KV, hd, self.inv_freq, self.position.rotary_dim,
                              ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool, rows_cap)
            out = ops.attention_decode(q, H, KV, hd, ctx.new_len, table, k_pool, v_pool, rows_cap,
                                       self.query_scale, self.softcap, self.window, ctx.dtype,
                                       max_keys=ctx.max_rows_visible(site), **more)
            if self.value_back is not None:
                self._turn(ctx, out, H, self.value_back)
            return self._project_out(ctx, x, out)
        # Sequences that go on by several tokens (or some start while others go on) see cached positions and the
        # step's own rows.  The attention reads the cached ones where they lie, as earlier steps left them, and the
        # step's rows from the step; only then are the step's rows cached: in a window's ring without a row to spare
        # they take the places of positions that the step's earlier queries still see.
        extend = ctx.mode == "extend"
        ops.rope_kv_write(q, k, v, H, KV, hd, self.inv_freq, self.position.rotary_dim,
                          ctx.row_seq, ctx.row_pos, ctx.new_len, table, k_pool, v_pool, rows_cap,
                          write=not extend)
        if owns_cache:
            ctx.offer_step_rows(k=k, v=v)
        else:
            theirs = ctx.step_rows_of(ctx.cache_owner)
            k, v = theirs["k"], theirs["v"]
        out = ops.attention_prefill(q, k, v, H, KV, hd, ctx.cu_rows, ctx.max_count,
                                    self.query_scale, self.softcap, self.window, ctx.dtype,
                                    row_seq=ctx.row_seq, row_pos=ctx.row_pos,
                                    cached=(ctx.new_len, table, k_pool, v_pool, rows_cap) if extend else None,
                                    wide_weights=self.precise_weights, **more)
        if self.value_back is not None:
            self._turn(ctx, out, H, self.value_back)
        if extend and owns_cache:
            row_seq, row_pos, new_len = ctx.row_seq, ctx.row_pos, ctx.new_len
            ctx.after_readers(lambda: ops.kv_write(k, v, KV, hd, row_seq, row_pos, new_len, table, k_pool, v_pool, rows_cap))
        return self._project_out(ctx, x, out)


register_part("mixer", "attention", Attention)
