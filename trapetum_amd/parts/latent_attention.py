"""Attention through a latent: one small vector per token is cached, and every head's keys and values are products of it.

Per token the layer caches c = rmsnorm(W_dkv h)[:rank] * w_norm (the latent) and r = rope(W_dkv h)[rank:] (one rotated
key part shared by all heads).  Head h has queries [q_n | q_r] = W_q h (q_r rotated like r), keys [W_uk,h c | r] and
values W_uv,h c; score = (q_n . W_uk,h c + q_r . r) * scale, causal softmax in fp32, output W_o over the heads.

Neither keys nor values are ever formed: q_n . (W_uk,h c) = (W_uk,h^T q_n) . c, so the query is carried into the
latent's space (one small product per head), the attention runs over the cached rows [r | c] themselves as one kv
head of rope_dim + rank elements that every query head shares, with the row serving as key and as value, and each
head's weighted sum of latents goes through W_uv,h afterwards.  The attention kernels are the ones grouped-query
attention uses (its `k` and `v` pools are one tensor here); the rotated part stands first in a row because those
kernels rotate a head's leading elements.  A step's cost is then one read of rope_dim + rank elements per cached
token for all heads, instead of heads * (dim + vdim).

Further parameters: `query_rank` (the queries go through a latent of their own, q = W_uq rmsnorm(W_dq h) * w_qnorm,
instead of one product), `window` W (the query at p sees the positions p - W + 1 .. p; the cache then keeps a ring),
`output_gate` (head h's output is multiplied by sigmoid(W_g h)_h, one number per head and token) and a rotation of
neighbouring pairs (2f, 2f + 1), carried out as the rotation of halves on projection rows reordered at bind (queries
and key part alike: every score is the same sum in another order).

A run with `own_latent=False` has no W_dkv: it attends over what the run named by its schedule entry's `cache_of`
cached (and, in the step that caches them, over that run's rows of this step), with its own queries, W_uk, W_uv, W_o.
"""
from ..cache.store import TokenSpec
from ..models.spec import TensorSpec
from ..registry import build_part, register_part
from .base import Mixer


class LatentAttention(Mixer):
    DECODE_GROUP, DECODE_GROUP_LONG, LONG_KEYS = 4, 8, 1536       # query heads a block of the decode attention takes (see forward)

    def __init__(self, hidden_size, num_heads, nope_dim, rope_dim, value_dim, latent_rank, scale, latent_eps,
                 position=("none", {}), own_latent=True,
                 tensors=("q", "dkv", "dkv.norm", "uk", "uv", "o"), query_rank=None, query_tensors=("dq", "dq.norm", "uq"),
                 window=None, output_gate=None, precise_weights=False):
        """query_rank: size of the queries' latent (None: queries are one product, tensor `q`); query_tensors: local
        names of W_dq, the latent's gain and W_uq.  window: positions back a query sees, its own included (None: all).
        output_gate: local name of W_g [heads, hidden] (None: no gate).  precise_weights: softmax weights of 16 bits of
        mantissa in the matrix-core kernel of many queries."""
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.nope_dim, self.rope_dim, self.value_dim, self.rank = int(nope_dim), int(rope_dim), int(value_dim), int(latent_rank)
        self.scale = float(scale)
        self.latent_eps = float(latent_eps)
        self.own_latent = bool(own_latent)
        self.position = build_part("position", position)
        if self.position.rotary_dim > self.rope_dim:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds the rotated part of {self.rope_dim}")
        self.names = dict(zip(("q", "dkv", "dkv_norm", "uk", "uv", "o"), tensors))
        self.query_rank = int(query_rank) if query_rank else 0
        self.names.update(zip(("dq", "dq_norm", "uq"), query_tensors))
        self.window = int(window) if window else 0
        self.gate_name = output_gate
        self.precise_weights = bool(precise_weights)

    @property
    def row(self):
        """Elements of a cached row: the rotated key part, then the latent."""
        return self.rope_dim + self.rank

    def tensor_specs(self):
        n, d, H = self.names, self.hidden_size, self.num_heads
        qd = H * (self.nope_dim + self.rope_dim)
        if self.query_rank:
            specs = {n["dq"]: TensorSpec((self.query_rank, d)), n["dq_norm"]: TensorSpec((self.query_rank,), init="gain"),
                     n["uq"]: TensorSpec((qd, self.query_rank))}
        else:
            specs = {n["q"]: TensorSpec((qd, d))}
        if self.gate_name:
            specs[self.gate_name] = TensorSpec((H, d))
        specs.update({n["uk"]: TensorSpec((H * self.nope_dim, self.rank)), n["uv"]: TensorSpec((H * self.value_dim, self.rank)),
                 n["o"]: TensorSpec((d, H * self.value_dim))})
        if self.own_latent:
            specs[n["dkv"]] = TensorSpec((self.rank + self.rope_dim, d))
            specs[n["dkv_norm"]] = TensorSpec((self.rank,), init="gain")
        return specs

    def cache_spec(self):
        return TokenSpec.of(self.window or None, latent=(1, self.row))

    def bind(self, tensors, rt):
        import torch
        self.rt = rt
        n, H, dn, dr, dv, R = self.names, self.num_heads, self.nope_dim, self.rope_dim, self.value_dim, self.rank
        # queries head by head as [rotated | unrotated], the down-projection as [rotated key part | latent]: the order
        # of a cached row, and of the query that meets it
        rot = self.position.rotary_dim
        turned = list(range(dr))                         # the rotated part's rows in the order the kernels turn them
        if rot and self.position.pairing == "neighbours":
            turned = list(range(0, rot, 2)) + list(range(1, rot, 2)) + list(range(rot, dr))
        wq = tensors[n["uq"] if self.query_rank else n["q"]].reshape(H, dn + dr, -1)
        wq = torch.cat([wq[:, dn:][:, turned], wq[:, :dn]], dim=1).reshape(H * (dn + dr), -1)
        wd = tensors[n["dkv"]] if self.own_latent else None
        tail = torch.cat([wd[R:][turned], wd[:R]], dim=0) if self.own_latent else None
        self.latent_gain = tensors[n["dkv_norm"]].float().contiguous() if self.own_latent else None
        self.w_in = self.w_tail = self.w_dq = self.w_uq = self.query_gain = None
        if self.query_rank:
            self.w_dq = rt.matrix(tensors[n["dq"]].contiguous())
            self.query_gain = tensors[n["dq_norm"]].float().contiguous()
            self.w_uq = rt.matrix(wq.contiguous())
            if self.own_latent:
                self.w_tail = rt.matrix(tail.contiguous())
        else:
            self.w_in = rt.matrix((torch.cat([wq, tail], dim=0) if self.own_latent else wq).contiguous())
        self.w_gate = rt.matrix(tensors[self.gate_name].contiguous()) if self.gate_name else None
        self.w_absorb = rt.matrix(tensors[n["uk"]].reshape(H, dn, R).transpose(1, 2).contiguous())     # [H, rank, dim]
        self.w_up = rt.matrix(tensors[n["uv"]].reshape(H, dv, R).contiguous())                         # [H, vdim, rank]
        self.w_o = rt.matrix(tensors[n["o"]])
        self.inv_freq = self.position.inv_freq(rt.device)

    def forward(self, ctx, x, site):
        ops = ctx.ops
        H, dn, dr, dv, R, row = self.num_heads, self.nope_dim, self.rope_dim, self.value_dim, self.rank, self.row
        owns = ctx.cache_owner == ctx.entry
        if owns != self.own_latent:
            raise ValueError("a latent attention without a down-projection must read another run's cache, and one with it its own")
        if site.spec.shape_of("latent") != (1, row):
            raise ValueError(f"the cache read here keeps rows of {site.spec.shape_of('latent')}, this layer needs (1, {row})")
        table = ctx.page_table(site.group_index)
        pool = site.tensor("latent")                              # [pages, 1, page, rope_dim + rank]
        rows_cap = site.rows_cap or 0
        m = x.shape[0]
        import torch
        tail = None
        if self.query_rank:
            cq = ops.rms_norm(ops.linear(x, self.w_dq, torch.float32), self.query_gain, self.latent_eps, ctx.dtype)
            proj = ops.linear(cq, self.w_uq, ctx.dtype)           # [M, H (dr + dn)]
            if owns:
                tail = ops.linear(x, self.w_tail, ctx.dtype)      # [M, dr + rank]
        else:
            proj = ops.linear(x, self.w_in, ctx.dtype)            # [M, H (dr + dn) (+ dr + rank)]
        # A step that continues sequences by several tokens reads the ring as earlier steps left it, so its rows are
        # cached after the attention: in a ring they may take the places of positions that its first queries still see.
        late = owns and ctx.mode == "extend" and bool(rows_cap)
        # rotations, the latent's norm and the cache write in one launch: the queries' rotated parts go to their
        # places in q, the step's rows [r | c] to `mine` and into the cache
        q, mine = ops.latent_prepare(proj, H, dn, dr, R, self.latent_gain, self.latent_eps, self.inv_freq,
                                     self.position.rotary_dim, ctx.row_seq, ctx.row_pos, ctx.new_len, table, pool,
                                     rows_cap, own=owns, out_dtype=ctx.dtype, tail=tail, write=not late)
        ops.head_linear(proj[:, :H * (dr + dn)].view(m, H, dr + dn)[:, :, dr:], self.w_absorb, q.view(m, H, row)[:, :, dr:])
        if ctx.mode == "decode":
            # All heads share the one kv head.  A block of the decode kernel forms the weighted sums of a kv head's
            # query heads by multiply-adds in its lanes, so the heads are cut into groups, each group a block of its
            # own on the same cached rows, and the keys' slices are counted for that many kv heads.  Measured at 16
            # heads and rows of 256 elements, heads a block 16 / 8 / 4 / 2: 8 sequences at 552 keys 18.3 / 13.4 / 11.9 /
            # 11.2 us, at 2,048 keys 20.7 / 17.6 / 22.3 / 23.1, at 7,900 keys 68.7 / 39.6 / 46.2 / 51.9; 64 sequences at
            # 552 keys 46.8 / 35.5 / 30.0 / 36.5.
            keys = ctx.max_rows_visible(site)
            per = next(g for g in (self.DECODE_GROUP_LONG if keys >= self.LONG_KEYS else self.DECODE_GROUP, 4, 2, 1) if H % g == 0)
            out = ops.attention_decode(q, H, 1, row, ctx.new_len, table, pool, pool, rows_cap, self.scale, 0.0, self.window,
                                       ctx.dtype, max_keys=keys, head_groups=H // per,
                                       splits=ops.decode_splits(m * (H // per), 1, row, keys))
        else:
            if owns:
                ctx.offer_step_rows(latent=mine)
            else:
                mine = ctx.step_rows_of(ctx.cache_owner)["latent"]
            extend = ctx.mode == "extend"
            out = ops.attention_prefill(q, mine, mine, H, 1, row, ctx.cu_rows, ctx.max_count, self.scale, 0.0, self.window, ctx.dtype,
                                        row_seq=ctx.row_seq, row_pos=ctx.row_pos,
                                        cached=(ctx.new_len, table, pool, pool, rows_cap) if extend else None,
                                        wide_weights=self.precise_weights)
            if late:
                row_seq, row_pos, new_len = ctx.row_seq, ctx.row_pos, ctx.new_len
                ctx.after_readers(lambda: ops.kv_write(mine, mine, 1, row, row_seq, row_pos, new_len, table, pool, pool, rows_cap))
        heads = ops.head_linear(out.view(m, H, row)[:, :, dr:], self.w_up, None)      # [M, H, vdim]
        if self.w_gate is not None:
            ops.mul_sigmoid_heads(heads.view(m, H * dv), ops.linear(x, self.w_gate, torch.float32), H)
        return ops.linear(heads.view(m, H * dv), self.w_o, ctx.dtype, defer=True)


register_part("mixer", "latent_attention", LatentAttention)
