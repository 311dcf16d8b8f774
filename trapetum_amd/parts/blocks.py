"""How a layer's parts are arranged around the residual stream.

sandwich  x += post_mixer_norm(mixer(pre_mixer_norm(x)));
          x += post_ff_norm(ff(pre_ff_norm(x)))          (runtime/src/lib.rs:4527-4540)
pre_norm  x += mixer(pre_mixer_norm(x));  x += ff(pre_ff_norm(x)); the feed-forward may be absent
          (the reference's other layer type, runtime/src/lib.rs:721-730).  With `token_shift` the mixer reads
          h + (h' - h) * w instead of h = pre_mixer_norm(x), h' being the h of the token before (zeros before the
          sequence) and w a vector of the layer; the last token's h is a state of the sequence.
post_norm x += post_mixer_norm(mixer(c1(x)));  x += post_ff_norm(ff(c2(x))): no norm in front of a sub-layer; c1
          and c2 are what it reads of the stream, the stream itself or (input_conv) the stream through a short
          causal convolution whose last rows are a state of the sequence.  The feed-forward may be absent.

The stream is fp32 and the sum is formed in fp32 (the reference adds in fp32 and
stores fp16: runtime/cuda/codebook_gemv.cu:539-542).  Where a norm of a sub-layer's
output is followed by the add and by the next norm, one kernel does all three; that
includes the first norm of the block that runs next (`next_norm`), whose result the
next block receives as `normed`.
"""
from ..registry import register_part
from .base import Block


def add_then_norm(ctx, stream, rows, post, nxt):
    """stream += post(rows) (or rows); returns nxt(stream) (or None).  One kernel when both norms
    expose an RMS gain, else the norms' own forward around a plain add."""
    fusable = all(n is None or n.gain is not None for n in (post, nxt))
    groups = {getattr(n, "groups", 1) for n in (post, nxt) if n is not None}      # one kernel cuts both norms alike
    if fusable and len(groups) <= 1:
        return ctx.ops.add_rms_norm(stream, rows,
                                    post.gain if post else None, post.eps if post else 0.0,
                                    nxt.gain if nxt else None, nxt.eps if nxt else 0.0,
                                    getattr(nxt, "reader_dtype", None) or ctx.dtype,       # a reader may ask for float32 rows
                                    groups=groups.pop() if groups else 1)
    rows = ctx.ops.rows(rows, ctx.dtype)
    if post is not None:
        rows = post.forward(ctx, rows)
    ctx.ops.add_rms_norm(stream, rows, None, 0.0, None, 0.0, ctx.dtype)
    return nxt.forward(ctx, stream, getattr(nxt, "reader_dtype", None)) if nxt is not None else None


class SandwichBlock(Block):
    def __init__(self, mixer, feed_forward, make_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward                 # None: the layer is its mixer, with the norms around it
        sites = self.norm_sites() if feed_forward is not None else self.norm_sites()[:2]
        self.norms = {name: make_norm(name) for name in sites}

    @classmethod
    def norm_sites(cls):
        return ("pre_mixer_norm", "post_mixer_norm", "pre_ff_norm", "post_ff_norm")

    def entry_norm(self):
        return self.norms["pre_mixer_norm"]

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        n = self.norms
        x = normed if normed is not None else n["pre_mixer_norm"].forward(ctx, stream)
        ctx.dump("mixer_in", x)
        a = self.mixer.forward(ctx, x, site)
        ctx.dump("mixer_out", a)
        if self.feed_forward is None:
            normed_next = add_then_norm(ctx, stream, a, n["post_mixer_norm"], next_norm)
            ctx.dump("layer_out", stream)
            return stream, normed_next
        x = add_then_norm(ctx, stream, a, n["post_mixer_norm"], n["pre_ff_norm"])
        ctx.dump("after_mixer", stream)
        m = self.feed_forward.forward(ctx, x)
        ctx.dump("ff_out", m)
        normed_next = add_then_norm(ctx, stream, m, n["post_ff_norm"], next_norm)
        ctx.dump("layer_out", stream)
        return stream, normed_next


class PreNormBlock(Block):
    def __init__(self, mixer, feed_forward, make_norm, token_shift=None):
        """token_shift: the local name of the mixing vector [hidden] (None: the mixer reads the normed rows as they are)."""
        self.mixer = mixer
        self.feed_forward = feed_forward                 # None: the layer is its mixer behind its norm
        sites = self.norm_sites() if feed_forward is not None else self.norm_sites()[:1]
        self.norms = {name: make_norm(name) for name in sites}
        self.token_shift = token_shift
        if token_shift is not None:
            import torch
            # the mix is formed in float32 from float32 rows and rounded once; whoever applies this block's first norm
            # (the block itself, or the block before in the kernel of its last add) leaves the rows in float32
            self.norms["pre_mixer_norm"].reader_dtype = torch.float32

    @classmethod
    def norm_sites(cls):
        return ("pre_mixer_norm", "pre_ff_norm")

    def entry_norm(self):
        return self.norms["pre_mixer_norm"]

    def tensor_specs(self):
        if self.token_shift is None:
            return {}
        from ..models.spec import TensorSpec
        return {self.token_shift: TensorSpec((self.norms["pre_mixer_norm"].size,), init="norm")}

    def state_specs(self):
        if self.token_shift is None:
            return {}
        from ..cache.store import StateSpec
        return {"token_shift": StateSpec((self.norms["pre_mixer_norm"].size,), "float32")}

    def bind(self, tensors, rt):
        self.rt = rt
        if self.token_shift is not None:
            self.shift_weight = tensors[self.token_shift].float().reshape(1, -1).contiguous()

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        n = self.norms
        first = n["pre_mixer_norm"]
        x = normed if normed is not None else first.forward(ctx, stream, getattr(first, "reader_dtype", None))
        if self.token_shift is not None:
            x = ctx.ops.shift_mix(x, self.shift_weight, ctx.cache.entry_state(ctx.entry, "token_shift"), ctx.slot_ids, ctx.cu_rows,
                                  ctx.row_seq, one_row_each=ctx.mode == "decode", out_dtype=ctx.dtype)[0]
        ctx.dump("mixer_in", x)
        a = self.mixer.forward(ctx, x, site)
        ctx.dump("mixer_out", a)
        if self.feed_forward is None:
            normed_next = add_then_norm(ctx, stream, a, None, next_norm)
            ctx.dump("layer_out", stream)
            return stream, normed_next
        x = add_then_norm(ctx, stream, a, None, n["pre_ff_norm"])
        ctx.dump("after_mixer", stream)
        m = self.feed_forward.forward(ctx, x)
        ctx.dump("ff_out", m)
        normed_next = add_then_norm(ctx, stream, m, None, next_norm)
        ctx.dump("layer_out", stream)
        return stream, normed_next


class PostNormBlock(Block):
    def __init__(self, mixer, feed_forward, make_norm, input_conv=None):
        """input_conv: (registered conv, parameters) built once in front of each sub-layer, or None."""
        from ..registry import build_part
        self.mixer = mixer
        self.feed_forward = feed_forward
        sites = ("post_mixer_norm", "post_ff_norm") if feed_forward is not None else ("post_mixer_norm",)
        self.norms = {name: make_norm(name) for name in sites}
        self.convs = {}
        if input_conv is not None:
            for site in ("mixer_conv", "ff_conv")[:len(sites)]:
                self.convs[site] = build_part("conv", input_conv)

    @classmethod
    def norm_sites(cls):
        return ("post_mixer_norm", "post_ff_norm")

    def inner_parts(self):
        return dict(self.convs)

    def state_specs(self):
        return {site: c.state_spec() for site, c in self.convs.items() if c.state_spec() is not None}

    def _read(self, ctx, stream, site):
        conv = self.convs.get(site)
        if conv is None:
            return stream.to(ctx.dtype)
        state = ctx.cache.entry_state(ctx.entry, site) if conv.state_spec() is not None else None
        return conv.forward(ctx, stream, state)

    def forward(self, ctx, stream, site, normed=None, next_norm=None):
        n = self.norms
        x = self._read(ctx, stream, "mixer_conv")
        ctx.dump("mixer_in", x)
        a = self.mixer.forward(ctx, x, site)
        ctx.dump("mixer_out", a)
        if self.feed_forward is None:
            normed_next = add_then_norm(ctx, stream, a, n["post_mixer_norm"], next_norm)
            ctx.dump("layer_out", stream)
            return stream, normed_next
        add_then_norm(ctx, stream, a, n["post_mixer_norm"], None)
        ctx.dump("after_mixer", stream)
        x = self._read(ctx, stream, "ff_conv")
        m = self.feed_forward.forward(ctx, x)
        ctx.dump("ff_out", m)
        normed_next = add_then_norm(ctx, stream, m, n["post_ff_norm"], next_norm)
        ctx.dump("layer_out", stream)
        return stream, normed_next


register_part("block", "sandwich", SandwichBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "pre_norm", PreNormBlock)
