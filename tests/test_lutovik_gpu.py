"""Lutovik on the GPU: each mechanism's kernels alone against the plain functions of tests/plain, then the model through
the step function, the cache and the generation entry point, in float32 and bfloat16."""
import pytest
import torch

from trapetum_amd.cache import ModelCache
from trapetum_amd.engine.batch import StepContext
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.registry import build_part

from . import lutovik_tiny as lt
from . import model_cases as mc
from . import ref_ops
from .plain import lutovik_plain as plain
from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-5, "bfloat16": mc.Rounded(4e-2)}
PART_TOL = {torch.float32: 4e-6, torch.bfloat16: 1e-2}
WIDTH = 72


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def rt(request):
    return Runtime(dtype=request.param, device=DEV)


def stored(t):
    """A tensor as a model folder stores it (bf16), for the device and widened for the plain functions."""
    b = t.to(torch.bfloat16)
    return b.to(DEV), b.double()


def acts(rt, t):
    a = t.to(rt.dtype)
    return a.to(DEV), a.double()


def bound(rt, kind, ref, tensors):
    """A part with its tensors bound; returns (part, {name: the stored values in float64})."""
    part = build_part(kind, ref)
    dev, wide = {}, {}
    for k, v in tensors.items():
        dev[k], wide[k] = stored(v)
    assert set(part.tensor_specs()) == set(tensors), (sorted(part.tensor_specs()), sorted(tensors))
    for k, spec in part.tensor_specs().items():
        assert tuple(spec.shape) == tuple(tensors[k].shape), k
    part.bind(dev, rt)
    return part, wide


def run_mixers(rt, mixers, seqs, steps, page=16):
    """`mixers`: [(part, entry whose cache it reads)], one schedule entry each.  `seqs`: {id: rows [n, WIDTH] on the
    device}.  `steps`: [{id: count}]: every step brings the next `count` rows of its sequences.  Returns
    {id: [per mixer: rows [n, WIDTH]]}."""
    specs = [m.cache_spec() if owner == i else None for i, (m, owner) in enumerate(mixers)]
    states = [{"mixer." + k: v for k, v in m.state_specs().items()} for m, _ in mixers]
    tokens = [{"mixer." + k: v for k, v in m.token_specs().items()} if owner == i else {} for i, (m, owner) in enumerate(mixers)]
    cache = ModelCache(specs, 4096, 4096, 8, page, rt.dtype, rt.device, entry_states=states, entry_tokens=tokens)
    slots = {i: cache.acquire() for i in seqs}
    done = {i: 0 for i in seqs}
    got = {i: [[] for _ in mixers] for i in seqs}
    for counts in steps:
        ids = sorted(counts)
        starts = [cache.length(slots[i]) for i in ids]
        for i in ids:
            cache.grow(slots[i], counts[i])
        ctx = StepContext(rt, cache, [slots[i] for i in ids], [counts[i] for i in ids], starts, [])
        ctx.mark_shared(sorted({owner for e, (_, owner) in enumerate(mixers) if owner != e}))
        x = torch.cat([seqs[i][done[i]:done[i] + counts[i]] for i in ids])
        for e, (part, owner) in enumerate(mixers):
            ctx.entry, ctx.cache_owner = e, owner
            out = rt.ops.rows(part.forward(ctx, x, cache.site(owner)), rt.dtype)
            at = 0
            for i in ids:
                got[i][e].append(out[at:at + counts[i]])
                at += counts[i]
        ctx.finish()
        for i in ids:
            done[i] += counts[i]
    for i in seqs:
        assert done[i] == seqs[i].shape[0]
    return {i: [torch.cat(rows) for rows in got[i]] for i in seqs}


# a long prompt, single tokens, portions down to two rows, a second sequence that joins and goes on beside the first
STEPS = [{0: 70}, {0: 1, 1: 1}, {0: 1, 1: 1}, {0: 2, 1: 37}, {0: 1}, {1: 1}, {0: 25, 1: 2}, {0: 1, 1: 1}]
LENS = {0: 101, 1: 43}


# ---- attention: values of their own size, scaled frequencies, both pairings, a gate, another layer's cache -----------------
def attention_part(rt, H, G, dim, vdim, rot, pairing, scaling=None, gate=False, own=True, seed=0, scale=0.3, edit=None):
    sc = None if scaling is None else dict(zip(("factor", "low", "high", "original"), scaling))
    position = ("rope", {"rotary_dim": rot, "theta": 300.0, "pairing": pairing, "scaling": sc}) if rot else ("none", {})
    T = {"q": rnd(H * dim, WIDTH, seed=seed + 1, scale=0.25), "o": rnd(WIDTH, H * vdim, seed=seed + 2, scale=0.2)}
    if own:
        T["k"], T["v"] = rnd(G * dim, WIDTH, seed=seed + 3, scale=0.25), rnd(G * vdim, WIDTH, seed=seed + 4, scale=0.3)
    if gate:
        T["g"] = rnd(H * vdim, WIDTH, seed=seed + 5, scale=0.3)
    if edit is not None:
        edit(T)
    part, W = bound(rt, "mixer", ("attention", dict(
        hidden_size=WIDTH, num_heads=H, num_kv_heads=G, head_dim=dim, value_dim=vdim, query_scale=scale, position=position,
        output_gate=gate, own_kv=own, precise_weights=True, tensors=("q", "k", "v", "o", "g"))), T)
    sizes = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": 300.0, "dims": rot}}
    if sc is not None:
        sizes["rot"]["scaling"] = sc
    return part, W, sizes


@pytest.mark.parametrize("H,G,dim,vdim,rot,pairing,scaling,gate", [
    (4, 2, 16, 24, 8, "neighbours", (8.0, 1.0, 3.0, 64), False), (2, 1, 32, 16, 32, "halves", None, True),
    (10, 5, 64, 64, 24, "neighbours", (3.0, 2.0, 8.0, 100), False), (4, 4, 48, 80, 48, "halves", None, True),
    (1, 1, 12, 12, 0, "halves", None, True), (3, 1, 20, 36, 6, "neighbours", None, True), (8, 2, 128, 64, 64, "neighbours", None, False)])
def test_attention_part(rt, H, G, dim, vdim, rot, pairing, scaling, gate):
    """The mixer alone, and a second one without key and value projections on the first one's cache."""
    tol = PART_TOL[rt.dtype] * (3 if rt.dtype == torch.float32 else 1.5)
    part, W, sizes = attention_part(rt, H, G, dim, vdim, rot, pairing, scaling, gate)
    reader, W2, _ = attention_part(rt, 2 * H, G, dim, vdim, rot, pairing, scaling, gate, own=False, seed=40)
    seqs, wide = {}, {}
    for i, n in LENS.items():
        seqs[i], wide[i] = acts(rt, rnd(n, WIDTH, seed=9 + i))
    got = run_mixers(rt, [(part, 0), (reader, 0)], seqs, STEPS)
    for i in seqs:
        want, kv = plain.attention(wide[i], W, "", sizes, pairing, gated=gate)
        want2, _ = plain.attention(wide[i], W2, "", dict(sizes, heads=2 * H), pairing, kv=kv, gated=gate)
        assert rel_l2(got[i][0], want) < tol, i
        assert rel_l2(got[i][1], want2) < tol, i


@pytest.mark.parametrize("page,first", [(16, 64), (16, 63), (16, 65), (64, 257)])
def test_attention_one_key_stands_out(rt, page, first):
    """One early key is made to stand out for every later query (a large component that only it and the queries have, in
    an element outside the rotation): the outputs are then that key's value, from a prompt, a portion and single tokens
    alike, wherever the pages' borders fall.  Lost, or taken one place off, it would show whole."""
    H, G, dim, vdim, rot, at = 4, 2, 16, 24, 8, 3

    def mark(T):                                         # a head's last element: keys read column 5 of the input, queries column 7
        for name, heads, col in (("k", G, 5), ("q", H, 7)):
            w = T[name].view(heads, dim, WIDTH)
            w[:, dim - 1, :] = 0.0
            w[:, dim - 1, col] = 1.0
    part, W, sizes = attention_part(rt, H, G, dim, vdim, rot, "neighbours", (8.0, 1.0, 3.0, 64), seed=7, scale=1.0, edit=mark)
    n = first + 2 * page + 9
    x = rnd(n, WIDTH, seed=3) * 0.3
    x[:, 5] = 0.0
    x[at, 5] = 30.0                                      # the marked key
    x[:, 7] = 3.0                                        # every query meets it with a score of 90
    x_dev, xw = acts(rt, x)
    want, _ = plain.attention(xw, W, "", sizes, "neighbours")
    steps = [{0: first}, {0: 2 * page + 1}] + [{0: 1}] * 8
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps, page=page)[0][0]
    assert rel_l2(got[at + 1:], want[at + 1:]) < (2e-5 if rt.dtype == torch.float32 else 2e-2)
    # and the plain outputs do rest on that key: without it they are something else
    x2 = xw.clone()
    x2[at, 5] = 0.0
    other, _ = plain.attention(x2, W, "", sizes, "neighbours")
    assert rel_l2(other[at + 1:], want[at + 1:]) > 0.3


# ---- the state-space mixer --------------------------------------------------------------------------------------------------
def state_space_part(rt, heads, P, N, groups, taps, norm_groups, seed=0, a_log=None):
    inner, ch = heads * P, heads * P + 2 * groups * N
    T = {"in": rnd(inner + ch + heads, WIDTH, seed=seed + 1, scale=0.2), "conv": rnd(ch, taps, seed=seed + 2, scale=0.4),
         "conv.b": rnd(ch, seed=seed + 3, scale=0.2), "dt_bias": rnd(heads, seed=seed + 4, scale=0.5),
         "A_log": rnd(heads, seed=seed + 5, scale=0.5) if a_log is None else torch.full((heads,), float(a_log)),
         "D": 1.0 + rnd(heads, seed=seed + 6, scale=0.3), "norm": 1.0 + rnd(inner, seed=seed + 7, scale=0.2),
         "o": rnd(WIDTH, inner, seed=seed + 8, scale=0.2)}
    part, W = bound(rt, "mixer", ("state_space", dict(hidden_size=WIDTH, num_heads=heads, head_dim=P, state_size=N, groups=groups,
                                                    conv_taps=taps, norm_groups=norm_groups, norm_eps=1e-5)), T)
    sizes = {"heads": heads, "vdim": P, "state": N, "groups": groups, "conv": taps, "norm_groups": norm_groups}
    return part, W, sizes


@pytest.mark.parametrize("heads,P,N,groups,taps,norm_groups", [(4, 12, 16, 2, 4, 3), (1, 10, 4, 1, 1, 1), (3, 20, 8, 1, 2, 1),
                                                              (6, 64, 48, 3, 3, 2), (2, 80, 24, 2, 5, 4), (6, 16, 128, 3, 2, 1),
                                                              (2, 130, 40, 1, 3, 2)])
def test_state_space_part(rt, heads, P, N, groups, taps, norm_groups):
    part, W, sizes = state_space_part(rt, heads, P, N, groups, taps, norm_groups)
    seqs, wide = {}, {}
    for i, n in LENS.items():
        seqs[i], wide[i] = acts(rt, rnd(n, WIDTH, seed=19 + i))
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        assert rel_l2(got[i][0], plain.state_space(wide[i], W, "", sizes, 1e-5)) < PART_TOL[rt.dtype] * 3, i


@pytest.mark.parametrize("cut", ["whole", "pieces", "one by one"])
def test_state_space_keeps_its_first_tokens(rt, cut):
    """A state that hardly decays: what the first tokens wrote is still most of every output hundreds of tokens later,
    through a scan cut into pieces, through portions and through single tokens.  A state lost, or started anew at a piece's
    edge, would show whole."""
    part, W, sizes = state_space_part(rt, 4, 24, 16, 2, 3, 2, seed=60, a_log=-9.0)
    n = 333
    x = rnd(n, WIDTH, seed=61) * 0.2
    x[:6] *= 20.0                                        # the first tokens write far more than the later ones
    x_dev, xw = acts(rt, x)
    want = plain.state_space(xw, W, "", sizes, 1e-5)
    steps = {"whole": [{0: n}], "pieces": [{0: 130}, {0: 64}, {0: 65}, {0: 2}, {0: 72}], "one by one": [{0: 200}] + [{0: 1}] * 133}[cut]
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps)[0][0]
    assert rel_l2(got, want) < PART_TOL[rt.dtype] * 5
    x2 = xw.clone()
    x2[:6] = 0.0
    assert rel_l2(plain.state_space(x2, W, "", sizes, 1e-5)[200:], want[200:]) > 0.3


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rate", [0.0, 2.5, 4.0])
@pytest.mark.parametrize("counts,heads,groups,N,P,taps", [([5], 2, 1, 16, 8, 3), ([1, 1, 1], 4, 2, 32, 40, 3), ([70, 1, 200, 33], 6, 3, 48, 40, 4),
                                                          ([300], 4, 4, 24, 80, 2), ([130, 65], 2, 1, 128, 64, 1), ([700], 1, 1, 200, 16, 2)])
def test_conv_and_scan_kernels(dt, rate, counts, heads, groups, N, P, taps):
    """The convolution and the scan against their plain torch references, from states that are not zero, in slots that are
    not the sequences' numbers.  rate: added to A_log; decays of e^-12 and e^-55 a row and less, whose running product
    leaves float32's range within a few rows, or which do so alone."""
    ops = Runtime(dtype="float32", device=DEV).ops
    m, inner, n = sum(counts), heads * P, len(counts)
    C = inner + 2 * groups * N
    u = rnd(m, 2 * inner + 2 * groups * N + heads, seed=1).to(dt)
    wt, bias = rnd(taps, C, seed=2, scale=0.5), rnd(C, seed=3, scale=0.2)
    slots = torch.tensor([3, 0, 5, 1][:n], dtype=torch.int32)
    cu = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
    row_seq = torch.repeat_interleave(torch.arange(n, dtype=torch.int32), torch.tensor(counts))
    cst = rnd(7, max(taps - 1, 1), C, seed=4)[:, :taps - 1].contiguous() if taps > 1 else None
    sst = rnd(7, heads, N, P, seed=5)
    dt_bias, a_log, skip = rnd(heads, seed=6), rnd(heads, seed=7, scale=0.5) + rate, 1 + rnd(heads, seed=8, scale=0.2)
    cst_r, sst_r = (cst.clone() if cst is not None else None), sst.clone()
    xbc_r = ref_ops.conv_act(u[:, inner:inner + C], wt, bias, cst_r, slots, cu, row_seq, "silu")
    y_r = ref_ops.ssd_scan(xbc_r, u[:, :inner], u[:, inner + C:], dt_bias, a_log, skip, sst_r, slots, cu, max(counts), heads, groups, N, P)
    ud, cst_d, sst_d = u.to(DEV), (cst.to(DEV) if cst is not None else None), sst.to(DEV)
    xbc = ops.conv_act(ud[:, inner:inner + C], wt.to(DEV), bias.to(DEV), cst_d, slots.to(DEV), cu.to(DEV), row_seq.to(DEV), "silu",
                       one_row_each=all(c == 1 for c in counts))
    y = ops.ssd_scan(xbc, ud[:, :inner], ud[:, inner + C:], dt_bias.to(DEV), a_log.to(DEV), skip.to(DEV), sst_d, slots.to(DEV), cu.to(DEV),
                     max(counts), heads, groups, N, P)
    assert rel_l2(xbc, xbc_r) < (2e-6 if dt == torch.float32 else 4e-3)
    assert cst is None or torch.equal(cst_d.cpu(), cst_r)
    assert rel_l2(y, y_r) < 3e-6 and rel_l2(sst_d, sst_r) < 2e-6 and bool(torch.isfinite(y).all()) and bool(torch.isfinite(sst_d).all())
    untouched = [s for s in range(7) if s not in slots.tolist()]
    assert torch.equal(sst_d[untouched].cpu(), sst[untouched])


# ---- two mixers side by side ------------------------------------------------------------------------------------------------
def test_parallel_part(rt):
    left, Wl, ls = attention_part(rt, 2, 1, 32, 16, 32, "halves", gate=True, seed=70)
    right, Wr, rs = state_space_part(rt, 4, 12, 16, 2, 4, 3, seed=80)
    T = {"left." + k: v for k, v in Wl.items()}
    T.update({"right." + k: v for k, v in Wr.items()})
    T["left.out"], T["right.out"] = 1.0 + rnd(WIDTH, seed=90, scale=0.2), 1.0 + rnd(WIDTH, seed=91, scale=0.2)
    part, W = bound(rt, "mixer", ("parallel", dict(
        hidden_size=WIDTH, eps=1e-5,
        left=("attention", dict(hidden_size=WIDTH, num_heads=2, num_kv_heads=1, head_dim=32, value_dim=16, query_scale=0.3,
                                position=("rope", {"rotary_dim": 32, "theta": 300.0}), output_gate=True, tensors=("q", "k", "v", "o", "g"))),
        right=("state_space", dict(hidden_size=WIDTH, num_heads=4, head_dim=12, state_size=16, groups=2, conv_taps=4, norm_groups=3,
                                   norm_eps=1e-5)))), {k: v.float() for k, v in T.items()})
    assert set(part.state_specs()) == {"right.ssm", "right.conv"} and part.cache_spec() == left.cache_spec()
    seqs, wide = {}, {}
    for i, n in LENS.items():
        seqs[i], wide[i] = acts(rt, rnd(n, WIDTH, seed=29 + i))
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        want, _ = plain.parallel(wide[i], W, "", {"left": ls, "right": rs}, 1e-5)
        assert rel_l2(got[i][0], want) < PART_TOL[rt.dtype] * 3, i


@pytest.mark.parametrize("m,d", [(1, 64), (9, 200), (300, 96), (5, 3000)])
def test_pair_norm_mean_and_gate_kernels(rt, m, d):
    a, b = rnd(m, d, seed=1).to(rt.dtype), rnd(m, d, seed=2, scale=30.0).to(rt.dtype)
    ga, gb = 1 + rnd(d, seed=3, scale=0.1), 1 + rnd(d, seed=4, scale=0.1)
    got = rt.ops.pair_norm_mean(a.to(DEV), b.to(DEV), ga.to(DEV), gb.to(DEV), 1e-5)
    want = 0.5 * (plain.unit_rms(a.double(), 1e-5) * ga + plain.unit_rms(b.double(), 1e-5) * gb)
    assert got.dtype == torch.float32 and rel_l2(got, want) < 2e-6
    g = rnd(m, d + 40, seed=5).to(rt.dtype)
    x = a.to(DEV).clone()
    rt.ops.mul_sigmoid(x, g.to(DEV)[:, 20:d + 20])       # the gates are a view of wider rows
    assert rel_l2(x, a.double() * torch.sigmoid(g.double()[:, 20:d + 20])) < (1e-6 if rt.dtype == torch.float32 else 4e-3)


# ---- feed-forward -------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("m,d,f,e,top,shared", [(1, 64, 40, 5, 3, 24), (9, 50, 18, 2, 2, None), (150, 96, 70, 16, 2, 56), (70, 128, 33, 9, 1, 16),
                                                (650, 136, 200, 3, 2, None), (700, 128, 192, 3, 3, 64), (5, 64, 1024, 4, 1, 128)])
def test_sigmoid_routed_experts(rt, m, d, f, e, top, shared):
    """Scores are sigmoids, the chosen experts' scores scale their inputs, a shared expert is added."""
    sh = None if shared is None else ("gated_mlp", dict(hidden_size=d, intermediate_size=shared, activation="silu",
                                                        tensors=("gate", "up", "down"), prefix="shared."))
    T = {"router": rnd(e, d, seed=20, scale=0.4)}
    for k in range(e):
        for name, shape in (("gate", (f, d)), ("up", (f, d)), ("down", (d, f))):
            T[f"e{k}.{name}"] = rnd(*shape, seed=21 + 3 * k + len(name), scale=0.3)
    if shared is not None:
        T.update({"shared.gate": rnd(shared, d, seed=5, scale=0.3), "shared.up": rnd(shared, d, seed=6, scale=0.3),
                  "shared.down": rnd(d, shared, seed=7, scale=0.3)})
    part, W = bound(rt, "feed_forward", ("routed_experts", dict(
        hidden_size=d, intermediate_size=f, n_experts=e, top=top, limit=None, gate_alpha=1.0, up_shift=0.0, score="sigmoid",
        weight_input=True, shared=sh)), T)
    x_dev, x = acts(rt, rnd(m, d, seed=19))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    mlp = {"router": {"experts": e, "top": top}}
    if shared is not None:
        mlp["shared"] = {"ff": shared}
    logits = rt.ops.linear(x_dev, part.w_router, torch.float32)
    chosen, weights = rt.ops.route_top(logits, top, score="sigmoid")
    s = torch.sigmoid(x @ W["router"].T)
    order = torch.argsort(-s, dim=-1, stable=True)[:, :top]
    assert torch.equal(chosen.cpu().long(), order) and rel_l2(weights, torch.gather(s, 1, order)) < 1e-5
    got = rt.ops.rows(part.forward(ctx, x_dev), torch.float32)
    assert got.dtype == torch.float32
    assert rel_l2(got, plain.mixture(x, W, "", mlp)) < PART_TOL[rt.dtype]


def test_a_score_scales_the_input_not_the_output():
    """With inputs large enough for SiLU to bend, expert(s h) and s expert(h) differ by tenths: the kernels give the first."""
    rt = Runtime(dtype="float32", device=DEV)
    d, f, e = 64, 48, 4
    T = {"router": rnd(e, d, seed=1, scale=0.02)}
    for k in range(e):
        T.update({f"e{k}.gate": rnd(f, d, seed=2 + k, scale=0.4), f"e{k}.up": rnd(f, d, seed=12 + k, scale=0.4),
                  f"e{k}.down": rnd(d, f, seed=22 + k, scale=0.4)})
    part, W = bound(rt, "feed_forward", ("routed_experts", dict(hidden_size=d, intermediate_size=f, n_experts=e, top=2, limit=None,
                                                                gate_alpha=1.0, up_shift=0.0, score="sigmoid", weight_input=True)), T)
    x_dev, x = acts(rt, rnd(20, d, seed=3))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    want = plain.mixture(x, W, "", {"router": {"experts": e, "top": 2}})
    assert rel_l2(part.forward(ctx, x_dev), want) < 4e-6
    s = torch.sigmoid(x @ W["router"].T)
    order = torch.argsort(-s, dim=-1, stable=True)[:, :2]
    outside = torch.zeros_like(x)
    for r in range(x.shape[0]):
        for k in order[r].tolist():
            outside[r] += s[r, k] * plain.gated_ff(x[r:r + 1], W, f"e{k}.", plain.silu)[0]
    assert rel_l2(outside, want) > 0.1


@pytest.mark.parametrize("m,d,f", [(1, 64, 40), (8, 256, 320), (70, 128, 100), (300, 96, 512)])
def test_relu_gated_layer(rt, m, d, f):
    part, W = bound(rt, "feed_forward", ("gated_mlp", dict(hidden_size=d, intermediate_size=f, activation="relu", tensors=("gate", "up", "down"))),
                    {"gate": rnd(f, d, seed=1, scale=0.2), "up": rnd(f, d, seed=2, scale=0.2), "down": rnd(d, f, seed=3, scale=0.2)})
    x_dev, x = acts(rt, rnd(m, d, seed=4))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    got = rt.ops.rows(part.forward(ctx, x_dev), rt.dtype)
    assert rel_l2(got, plain.gated_ff(x, W, "", torch.relu)) < PART_TOL[rt.dtype]


# ---- the model ------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module", params=[("P", "float32"), ("P", "bfloat16"), ("Q", "float32"), ("Q", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def m(request, tmp_path_factory):
    from .gpu_engine import load_gpu_model
    which, dtype = request.param
    folder = lt.make_folder(tmp_path_factory.mktemp("l"), which)
    model, cfg = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL[dtype]


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    from .gpu_engine import load_gpu_model
    folder = lt.make_folder(tmp_path_factory.mktemp("l"), "S")
    model, cfg = load_gpu_model(folder, "float32")
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, 4e-3


def test_whole_and_token_by_token(m):
    mc.whole_and_token_by_token(m)


def test_prompt_then_long_decode(m):
    mc.prompt_then_decode(m, n=400, tail=300)


def test_portions(m):
    mc.portions(m)


def test_unequal_batches_and_reuse(m):
    mc.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    mc.slot_after_a_longer_sequence(m)


def test_sharp_scores_far_keys(sharp):
    mc.sharp_scores_far_keys(sharp, n=420, page=64)
    mc.sharp_scores_far_keys(sharp, n=150, page=16)


def test_layers_one_by_one(m):
    """The residual stream after every layer, as the debug dump's stage `layer_out` shows it."""
    model, cfg, pcfg, pw, tol = m
    toks = random_tokens(21, cfg.vocab_size, 81)
    want = []
    plain.forward(pcfg, pw, toks, want)
    seen = []
    cache = model.new_cache(max_tokens=64, page_size=16)
    s = cache.acquire()
    counts, starts, rows, tok = model.prepare(cache, [s], toks, counts=[len(toks)], want=[len(toks) - 1])    # reserves the pages first
    ctx = StepContext(model.rt, cache, [s], counts, starts, rows)
    ctx.dump = lambda stage, x: seen.append(x.clone()) if stage == "layer_out" else None
    model.run(ctx, tok)
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        mc.rows_close(a, b, tol, i)


@pytest.mark.parametrize("which,dtype", [("P", "float32"), ("Q", "float32"), ("P", "bfloat16")])
def test_greedy_generation_through_the_entry_point(which, dtype, tmp_path):
    from trapetum_amd import load_model
    folder = lt.make_folder(tmp_path, which)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_tokens(n, pcfg["vocab"], 90 + n) for n in (7, 1, 19, 4, 33)]
    engine = load_model(folder, dtype=dtype, max_tokens_in_cache=64 * 3, max_batch=3)      # graphs on; slots are used again
    got = engine.generate(prompts, max_tokens=12, stop_ids=())
    assert [len(g) for g in got] == [12] * len(prompts)
    if dtype == "float32":
        assert got == [plain.greedy_generate(pcfg, pw, p, 12) for p in prompts]
    again = engine.generate(prompts[::-1], max_tokens=12, stop_ids=())       # replayed graphs, other slots
    assert again == got[::-1]
    assert engine.cache.live_slots() == []


# ---- the programs a user runs ------------------------------------------------------------------------------------------------
def test_command_line_and_trace_runner(tmp_path):
    """`python -m trapetum_amd random | run | generate` and bin/trace_run on a Lutovik folder: the model class comes from
    config.json, the ids and logits are the plain implementation's."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    from . import trace_schedules as ts
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

    def run(cmd, **kw):
        p = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=300, **kw)
        assert p.returncode == 0, p.stderr[-2000:]
        return p.stdout
    cfg, init = lt.CONFIGS["P"]
    config = tmp_path / "config.json"
    config.write_text(json.dumps(cfg))
    folder = tmp_path / "model"
    module = [sys.executable, "-m", "trapetum_amd"]
    assert "wrote" in run(module + ["random", "--config", str(config), "--out", str(folder), "--seed", str(init["seed"]),
                                    "--sigma", str(init["sigma"]), "--sigma-norm", str(init["sigma_norm"])])
    pcfg, pw = plain.read_folder(str(folder))
    prompts = [random_tokens(n, pcfg["vocab"], 95 + n) for n in (6, 13)]
    want = [plain.greedy_generate(pcfg, pw, p, 7) for p in prompts]
    out = run(module + ["run", str(folder), "--prompt-ids", ",".join(map(str, prompts[0])), "--max-tokens", "7", "--dtype", "float32"])
    assert out.strip() == f"continuation ids: {want[0]}"
    ids = tmp_path / "ids.txt"
    ids.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    out = run(module + ["generate", str(folder), "--prompts-file", str(ids), "--max-tokens", "7", "--dtype", "float32"])
    assert [[int(t) for t in line.split()] for line in out.strip().splitlines()] == want
    # the trace runner: requests whole, in unequal batches, and with their last tokens one by one
    requests = {f"r{i}": random_tokens(n, pcfg["vocab"], 20 + i) for i, n in enumerate([40, 3, 21])}
    ref = {rid: plain.forward(pcfg, pw, t) for rid, t in requests.items()}
    for name, steps in (("whole", ts.whole(requests)), ("tail", ts.last_one_by_one(requests, 12)), ("batches", ts.batches(requests, 3))):
        out_dir = tmp_path / name
        stdout = run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out_dir),
                      "--max-tokens", str(ts.held_tokens(steps))], input="".join(json.dumps(s) + "\n" for s in steps))
        assert [l for l in stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = {s["step"]: np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4") for s in steps if any(e["want"] for e in s["entries"])}
        got = ts.collect(steps, outputs, pcfg["vocab"])
        for rid in requests:
            assert rel_l2(torch.from_numpy(got[rid]), ref[rid]) < 2e-5, (name, rid)
