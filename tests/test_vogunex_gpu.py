"""Vogunex on the GPU: each mechanism's kernels alone against the plain functions of tests/plain, then the model through
the step function, the cache and the generation entry point, in float32 and bfloat16."""
import random

import pytest
import torch

from trapetum_amd.config import VogunexConfig
from trapetum_amd.engine.batch import StepContext
from trapetum_amd.engine.runtime import Runtime
from trapetum_amd.weights import write_model_folder

from . import model_cases as mc
from . import vogunex_tiny as vt
from .plain import vogunex_plain as plain
from .test_lutovik_gpu import DEV, LENS, PART_TOL, STEPS, WIDTH, acts, bound, rnd, rt, run_mixers  # noqa: F401  (rt is the fixture)
from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": mc.Rounded(4e-2)}
EPS = 1e-5


def sequences(rt, seed, scale=1.0, lens=LENS):
    seqs, wide = {}, {}
    for i, n in lens.items():
        seqs[i], wide[i] = acts(rt, rnd(n, WIDTH, seed=seed + i) * scale)
    return seqs, wide


def tolerance(rt):
    return PART_TOL[rt.dtype] * (3 if rt.dtype == torch.float32 else 1.5)


# ---- attention over a window and pooled blocks, unit norms, talking heads ---------------------------------------------------
def pooled_attention(rt, H, G, dim, vdim, rot, size, pool, cap, scale=0.3, base=300.0, seed=0, edit=None, talk=None):
    position = ("rope", {"rotary_dim": rot, "theta": base}) if rot else ("none", {})
    ref = ("attention", dict(hidden_size=WIDTH, num_heads=H, num_kv_heads=G, head_dim=dim, value_dim=vdim, query_scale=scale,
                             softcap=cap, window=size, position=position, tensors=("q", "k", "v", "o"), bias_suffix=".b",
                             unit_norm_eps=EPS, pool=pool, talk="talk"))
    T = {"q": rnd(H * dim, WIDTH, seed=seed + 1, scale=0.25), "q.b": rnd(H * dim, seed=seed + 2, scale=0.3),
         "k": rnd(G * dim, WIDTH, seed=seed + 3, scale=0.25), "k.b": rnd(G * dim, seed=seed + 4, scale=0.3),
         "v": rnd(G * vdim, WIDTH, seed=seed + 5, scale=0.3), "v.b": rnd(G * vdim, seed=seed + 6, scale=0.3),
         "talk": torch.eye(H) + rnd(H, H, seed=seed + 7, scale=0.4) if talk is None else talk,
         "o": rnd(WIDTH, H * vdim, seed=seed + 9, scale=0.2)}
    if edit is not None:
        edit(T)
    part, W = bound(rt, "mixer", ref, T)
    mask = {"size": size} if pool is None else {"size": size, "pool": pool}
    sizes = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": scale, "softcap": cap, "rot": {"base": base, "dims": rot}, "mask": mask}
    return part, W, sizes


@pytest.mark.parametrize("H,G,dim,vdim,rot,size,pool,cap", [
    (4, 2, 16, 24, 8, 11, 3, 30.0), (3, 3, 24, 8, 24, 20, 5, 12.0), (2, 1, 32, 32, 16, 16, 16, None), (1, 1, 12, 12, 0, 1, 1, 5.0),
    (6, 2, 64, 80, 16, 40, 6, 18.0), (8, 2, 128, 64, 64, 33, 4, 50.0), (2, 2, 40, 72, 40, 7, None, 9.0), (4, 1, 80, 96, 20, 64, 2, None),
    (6, 3, 48, 130, 48, 1000, 7, 15.0), (3, 1, 16, 16, 4, 2, 30, 10.0)])
def test_pooled_attention_part(rt, H, G, dim, vdim, rot, size, pool, cap):
    """Prompts, single tokens and portions down to two rows, two sequences side by side."""
    part, W, sizes = pooled_attention(rt, H, G, dim, vdim, rot, size, pool, cap)
    seqs, wide = sequences(rt, 9)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        assert rel_l2(got[i][0], plain.attention(wide[i], W, "", sizes, EPS)) < tolerance(rt), i


@pytest.mark.parametrize("H,G,dim,vdim,size,pool", [(8, 4, 256, 256, 300, 8), (4, 2, 128, 64, 129, 16), (2, 1, 64, 32, 1000, None), (6, 3, 32, 96, 64, 1)])
def test_matrix_core_kernel_over_many_chunks(H, G, dim, vdim, size, pool):
    """Sequences long enough for every wave of a block to take several chunks of keys, pooled blocks by the dozen: the
    matrix-core kernel against the plain implementation, and against the plain kernel on the same rows."""
    rt = Runtime(dtype="bfloat16", device=DEV)
    part, W, sizes = pooled_attention(rt, H, G, dim, vdim, 32, size, pool, 25.0, scale=0.5)
    seqs, wide = sequences(rt, 59, lens={0: 700, 1: 180})
    steps = [{0: 500, 1: 100}, {0: 1, 1: 1}, {0: 150, 1: 2}] + [{0: 1, 1: 1}] * 49 + [{1: 28}]
    got = run_mixers(rt, [(part, 0)], seqs, steps, page=64)
    rt.ops.force_plain_attention = True
    try:
        slow = run_mixers(rt, [(part, 0)], seqs, steps, page=64)
    finally:
        rt.ops.force_plain_attention = False
    for i in seqs:
        assert rel_l2(got[i][0], plain.attention(wide[i], W, "", sizes, EPS)) < tolerance(rt), i
        assert rel_l2(got[i][0], slow[i][0]) < 4e-3, i


def rows_differ(a, b):
    return float(((a - b).norm(dim=1) / b.norm(dim=1)).max())


@pytest.mark.parametrize("page,first", [(16, 24), (16, 25), (16, 26), (16, 27), (16, 28), (16, 32), (16, 33), (64, 64), (64, 6)])
def test_one_key_at_the_windows_edge_and_in_its_block(rt, page, first):
    """One early key is made to stand out for every later query (a large component that only it and the queries have, in
    an element outside the rotation).  While the window holds it the outputs are its value; then nothing of it is seen
    until its block is whole and lies before the window; then a third of it, in the block's mean.  The step's border is
    put just before, on and just after both edges, in a prompt, a portion and single tokens."""
    H, G, dim, vdim, rot, size, pool, at = 4, 2, 16, 24, 8, 20, 4, 5

    def mark(T):                                         # a head's last element: keys read column 5 of the input, queries column 7
        for name, heads, col in (("k", G, 5), ("q", H, 7)):
            w = T[name].view(heads, dim, WIDTH)
            w[:, dim - 1, :] = 0.0
            w[:, dim - 1, col] = 1.0
            T[name + ".b"].view(heads, dim)[:, dim - 1] = 0.0
    part, W, sizes = pooled_attention(rt, H, G, dim, vdim, rot, size, pool, None, scale=2.5, seed=7, edit=mark)
    n = max(first, 34) + 2 * page + 9
    x = rnd(n, WIDTH, seed=3) * 0.3
    x[:, 5] = 0.0
    x[at, 5] = 30.0                                      # the marked key
    x[:, 7] = 3.0                                        # every query meets it with a large score
    x_dev, xw = acts(rt, x)
    want = plain.attention(xw, W, "", sizes, EPS)
    steps = [{0: first}, {0: 2 * page + 1}] + [{0: 1}] * (n - first - 2 * page - 1)
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps, page=page)[0][0]
    assert rel_l2(got, want) < (2e-5 if rt.dtype == torch.float32 else 2e-2)
    assert rows_differ(got.double().cpu(), want) < (1e-4 if rt.dtype == torch.float32 else 6e-2)
    # and the plain outputs do rest on the edges: a window one longer or shorter, or blocks seen one position earlier
    # or later, give something else in the rows at the edge
    for other in (dict(size=size + 1, pool=pool), dict(size=size - 1, pool=pool)):
        assert rows_differ(plain.attention(xw, W, "", dict(sizes, mask=other), EPS), want) > 0.3, other
    x2 = xw.clone()
    x2[at, 5] = 0.0
    assert rows_differ(plain.attention(x2, W, "", sizes, EPS)[at + size + pool:], want[at + size + pool:]) > 0.1       # its block still tells


def test_heads_that_talk_take_other_heads_weights(rt):
    """A mixing matrix that gives head 0 the weights of head 3 (another kv head's) and nothing of its own: head 0 then
    weighs its own kv head's values by head 3's softmax.  Applied to the wrong values, or mixed before the softmax, it shows."""
    H, G = 4, 2
    talk = torch.eye(H)
    talk[0] = torch.tensor([0.0, 0.0, 0.0, 1.0])
    talk[2] = torch.tensor([0.5, -0.5, 1.0, 0.25])
    part, W, sizes = pooled_attention(rt, H, G, 16, 24, 8, 13, 3, 30.0, scale=1.5, talk=talk)
    seqs, wide = sequences(rt, 19)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        want = plain.attention(wide[i], W, "", sizes, EPS)
        assert rel_l2(got[i][0], want) < tolerance(rt), i
        assert rel_l2(plain.attention(wide[i], dict(W, talk=torch.eye(H, dtype=torch.float64)), "", sizes, EPS), want) > 0.1


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("counts,block,KV,row", [([5], 3, 2, 16), ([1, 1, 1], 1, 1, 8), ([70, 1, 200, 33], 7, 3, 24), ([2, 64], 64, 2, 40)])
def test_block_means_however_the_rows_are_cut(dt, counts, block, KV, row):
    """The pooled rows after two steps equal the means over the positions of both, and the unfinished block's sums wait."""
    ops = Runtime(dtype="float32", device=DEV).ops
    page, n = 16, len(counts)
    first = [c // 2 for c in counts]
    k = rnd(2 * sum(counts), KV * row, seed=1).to(dt).to(DEV)
    v = rnd(2 * sum(counts), KV * row, seed=2).to(dt).to(DEV)
    sums = torch.zeros((n + 1, 2, KV * row), dtype=torch.float32, device=DEV)
    kb = torch.zeros((8 * n, KV, page, row), dtype=dt, device=DEV)
    vb = torch.zeros_like(kb)
    table = torch.arange(8 * n, dtype=torch.int32, device=DEV).reshape(n, 8)
    slots = torch.arange(n, dtype=torch.int32, device=DEV)
    at, held, rows_of = 0, [0] * n, [[] for _ in range(n)]
    for part in (first, [c - f for c, f in zip(counts, first)], counts):          # three steps: a half, the rest, as much again
        live = [i for i in range(n) if part[i] > 0]
        if not live:
            continue
        cu, take = [0], []
        for i in live:
            take += list(range(at, at + part[i]))
            rows_of[i] += list(range(at, at + part[i]))
            at += part[i]
            held[i] += part[i]
            cu.append(cu[-1] + part[i])
        idx = torch.tensor(take, dtype=torch.long, device=DEV)
        ops.pool_write(k[idx], v[idx], KV, row, block, torch.tensor(cu, dtype=torch.int32, device=DEV), max(part),
                       torch.tensor([held[i] for i in live], dtype=torch.int32, device=DEV), slots[live].contiguous(), sums,
                       table[live].contiguous(), kb, vb)
    for i in range(n):
        mine_k, mine_v = k[rows_of[i]].double().cpu(), v[rows_of[i]].double().cpu()
        for b in range(held[i] // block):
            pg = int(table[i, b // page])
            for pool_rows, src in ((kb, mine_k), (vb, mine_v)):
                want = src[b * block:(b + 1) * block].mean(0).reshape(KV, row)
                assert rel_l2(pool_rows[pg, :, b % page, :], want) < (1e-6 if dt == torch.float32 else 6e-3), (i, b)
        rest = held[i] % block
        if rest:
            assert rel_l2(sums[i, 0], mine_k[-rest:].sum(0)) < 1e-6


# ---- attention through a latent: a latent for the queries, neighbouring pairs, a window, a gate per head -----------------------
def latent_part(rt, H, dim, rot_dim, vdim, rank, q_rank, dims, size, scale=0.3, base=200.0, seed=0):
    position = ("rope", {"rotary_dim": dims, "theta": base, "pairing": "neighbours"}) if dims else ("none", {})
    ref = ("latent_attention", dict(hidden_size=WIDTH, num_heads=H, nope_dim=dim, rope_dim=rot_dim, value_dim=vdim, latent_rank=rank,
                                    scale=scale, latent_eps=EPS, position=position, query_rank=q_rank, window=size, output_gate="g",
                                    precise_weights=True))
    T = {"dq": rnd(q_rank, WIDTH, seed=seed + 1, scale=0.3), "dq.norm": 1.0 + rnd(q_rank, seed=seed + 2, scale=0.2),
         "uq": rnd(H * (dim + rot_dim), q_rank, seed=seed + 3, scale=0.3), "dkv": rnd(rank + rot_dim, WIDTH, seed=seed + 4, scale=0.3),
         "dkv.norm": 1.0 + rnd(rank, seed=seed + 5, scale=0.2), "uk": rnd(H * dim, rank, seed=seed + 6, scale=0.3),
         "uv": rnd(H * vdim, rank, seed=seed + 7, scale=0.3), "g": rnd(H, WIDTH, seed=seed + 8, scale=0.4),
         "o": rnd(WIDTH, H * vdim, seed=seed + 9, scale=0.2)}
    part, W = bound(rt, "mixer", ref, T)
    sizes = {"heads": H, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank, "scale": scale,
             "rot": {"base": base, "dims": dims}, "mask": {"size": size}}
    return part, W, sizes


@pytest.mark.parametrize("H,dim,rot_dim,vdim,rank,q_rank,dims,size", [
    (3, 16, 8, 12, 24, 20, 8, 13), (2, 8, 16, 16, 16, 12, 12, 18), (1, 10, 4, 10, 6, 6, 0, 1000), (6, 48, 16, 64, 112, 72, 16, 40),
    (5, 24, 2, 20, 14, 5, 2, 1), (4, 32, 16, 32, 48, 24, 8, 64), (16, 64, 32, 64, 96, 48, 32, 70), (2, 8, 8, 8, 8, 8, 8, 2)])
def test_latent_attention_part(rt, H, dim, rot_dim, vdim, rank, q_rank, dims, size):
    part, W, sizes = latent_part(rt, H, dim, rot_dim, vdim, rank, q_rank, dims, size)
    seqs, wide = sequences(rt, 29)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    # in bfloat16 a row passes two more roundings than an attention without the queries' latent (the latent and the queries)
    tol = tolerance(rt) if rt.dtype == torch.float32 else 2 * PART_TOL[rt.dtype]
    for i in seqs:
        assert rel_l2(got[i][0], plain.latent_attention(wide[i], W, "", sizes, EPS)) < tol, i


@pytest.mark.parametrize("page,first", [(16, 23), (16, 24), (16, 25), (16, 32), (64, 64), (64, 65)])
def test_latent_attention_at_its_windows_edge(rt, page, first):
    """Scores scaled up until a softmax picks single keys; the window's last position is at 4 + 20 for the query after it."""
    part, W, sizes = latent_part(rt, 3, 16, 8, 12, 32, 20, 8, 20, scale=6.0, seed=50)
    n = first + 2 * page + 9
    x_dev, xw = acts(rt, rnd(n, WIDTH, seed=5))
    want = plain.latent_attention(xw, W, "", sizes, EPS)
    steps = [{0: first}, {0: 2 * page + 1}] + [{0: 1}] * 8
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps, page=page)[0][0]
    assert rel_l2(got, want) < (2e-5 if rt.dtype == torch.float32 else 3e-2)
    for other in (19, 21):
        assert rel_l2(plain.latent_attention(xw, W, "", dict(sizes, mask={"size": other}), EPS), want) > 0.05


# ---- the token shift, the biased feed-forward, the router with a bias and the gated shared expert ---------------------------------
@pytest.mark.parametrize("counts,d", [([5], 64), ([1, 1, 1], 50), ([70, 1, 33], 200)])
def test_token_shift_rows_and_state(rt, counts, d):
    ops = rt.ops
    n = len(counts)
    w = rnd(1, d, seed=1, scale=0.5).to(DEV)
    state = torch.zeros((n + 1, d), dtype=torch.float32, device=DEV)
    xs = [rnd(2 * c, d, seed=10 + i) for i, c in enumerate(counts)]
    outs = [[] for _ in counts]
    for step in range(2):
        x = torch.cat([xs[i][step * c:(step + 1) * c] for i, c in enumerate(counts)]).to(DEV)
        cu = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
        row_seq = torch.repeat_interleave(torch.arange(n, dtype=torch.int32), torch.tensor(counts)).to(DEV)
        got = ops.shift_mix(x, w, state, torch.arange(n, dtype=torch.int32, device=DEV), cu, row_seq,
                            one_row_each=all(c == 1 for c in counts), out_dtype=rt.dtype)[0]
        at = 0
        for i, c in enumerate(counts):
            outs[i].append(got[at:at + c])
            at += c
    for i in range(n):
        want = plain.token_shift(xs[i].double(), w[0].double().cpu())
        assert rel_l2(torch.cat(outs[i]), want) < (1e-6 if rt.dtype == torch.float32 else 4e-3), i


@pytest.mark.parametrize("m,d,f", [(1, 64, 40), (8, 256, 320), (70, 128, 100), (300, 96, 512), (9, 50, 33)])
def test_biased_feed_forward(rt, m, d, f):
    T = {"up": rnd(f, d, seed=1, scale=0.2), "up.b": rnd(f, seed=2, scale=0.5), "down": rnd(d, f, seed=3, scale=0.2), "down.b": rnd(d, seed=4, scale=0.5)}
    part, W = bound(rt, "feed_forward", ("biased_mlp", dict(hidden_size=d, intermediate_size=f, activation="gelu_erf", tensors=("up", "down"))), T)
    x_dev, x = acts(rt, rnd(m, d, seed=5))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    got = rt.ops.rows(part.forward(ctx, x_dev), torch.float32)
    assert rel_l2(got, plain.feed_forward(x, W, "", {"kind": "dense", "ff": f})) < PART_TOL[rt.dtype]


@pytest.mark.parametrize("m,d,f,e,top,shared", [(1, 64, 40, 5, 3, 24), (9, 50, 18, 2, 2, None), (150, 96, 70, 16, 2, 56), (70, 128, 33, 9, 1, 16),
                                                (650, 136, 200, 3, 2, None), (5, 64, 96, 1, 1, 128)])
def test_router_with_a_bias_and_gated_shared_expert(rt, m, d, f, e, top, shared):
    sh = None if shared is None else ("gated_mlp", dict(hidden_size=d, intermediate_size=shared, activation="quick_gelu", limit=0.9,
                                                        up_shift=1.0, tensors=("gate", "up", "down"), prefix="shared."))
    T = {"router": rnd(e, d, seed=20, scale=0.4), "router.b": rnd(e, seed=30, scale=1.5)}
    for k in range(e):
        for name, shape in (("gate", (f, d)), ("up", (f, d)), ("down", (d, f))):
            T[f"e{k}.{name}"] = rnd(*shape, seed=21 + 3 * k + len(name), scale=0.3)
    if shared is not None:
        T.update({"shared.gate": rnd(shared, d, seed=5, scale=0.3), "shared.up": rnd(shared, d, seed=6, scale=0.3),
                  "shared.down": rnd(d, shared, seed=7, scale=0.3), "shared.sg": rnd(1, d, seed=8, scale=0.3)})
    part, W = bound(rt, "feed_forward", ("routed_experts", dict(
        hidden_size=d, intermediate_size=f, n_experts=e, top=top, limit=1.4, gate_alpha=1.702, up_shift=1.0, renormalize=True,
        router_bias="router.b", shared=sh, shared_gate=None if sh is None else "shared.sg")), T)
    x_dev, x = acts(rt, rnd(m, d, seed=19))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    mlp = {"kind": "moe", "expert": {"ff": f, "limit": 1.4}, "router": {"experts": e, "top": top}}
    if shared is not None:
        mlp["shared"] = {"ff": shared, "limit": 0.9}
    order, weight = plain.router_choice(x, W, "", top)
    chosen, weights = rt.ops.route_top(rt.ops.linear(x_dev, part.w_router, torch.float32, bias=part.router_bias), top, True)
    assert torch.equal(chosen.cpu().long(), order) and rel_l2(weights, weight) < 1e-5
    got = rt.ops.rows(part.forward(ctx, x_dev), torch.float32)
    assert rel_l2(got, plain.feed_forward(x, W, "", mlp)) < PART_TOL[rt.dtype]
    # the bias does choose: without it other experts win somewhere (where there is a choice)
    if e > top and m > 8:
        assert not torch.equal(plain.router_choice(x, dict(W, **{"router.b": torch.zeros(e, dtype=torch.float64)}), "", top)[0], order)


# ---- the model ------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module", params=[("P", "float32"), ("P", "bfloat16"), ("Q", "float32"), ("Q", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def m(request, tmp_path_factory):
    from .gpu_engine import load_gpu_model
    which, dtype = request.param
    folder = vt.make_folder(tmp_path_factory.mktemp("v"), which)
    model, cfg = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL[dtype]


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    from .gpu_engine import load_gpu_model
    folder = vt.make_folder(tmp_path_factory.mktemp("v"), "S")
    model, cfg = load_gpu_model(folder, "float32")
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, 4e-3


def test_whole_and_token_by_token(m):
    mc.whole_and_token_by_token(m)


def test_prompt_then_long_decode(m):
    mc.prompt_then_decode(m, n=300, tail=220)


def test_portions(m):
    mc.portions(m)


def test_unequal_batches_and_reuse(m):
    mc.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    mc.slot_after_a_longer_sequence(m)


def test_sharp_scores_far_keys(sharp):
    mc.sharp_scores_far_keys(sharp, n=300, page=64)
    mc.sharp_scores_far_keys(sharp, n=150, page=16)


def test_layers_one_by_one(m):
    """The residual stream after every layer run, as the debug dump's stage `layer_out` shows it."""
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


@pytest.mark.parametrize("case", range(8))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_configuration(case, dtype, tmp_path):
    """A configuration drawn at random: a prompt whole, then in two portions and single tokens, beside a second sequence."""
    from .gpu_engine import load_gpu_model
    rng = random.Random(900 + case)
    cfg = vt.draw(rng)
    folder = str(tmp_path)
    write_model_folder(VogunexConfig.from_dict(cfg), folder, seed=case, sigma=0.1, sigma_norm=0.2)
    model, c = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    a, b = random_tokens(90, c.vocab_size, case), random_tokens(31, c.vocab_size, 50 + case)
    ref = torch.cat([plain.forward(pcfg, pw, a), plain.forward(pcfg, pw, b)])
    cache = model.new_cache(max_tokens=512, page_size=16)
    s, t = cache.acquire(), cache.acquire()
    got_a = [model.step(cache, [s], a[:40], counts=[40], want=list(range(40)))]
    both = model.step(cache, [s, t], a[40:71] + b[:12], counts=[31, 12], want=list(range(43)))
    got_a.append(both[:31])
    got_b = [both[31:]]
    for i in range(19):
        one = model.step(cache, [s, t], [a[71 + i], b[12 + i]])
        got_a.append(one[:1])
        got_b.append(one[1:])
    mc.rows_close(torch.cat(got_a + got_b), ref, TOL[dtype] if dtype == "float32" else mc.Rounded(5e-2), cfg)


@pytest.mark.parametrize("which,dtype", [("P", "float32"), ("Q", "float32"), ("P", "bfloat16")])
def test_greedy_generation_through_the_entry_point(which, dtype, tmp_path):
    from trapetum_amd import load_model
    folder = vt.make_folder(tmp_path, which)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_tokens(n, pcfg["vocab"], 90 + n) for n in (7, 1, 19, 4, 33)]
    engine = load_model(folder, dtype=dtype, max_tokens_in_cache=64 * 3, max_batch=3)      # graphs on; slots are used again
    got = engine.generate(prompts, max_tokens=40, stop_ids=())                            # past every window and block of the tiny model
    assert [len(g) for g in got] == [40] * len(prompts)
    if dtype == "float32":
        assert got == [plain.greedy_generate(pcfg, pw, p, 40) for p in prompts]
    again = engine.generate(prompts[::-1], max_tokens=40, stop_ids=())       # replayed graphs, other slots
    assert again == got[::-1]
    assert engine.cache.live_slots() == []


def test_command_line_and_trace_runner(tmp_path):
    """`python -m trapetum_amd random | run` and bin/trace_run on a Vogunex folder: the model class comes from config.json,
    the ids and logits are the plain implementation's."""
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
    cfg, init = vt.CONFIGS["P"]
    config = tmp_path / "config.json"
    config.write_text(json.dumps(cfg))
    folder = tmp_path / "model"
    module = [sys.executable, "-m", "trapetum_amd"]
    assert "wrote" in run(module + ["random", "--config", str(config), "--out", str(folder), "--seed", str(init["seed"]),
                                    "--sigma", str(init["sigma"]), "--sigma-norm", str(init["sigma_norm"])])
    pcfg, pw = plain.read_folder(str(folder))
    prompt = random_tokens(13, pcfg["vocab"], 95)
    out = run(module + ["run", str(folder), "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "7", "--dtype", "float32"])
    assert out.strip() == f"continuation ids: {plain.greedy_generate(pcfg, pw, prompt, 7)}"
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
            mc.rows_close(torch.from_numpy(got[rid]), ref[rid], 2e-5, (name, rid))
