"""Besulix on the GPU: each mechanism's kernels alone against the plain functions of tests/plain, then the model through
the step function, the cache and the generation entry point, in float32 and bfloat16."""
import random

import pytest
import torch

from trapetum_amd.config import BesulixConfig
from trapetum_amd.engine.batch import StepContext
from trapetum_amd.weights import write_model_folder

from . import besulix_tiny as bt
from . import model_cases as mc
from .plain import besulix_plain as plain
from .test_lutovik_gpu import LENS, PART_TOL, STEPS, WIDTH, acts, bound, rnd, rt, run_mixers  # noqa: F401  (rt is the fixture)
from .tiny import random_tokens, rel_l2

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": mc.Rounded(4e-2)}
EPS = 1e-5


def sequences(rt, seed, scale=1.0, lens=LENS):
    seqs, wide = {}, {}
    for i, n in lens.items():
        seqs[i], wide[i] = acts(rt, rnd(n, WIDTH, seed=seed + i) * scale)
    return seqs, wide


# ---- the chunked attention with biases, temperatures, sinks and rotated values ---------------------------------------------
def chunk_attention_ref(H, G, dim, vdim, rot, chunk, scale, base=300.0):
    position = ("rope", {"rotary_dim": rot, "theta": base}) if rot else ("none", {})
    ref = ("attention", dict(hidden_size=WIDTH, num_heads=H, num_kv_heads=G, head_dim=dim, value_dim=vdim, query_scale=scale,
                             position=position, tensors=("q", "k", "v", "o"), bias_suffix=".b", chunk=chunk,
                             head_temperature="temp", sink="sink", value_rotation=base))
    sizes = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": rot}, "mask": {"size": chunk}}
    return ref, sizes


def chunk_attention_tensors(H, G, dim, vdim, seed=0, sink=1.0):
    return {"q": rnd(H * dim, WIDTH, seed=seed + 1, scale=0.25), "q.b": rnd(H * dim, seed=seed + 2, scale=0.3),
            "k": rnd(G * dim, WIDTH, seed=seed + 3, scale=0.25), "k.b": rnd(G * dim, seed=seed + 4, scale=0.3),
            "v": rnd(G * vdim, WIDTH, seed=seed + 5, scale=0.3), "v.b": rnd(G * vdim, seed=seed + 6, scale=0.3),
            "temp": 1.0 + rnd(H, seed=seed + 7, scale=0.4), "sink": rnd(H, seed=seed + 8, scale=sink),
            "o": rnd(WIDTH, H * vdim, seed=seed + 9, scale=0.2)}


@pytest.mark.parametrize("H,G,dim,vdim,rot,chunk", [
    (4, 2, 16, 24, 8, 8), (3, 3, 24, 8, 24, 20), (2, 1, 32, 32, 16, 16), (1, 1, 12, 12, 0, 1000), (6, 2, 64, 48, 32, 64),
    (8, 2, 128, 64, 64, 100), (2, 2, 40, 72, 40, 1), (4, 1, 80, 96, 20, 33), (2, 1, 48, 128, 48, 17)])
def test_chunk_attention_part(rt, H, G, dim, vdim, rot, chunk):
    ref, sizes = chunk_attention_ref(H, G, dim, vdim, rot, chunk, 0.3)
    part, W = bound(rt, "mixer", ref, chunk_attention_tensors(H, G, dim, vdim))
    seqs, wide = sequences(rt, 9)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    tol = PART_TOL[rt.dtype] * (3 if rt.dtype == torch.float32 else 1.5)
    for i in seqs:
        assert rel_l2(got[i][0], plain.chunk_sink_attention(wide[i], W, "", sizes)) < tol, i


def test_a_sink_takes_its_share(rt):
    """Sinks of +6 and -6 on two heads: the first head's outputs shrink to a fraction, the second's hardly change.  A sink
    that is left out, scaled or multiplied by the temperature shows whole."""
    H, G, dim, vdim = 2, 1, 16, 16
    ref, sizes = chunk_attention_ref(H, G, dim, vdim, 8, 32, 0.3)
    T = chunk_attention_tensors(H, G, dim, vdim, seed=20)
    T["sink"] = torch.tensor([6.0, -6.0])
    T["temp"] = torch.tensor([1.5, 0.5])
    part, W = bound(rt, "mixer", ref, T)
    seqs, wide = sequences(rt, 29)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        want = plain.chunk_sink_attention(wide[i], W, "", sizes)
        assert rel_l2(got[i][0], want) < PART_TOL[rt.dtype] * 3, i
        for other in (torch.tensor([-30.0, -6.0]), torch.tensor([6.0 * 1.5, -6.0])):
            assert rel_l2(plain.chunk_sink_attention(wide[i], dict(W, sink=other.double()), "", sizes), want) > 0.05


@pytest.mark.parametrize("chunk,page,first", [(20, 16, 19), (20, 16, 20), (20, 16, 21), (64, 64, 63), (64, 64, 64), (64, 64, 65),
                                              (100, 64, 100), (16, 16, 17), (5, 16, 4)])
def test_keys_at_a_chunks_edge(rt, chunk, page, first):
    """The last key of every chunk and the first key of the next are made to stand out (a large component that only they
    and the queries have, outside the rotation).  A query then reads its own chunk's first key, alone or beside its own
    key if that is marked too, and never the key one place before the chunk, in a prompt, in a portion that starts
    next to the edge and token by token across the next edge.  An edge one place off shows whole."""
    H, G, dim, vdim, rot = 4, 2, 16, 24, 8

    def mark(T):                                         # a head's last element: keys read column 5 of the input, queries column 7
        for name, heads, col in (("k", G, 5), ("q", H, 7)):
            w = T[name].view(heads, dim, WIDTH)
            w[:, dim - 1, :] = 0.0
            w[:, dim - 1, col] = 1.0
            T[name + ".b"].view(heads, dim)[:, dim - 1] = 0.0
    ref, sizes = chunk_attention_ref(H, G, dim, vdim, rot, chunk, 1.0)
    T = chunk_attention_tensors(H, G, dim, vdim, seed=7, sink=0.3)
    T["temp"] = torch.ones(H)
    mark(T)
    part, W = bound(rt, "mixer", ref, T)
    n = 2 * chunk + 4
    marked = [p for p in (chunk - 1, chunk, 2 * chunk - 1, 2 * chunk) if p >= 0]
    x = rnd(n, WIDTH, seed=3) * 0.3
    x[:, 5] = 0.0
    x[marked, 5] = 30.0
    x[:, 7] = 3.0                                        # every query meets a marked key with a score of 90
    x_dev, xw = acts(rt, x)
    want = plain.chunk_sink_attention(xw, W, "", sizes)
    tail = min(8, n - first - 1)
    steps = [{0: first}, {0: n - first - tail}] + [{0: 1}] * tail
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps, page=page)[0][0]
    assert rel_l2(got, want) < (2e-5 if rt.dtype == torch.float32 else 2e-2)
    # the plain outputs do rest on those keys: with a chunk one position longer or shorter they are something else
    for other in (chunk + 1, max(1, chunk - 1)):
        if other != chunk:
            assert rel_l2(plain.chunk_sink_attention(xw, W, "", dict(sizes, mask={"size": other})), want) > 0.2


# ---- the time-mixing recurrence ---------------------------------------------------------------------------------------------
def time_mix_tensors(heads, dim, rank, seed=0, w0=None):
    inner = heads * dim
    T = {"mu." + s: rnd(WIDTH, seed=seed + i, scale=0.3) + 0.5 for i, s in enumerate("rkvgw")}
    T.update({s: rnd(inner, WIDTH, seed=seed + 10 + i, scale=0.25) for i, s in enumerate("rkvg")})
    T.update({"w1": rnd(rank, WIDTH, seed=seed + 20, scale=0.3), "w2": rnd(inner, rank, seed=seed + 21, scale=0.5),
              "w0": rnd(inner, seed=seed + 22, scale=1.0) - 1.0 if w0 is None else torch.full((inner,), float(w0)),
              "u": rnd(heads, dim, seed=seed + 23, scale=0.5), "norm": 1.0 + rnd(inner, seed=seed + 24, scale=0.2),
              "o": rnd(WIDTH, inner, seed=seed + 25, scale=0.2)})
    return T


@pytest.mark.parametrize("heads,dim,rank", [(3, 20, 5), (1, 72, 8), (2, 32, 16), (6, 64, 4), (1, 4, 1), (2, 130, 7), (4, 16, 3)])
def test_time_mix_part(rt, heads, dim, rank):
    part, W = bound(rt, "mixer", ("time_mix", dict(hidden_size=WIDTH, num_heads=heads, head_dim=dim, norm_eps=EPS, decay_rank=rank)),
                    time_mix_tensors(heads, dim, rank))
    seqs, wide = sequences(rt, 19)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    for i in seqs:
        assert rel_l2(got[i][0], plain.time_mix(wide[i], W, "", {"heads": heads, "dim": dim}, EPS)) < PART_TOL[rt.dtype] * 3, i


@pytest.mark.parametrize("cut", ["whole", "pieces", "one by one"])
def test_time_mix_keeps_its_first_tokens(rt, cut):
    """Decays of exp(-exp(-7)): what the first tokens wrote is still most of every output hundreds of tokens later, through
    a prompt cut into pieces and through single tokens.  A state lost or started anew on the way would show whole."""
    heads, dim, rank = 3, 24, 4
    T = time_mix_tensors(heads, dim, rank, seed=60, w0=-7.0)
    T["w2"] = torch.zeros_like(T["w2"])
    part, W = bound(rt, "mixer", ("time_mix", dict(hidden_size=WIDTH, num_heads=heads, head_dim=dim, norm_eps=EPS, decay_rank=rank)), T)
    n = 333
    x = rnd(n, WIDTH, seed=61) * 0.2
    x[:6] *= 20.0
    x_dev, xw = acts(rt, x)
    steps = {"whole": [{0: n}], "pieces": [{0: 130}, {0: 2}, {0: 64}, {0: 137}], "one by one": [{0: 300}] + [{0: 1}] * 33}[cut]
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps)[0][0]
    sizes = {"heads": heads, "dim": dim}
    want = plain.time_mix(xw, W, "", sizes, EPS)
    assert rel_l2(got[200:], want[200:]) < PART_TOL[rt.dtype] * 5
    x2 = xw.clone()
    x2[:6] = 0.0
    assert rel_l2(plain.time_mix(x2, W, "", sizes, EPS)[200:], want[200:]) > 0.3


SCAN_LENS = (1, 7, 33, 64, 97, 130, 300)
SCAN_SLOTS = (5, 0, 3, 9, 1, 7, 2)


def scan_geometry(rt):
    cu = torch.tensor([0] + list(torch.tensor(SCAN_LENS).cumsum(0)), dtype=torch.int32)
    return cu, torch.tensor(SCAN_SLOTS, dtype=torch.int32), sum(SCAN_LENS)


@pytest.mark.parametrize("chunk", [0, None, 4, 32, 50])
@pytest.mark.parametrize("heads,dim", [(3, 20), (2, 64), (1, 130)])
def test_time_mix_scan_in_chunks(rt, heads, dim, chunk):
    """Sequences of unequal lengths from states that are not zero, in chunks of several sizes (a last chunk of one row, a
    sequence shorter than a chunk, one exactly a chunk long): the outputs and the states left behind are those of the
    rows taken one after the other.  The decays range from almost none to almost all."""
    from . import ref_ops
    cu, slots, M = scan_geometry(rt)
    inner = heads * dim
    r, k, v = (rnd(M, inner, seed=60 + i, scale=0.5) for i in range(3))
    rate = rnd(M, inner, seed=63, scale=2.0) - 2.0
    w0, bonus = rnd(inner, seed=64, scale=0.5), rnd(heads, dim, seed=65, scale=0.5)
    state = rnd(10, heads, dim, dim, seed=66, scale=0.3)
    rd, kd, vd = (acts(rt, t)[0] for t in (r, k, v))
    want_state = state.double()
    want = ref_ops.time_mix_scan(rd.cpu(), kd.cpu(), vd.cpu(), rate, w0, bonus, want_state, slots, cu, max(SCAN_LENS), heads, dim)
    got_state = state.to(rt.device)
    got = rt.ops.time_mix_scan(rd, kd, vd, rate.to(rt.device), w0.to(rt.device), bonus.to(rt.device), got_state, slots.to(rt.device),
                               cu.to(rt.device), max(SCAN_LENS), heads, dim, chunk=chunk)
    for i in range(len(SCAN_LENS)):
        assert rel_l2(got[cu[i]:cu[i + 1]], want[cu[i]:cu[i + 1]]) < 5e-6, i
        assert rel_l2(got_state[SCAN_SLOTS[i]], want_state[SCAN_SLOTS[i]].float()) < 5e-6, i
    assert torch.equal(got_state[[4, 6, 8]].cpu(), state[[4, 6, 8]])          # slots of no sequence are left alone


# ---- the matrix memory --------------------------------------------------------------------------------------------------------
def matrix_memory_tensors(heads, dim, vdim, seed=0, i_bias=0.0, f_bias=1.0, gate_scale=0.3):
    return {"q": rnd(heads * dim, WIDTH, seed=seed + 1, scale=0.25), "k": rnd(heads * dim, WIDTH, seed=seed + 2, scale=0.25),
            "v": rnd(heads * vdim, WIDTH, seed=seed + 3, scale=0.3), "g": rnd(heads * vdim, WIDTH, seed=seed + 4, scale=0.3),
            "o": rnd(WIDTH, heads * vdim, seed=seed + 5, scale=0.2), "norm": 1.0 + rnd(heads * vdim, seed=seed + 6, scale=0.2),
            "i": rnd(heads, WIDTH, seed=seed + 7, scale=gate_scale), "i.b": rnd(heads, seed=seed + 8, scale=0.5) + i_bias,
            "f": rnd(heads, WIDTH, seed=seed + 9, scale=gate_scale), "f.b": rnd(heads, seed=seed + 10, scale=0.5) + f_bias}


def matrix_memory_ref(heads, dim, vdim, cap):
    return ("matrix_memory", dict(hidden_size=WIDTH, num_heads=heads, key_dim=dim, value_dim=vdim, gate_cap=cap, norm_eps=EPS))


@pytest.mark.parametrize("heads,dim,vdim,cap,i_bias,gate_scale", [
    (2, 24, 40, 6.0, 0.0, 0.3), (3, 72, 70, 9.0, 0.0, 0.3), (1, 16, 16, 15.0, 0.0, 0.3), (6, 48, 64, 12.0, 0.0, 0.3),
    (2, 130, 200, 5.0, 0.0, 0.3), (4, 4, 6, 12.0, 0.0, 0.3),
    (2, 32, 32, 4.0, 0.0, 3.0),          # gate sums far beyond the cap: the tanh decides
    (2, 32, 32, 12.0, -9.0, 0.3),        # input gates far below zero: the running maximum stays where it starts for a while
    (2, 32, 32, 12.0, 7.0, 0.3)])        # and far above: it follows the input gates
def test_matrix_memory_part(rt, heads, dim, vdim, cap, i_bias, gate_scale):
    part, W = bound(rt, "mixer", matrix_memory_ref(heads, dim, vdim, cap),
                    matrix_memory_tensors(heads, dim, vdim, i_bias=i_bias, gate_scale=gate_scale))
    seqs, wide = sequences(rt, 39)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    sizes = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}
    for i in seqs:
        # bfloat16: the denominator max(|n . q|, e^(-m)) turns small now and then, and the rounding of q and k with it
        assert rel_l2(got[i][0], plain.matrix_memory(wide[i], W, "", sizes, EPS)) < PART_TOL[rt.dtype] * (3 if rt.dtype == torch.float32 else 6), i


@pytest.mark.parametrize("chunk", [0, None, 4, 32, 50])
@pytest.mark.parametrize("heads,dk,dv,i_bias", [(3, 20, 36, 0.0), (2, 64, 128, 6.0), (1, 130, 70, -6.0), (2, 32, 200, 0.0)])
def test_matrix_memory_scan_in_chunks(rt, heads, dk, dv, i_bias, chunk):
    """As for the time-mixing scan; the running maximum starts from states above and below what the chunks reach."""
    from . import ref_ops
    cu, slots, M = scan_geometry(rt)
    q, k = rnd(M, heads * dk, seed=70, scale=0.5), rnd(M, heads * dk, seed=71, scale=0.5)
    v = rnd(M, heads * dv, seed=72, scale=0.5)
    gates = torch.cat([rnd(M, heads, seed=73, scale=3.0) + i_bias, rnd(M, heads, seed=74, scale=3.0) + 1.0], dim=1).contiguous()
    S, n = rnd(10, heads, dk, dv, seed=75, scale=0.3), rnd(10, heads, dk, seed=76, scale=0.3)
    mx = rnd(10, heads, seed=77, scale=4.0)
    qd, kd, vd = (acts(rt, t)[0] for t in (q, k, v))
    want_states = [S.double(), n.double(), mx.double()]
    want = ref_ops.matrix_memory_scan(qd.cpu(), kd.cpu(), vd.cpu(), gates, 8.0, dk ** -0.5, *want_states, slots, cu, max(SCAN_LENS), heads, dk, dv)
    got_states = [t.to(rt.device) for t in (S, n, mx)]
    got = rt.ops.matrix_memory_scan(qd, kd, vd, gates.to(rt.device), 8.0, dk ** -0.5, *got_states, slots.to(rt.device), cu.to(rt.device),
                                    max(SCAN_LENS), heads, dk, dv, chunk=chunk)
    for i in range(len(SCAN_LENS)):
        # (max(|n . q|, e^(-m)) is a small difference of large terms now and then: float32 against float64, in any cut)
        assert rel_l2(got[cu[i]:cu[i + 1]], want[cu[i]:cu[i + 1]]) < 6e-5, i
        # a state is kept in units of e^(its maximum): compare what the pair stands for
        for g, w in zip(got_states[:2], want_states[:2]):
            lift = lambda t, m: t[SCAN_SLOTS[i]].cpu().double() * torch.exp(m[SCAN_SLOTS[i]].cpu().double()).reshape(heads, *([1] * (t.dim() - 2)))
            assert rel_l2(lift(g, got_states[2]), lift(w, want_states[2])) < 1e-5, i
        assert torch.allclose(got_states[2][SCAN_SLOTS[i]].cpu(), want_states[2][SCAN_SLOTS[i]].float(), atol=1e-5, rtol=1e-6), i
    for g, w in zip(got_states, (S, n, mx)):
        assert torch.equal(g[[4, 6, 8]].cpu(), w[[4, 6, 8]])


@pytest.mark.parametrize("cut", ["whole", "pieces", "one by one"])
def test_matrix_memory_keeps_its_first_tokens(rt, cut):
    """Forget gates of sigmoid(8) and small input gates after the first tokens: the memory is what the first tokens wrote,
    hundreds of tokens later."""
    heads, dim, vdim, cap = 2, 24, 40, 12.0
    T = matrix_memory_tensors(heads, dim, vdim, seed=70, f_bias=8.0, gate_scale=0.0)
    T["f.b"] = torch.full((heads,), 8.0)
    T["i"] = torch.zeros(heads, WIDTH)
    T["i"][:, 11] = 1.0                                  # the input gate's logarithm is the input's column 11
    T["i.b"] = torch.zeros(heads)
    part, W = bound(rt, "mixer", matrix_memory_ref(heads, dim, vdim, cap), T)
    n = 333
    x = rnd(n, WIDTH, seed=71) * 0.3
    x[:, 11] = -4.0
    x[:6, 11] = 3.0
    x_dev, xw = acts(rt, x)
    steps = {"whole": [{0: n}], "pieces": [{0: 130}, {0: 2}, {0: 64}, {0: 137}], "one by one": [{0: 300}] + [{0: 1}] * 33}[cut]
    got = run_mixers(rt, [(part, 0)], {0: x_dev}, steps)[0][0]
    sizes = {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}
    want = plain.matrix_memory(xw, W, "", sizes, EPS)
    assert rel_l2(got[200:], want[200:]) < PART_TOL[rt.dtype] * 5
    x2 = xw.clone()
    x2[:6, 11] = -4.0
    x2[:6, :11] = 0.0
    x2[:6, 12:] = 0.0
    assert rel_l2(plain.matrix_memory(x2, W, "", sizes, EPS)[200:], want[200:]) > 0.3


# ---- the two mixers side by side, the feed-forward, the embedding ------------------------------------------------------------
def test_weighted_sum_of_two_mixers(rt):
    H, G, dim, vdim, heads, d, rank = 4, 2, 16, 24, 3, 20, 5
    left, sizes = chunk_attention_ref(H, G, dim, vdim, 8, 24, 0.3)
    right = ("time_mix", dict(hidden_size=WIDTH, num_heads=heads, head_dim=d, norm_eps=EPS, decay_rank=rank))
    T = {"left." + k: v for k, v in chunk_attention_tensors(H, G, dim, vdim, seed=80).items()}
    T.update({"right." + k: v for k, v in time_mix_tensors(heads, d, rank, seed=90).items()})
    part, W = bound(rt, "mixer", ("parallel", dict(hidden_size=WIDTH, left=left, right=right, combine="weighted_sum", weights=(0.7, 1.2))), T)
    seqs, wide = sequences(rt, 49)
    got = run_mixers(rt, [(part, 0)], seqs, STEPS)
    m = {"left": sizes, "right": {"heads": heads, "dim": d}, "left_scale": 0.7, "right_scale": 1.2}
    for i in seqs:
        assert rel_l2(got[i][0], plain.parallel_mixer(wide[i], W, "", m, EPS)) < PART_TOL[rt.dtype] * 3, i


@pytest.mark.parametrize("m,d,f,limit", [(1, 64, 40, 0.5), (8, 256, 320, 1.0), (70, 128, 100, 7.0), (300, 96, 512, 0.2), (33, 50, 30, 1.0)])
def test_clamped_feed_forward(rt, m, d, f, limit):
    part, W = bound(rt, "feed_forward", ("gated_mlp", dict(hidden_size=d, intermediate_size=f, activation="quick_gelu",
                                                          tensors=("gate", "up", "down"), limit=limit, up_shift=1.0)),
                    {"gate": rnd(f, d, seed=1, scale=0.2), "up": rnd(f, d, seed=2, scale=0.2), "down": rnd(d, f, seed=3, scale=0.2)})
    x_dev, x = acts(rt, rnd(m, d, seed=4))
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    got = rt.ops.rows(part.forward(ctx, x_dev), rt.dtype)
    want = plain.clamped_ff(x, W, "", {"limit": limit})
    assert rel_l2(got, want) < PART_TOL[rt.dtype]
    assert rel_l2(plain.clamped_ff(x, W, "", {"limit": 100.0}), want) > (1e-3 if limit >= 7 else 0.05)     # the limit does cut


def test_embedding_with_a_norm(rt):
    V, D = 50, 72
    part, W = bound(rt, "embedding", ("scaled_embedding", dict(vocab_size=V, hidden_size=D, scale=1.0, tensor="", norm=(
        "rms_norm", {"size": D, "eps": 1e-3, "tensor": ".norm", "init": "gain"}))), {"": rnd(V, D, seed=1, scale=0.05), ".norm": 1.0 + rnd(D, seed=2, scale=0.3)})
    toks = [3, 49, 0, 3, 17]
    ctx = type("C", (), {"ops": rt.ops, "dtype": rt.dtype})()
    got = part.forward(ctx, torch.tensor(toks, dtype=torch.int32, device="cuda:0"))
    assert got.dtype == torch.float32
    assert rel_l2(got, plain.unit_rms(W[""][toks], 1e-3) * W[".norm"]) < 2e-6


# ---- the model ------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module", params=[("P", "float32"), ("P", "bfloat16"), ("Q", "float32"), ("Q", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def m(request, tmp_path_factory):
    from .gpu_engine import load_gpu_model
    which, dtype = request.param
    folder = bt.make_folder(tmp_path_factory.mktemp("b"), which)
    model, cfg = load_gpu_model(folder, dtype)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL[dtype]


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    from .gpu_engine import load_gpu_model
    folder = bt.make_folder(tmp_path_factory.mktemp("b"), "S")
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


def test_sharp_scores_at_chunk_edges(sharp):
    mc.sharp_scores_far_keys(sharp, n=420, page=64)
    mc.sharp_scores_far_keys(sharp, n=150, page=16)


def test_an_early_token_decides(tmp_path):
    from .gpu_engine import load_gpu_model
    folder = bt.make_long_memory_folder(tmp_path)
    model, cfg = load_gpu_model(folder, "float32")
    pcfg, pw = plain.read_folder(folder)
    bt.early_token_decides(model, cfg, pcfg, pw, 2e-3)


def test_layers_one_by_one(m):
    """The residual stream after every layer, as the debug dump's stage `layer_out` shows it."""
    model, cfg, pcfg, pw, tol = m
    toks = random_tokens(21, cfg.vocab_size, 81)
    want = []
    plain.forward(pcfg, pw, toks, want)
    seen = []
    cache = model.new_cache(max_tokens=64, page_size=16)
    s = cache.acquire()
    counts, starts, rows, tok = model.prepare(cache, [s], toks, counts=[len(toks)], want=[len(toks) - 1])
    ctx = StepContext(model.rt, cache, [s], counts, starts, rows)
    ctx.dump = lambda stage, x: seen.append(x.clone()) if stage == "layer_out" else None
    model.run(ctx, tok)
    assert len(seen) == len(want)
    for i, (a, b) in enumerate(zip(seen, want)):
        mc.rows_close(a, b, tol, i)


@pytest.mark.parametrize("which,dtype", [("P", "float32"), ("Q", "float32"), ("P", "bfloat16")])
def test_greedy_generation_through_the_entry_point(which, dtype, tmp_path):
    from trapetum_amd import load_model
    folder = bt.make_folder(tmp_path, which)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_tokens(n, pcfg["vocab"], 90 + n) for n in (7, 1, 19, 4, 33)]
    engine = load_model(folder, dtype=dtype, max_tokens_in_cache=64 * 3, max_batch=3)      # graphs on; slots are used again
    got = engine.generate(prompts, max_tokens=12, stop_ids=())
    assert [len(g) for g in got] == [12] * len(prompts)
    if dtype == "float32":
        assert got == [plain.greedy_generate(pcfg, pw, p, 12) for p in prompts]
    again = engine.generate(prompts[::-1], max_tokens=12, stop_ids=())       # replayed graphs, other slots, other batches
    if dtype == "float32":
        assert again == got[::-1]
    else:                                                # beside other requests a product's sums are added in another order: a close
        assert [len(g) for g in again] == [12] * len(prompts)                # call between two tokens may turn
        assert sum(a[:4] == b[:4] for a, b in zip(again, got[::-1])) >= len(prompts) - 1
    assert engine.cache.live_slots() == []


@pytest.mark.parametrize("case", range(10))
def test_random_configuration(case, tmp_path):
    """A configuration drawn at random, in float32 and bfloat16: unequal prompts in one step, a portion each, then six
    tokens each."""
    from .besulix_random import draw
    from .gpu_engine import load_gpu_model
    rng = random.Random(3000 + case)
    cfg = draw(rng)
    folder = str(tmp_path)
    write_model_folder(BesulixConfig.from_dict(cfg), folder, seed=case, sigma=rng.choice([0.05, 0.1]), sigma_norm=0.2)
    pcfg, pw = plain.read_folder(folder)
    lens = [rng.randint(1, 150) for _ in range(rng.randint(1, 4))]
    more = [rng.randint(2, 40) for _ in lens]
    seqs = [random_tokens(n + k + 6, cfg["vocab"], 100 * case + i) for i, (n, k) in enumerate(zip(lens, more))]
    refs = [plain.forward(pcfg, pw, s) for s in seqs]
    for dtype, tol in (("float32", 5e-5), ("bfloat16", 8e-2)):      # float32: up to six layers and no cap on the logits
        model, _ = load_gpu_model(folder, dtype)
        cache = model.new_cache(max_tokens=2048)
        slots = [cache.acquire() for _ in lens]
        got = [[r] for r in model.step(cache, slots, [t for s, n in zip(seqs, lens) for t in s[:n]], counts=lens)]
        out = model.step(cache, slots, [t for s, n, k in zip(seqs, lens, more) for t in s[n:n + k]], counts=more)
        for i in range(len(lens)):
            got[i].append(out[i])
        for step in range(6):
            out = model.step(cache, slots, [s[n + k + step] for s, n, k in zip(seqs, lens, more)])
            for i in range(len(lens)):
                got[i].append(out[i])
        errs = []
        for i, (n, k) in enumerate(zip(lens, more)):
            places = [n - 1, n + k - 1] + [n + k + j for j in range(6)]
            errs += [rel_l2(g, refs[i][p]) for g, p in zip(got[i], places)]
        errs.sort()
        if dtype == "float32":
            assert errs[-1] < tol, (cfg, lens, dtype, errs[-1])
        else:
            assert errs[len(errs) // 2] < tol, (cfg, lens, dtype, errs)


# ---- the programs a user runs ------------------------------------------------------------------------------------------------
def test_command_line_and_trace_runner(tmp_path):
    """`python -m trapetum_amd random | run | generate` and bin/trace_run on a Besulix folder: the model class comes from
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
    cfg, init = bt.CONFIGS["P"]
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
