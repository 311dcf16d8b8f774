"""Vogunex through the engine's host logic on the CPU (the product's model, cache, step function and generation loop
over the plain torch kernels of tests/ref_ops.py), against the plain implementation in tests/plain."""
import random

import pytest
import torch

from trapetum_amd.config import ConfigError, VogunexConfig
from trapetum_amd.engine.generate import generate
from trapetum_amd.weights import write_model_folder

from . import model_cases as mc
from . import vogunex_tiny as vt
from .cpu_engine import load_cpu_model
from .plain import vogunex_plain as plain
from .tiny import random_tokens

TOL = 2e-5


@pytest.fixture(scope="module", params=["P", "Q"])
def m(request, tmp_path_factory):
    folder = vt.make_folder(tmp_path_factory.mktemp("v"), request.param)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    folder = vt.make_folder(tmp_path_factory.mktemp("v"), "S")
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, 4e-3


def test_layout_cache_and_states(m):
    model, cfg, pcfg, _, _ = m
    names = set(model.tensor_layout())
    assert {"embed", "head", "final.norm"} <= names
    cache = model.new_cache(max_tokens=64, page_size=16)
    states, blocks = model.entry_state_specs(), model.entry_token_specs()
    for i, layer in enumerate(pcfg["layers"]):
        mx = layer["mixer"]
        if "weights_of" in layer:
            assert not any(n.startswith(f"l{i}.") for n in names)           # a run on another layer's weights has no tensors ...
        else:
            assert {f"l{i}.norm1", f"l{i}.shift", f"l{i}.mix.o"} <= names and (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
        assert states[i]["token_shift"].shape == (cfg.hidden_size,)         # ... and a cache and states of its own
        if layer["type"] == "attention":
            row = max(mx["dim"], mx["vdim"])
            spec = cache.site(i).spec
            assert list(spec.tensors) == [("k", (mx["kv_heads"], row)), ("v", (mx["kv_heads"], row))] and spec.window == mx["mask"]["size"]
            if mx["mask"].get("pool"):
                assert blocks[i]["mixer.blocks"].every == mx["mask"]["pool"] and blocks[i]["mixer.blocks"].window is None
                assert states[i]["mixer.block_sums"].shape == (2, mx["kv_heads"] * row)
            else:
                assert not blocks[i]
        elif layer["type"] == "latent_attention":
            spec = cache.site(i).spec
            assert list(spec.tensors) == [("latent", (1, mx["rot_dim"] + mx["kv_rank"]))] and spec.window == mx["mask"]["size"]
        else:
            assert cache.site(i) is None
            assert states[i]["mixer.ssm"].shape == (mx["heads"], mx["state"], mx["vdim"])
    sites = [cache.site(i) for i, l in enumerate(pcfg["layers"]) if l["type"] != "mamba2"]
    assert len({(s.group_index, s.index_in_group) for s in sites}) == len(sites)


def test_config_errors():
    for path, value, match in [(("layers", 0, "mixer", "kv_heads"), 3, "no multiple"),
                               (("layers", 0, "mixer", "rot", "dims"), 18, "at most"),
                               (("layers", 0, "mixer", "mask", "size"), 0, "positive"),
                               (("layers", 0, "mixer", "mask", "pool"), 0, "positive"),
                               (("layers", 1, "mixer", "q_rank"), 0, "positive"),
                               (("layers", 1, "mlp", "router", "top"), 6, "between"),
                               (("layers", 1, "mlp", "shared", "limit"), -1.0, "positive"),
                               (("layers", 2, "weights_of"), 2, "no other layer"),
                               (("layers", 2, "weights_of"), 4, "no other layer"),
                               (("layers", 2, "weights_of"), 1, "must be equal"),
                               (("layers", 0, "type"), "other", "mixers are")]:
        bad = vt.config_p()
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            VogunexConfig.from_dict(bad)
    for key, where in (("norm", None), ("q_rank", ("layers", 1, "mixer")), ("limit", ("layers", 1, "mlp", "expert")),
                       ("size", ("layers", 0, "mixer", "mask"))):
        d = vt.config_p()
        at = d
        for k in where or ():
            at = at[k]
        del at[key]
        with pytest.raises(ConfigError, match=key):
            VogunexConfig.from_dict(d)


def test_a_page_per_block_of_tokens():
    """A pool that keeps one row per P tokens takes a page when a sequence's first block is whole, and a further page
    every page-size blocks; its pages come back with the slot."""
    from trapetum_amd.cache.store import ModelCache, TokenSpec
    spec = TokenSpec.of(None, every=5, k=(1, 4))
    cache = ModelCache([None], 1000, 1000, 4, 16, torch.float32, "cpu", entry_tokens=[{"b": spec}])
    pages = cache.token_groups[cache.entry_site(0, "b").group_index].pages
    s = cache.acquire()
    for n, want in ((4, 0), (1, 1), (79, 1), (1, 2), (80, 3)):          # lengths 4, 5, 84, 85, 165: 0, 1, 16, 17, 33 blocks
        cache.grow(s, n)
        assert len(pages.lists.get(s, ())) == want, (cache.length(s), want)
    free = pages.pool.available()
    cache.release(s)
    assert pages.pool.available() == free + 3
    with pytest.raises(Exception, match="window"):
        TokenSpec.of(8, every=2, k=(1, 4))


def test_a_bias_rides_in_the_matrix_only_where_it_is_exact():
    """The second product of the biased feed-forward carries its bias as a column of its matrix when the bias has the
    matrix's width, and adds it in a launch of its own when it does not; both give the same rows."""
    import types

    from trapetum_amd.registry import build_part

    from .cpu_engine import ref_ops_namespace
    g = torch.Generator().manual_seed(3)
    d, f = 24, 40
    T = {"up": torch.randn(f, d, generator=g).to(torch.bfloat16), "up.b": torch.randn(f, generator=g).to(torch.bfloat16),
         "down": torch.randn(d, f, generator=g).to(torch.bfloat16), "down.b": torch.randn(d, generator=g).to(torch.bfloat16)}
    x = torch.randn(7, d, generator=g)
    rt = types.SimpleNamespace(matrix=lambda t: t.float(), ops=ref_ops_namespace())
    ctx = types.SimpleNamespace(ops=rt.ops, dtype=torch.float32)
    outs = []
    for exact in (True, False):
        t = dict(T)
        if not exact:
            t["down.b"] = T["down.b"].float() + 1e-3            # no bfloat16 number
        part = build_part("feed_forward", ("biased_mlp", dict(hidden_size=d, intermediate_size=f)))
        part.bind(t, rt)
        assert part.folded == exact
        a = x @ t["up"].float().T + t["up.b"].float()
        want = (0.5 * a * (1 + torch.erf(a / 2 ** 0.5))) @ t["down"].float().T + t["down.b"].float()
        assert torch.allclose(rt.ops.rows(part.forward(ctx, x), torch.float32), want, atol=1e-4)


def test_whole_and_token_by_token(m):
    mc.whole_and_token_by_token(m, n=45)


def test_prompt_then_decode(m):
    mc.prompt_then_decode(m, n=60, tail=35)


def test_portions(m):
    mc.portions(m)


def test_unequal_batches_and_reuse(m):
    mc.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    mc.slot_after_a_longer_sequence(m)


def test_sharp_scores_at_the_edges(sharp):
    mc.sharp_scores_far_keys(sharp, n=90)


def test_greedy_generation_through_the_loop(m):
    model, cfg, pcfg, pw, _ = m
    prompts = [random_tokens(n, cfg.vocab_size, 70 + n) for n in (7, 1, 19, 4)]
    want = [plain.greedy_generate(pcfg, pw, p, 6) for p in prompts]
    cache = model.new_cache(max_tokens=64 * 2, page_size=64)             # room for two sequences at a time: slots are used again
    assert generate(model, cache, prompts, max_tokens=6, stop_ids=()) == want
    assert cache.live_slots() == [] and cache.tokens_held() == 0


@pytest.mark.parametrize("case", range(6))
def test_random_configuration(case, tmp_path):
    """A configuration drawn at random: a prompt whole, then in two portions and single tokens."""
    rng = random.Random(900 + case)
    cfg = vt.draw(rng)
    folder = str(tmp_path)
    write_model_folder(VogunexConfig.from_dict(cfg), folder, seed=case, sigma=0.1, sigma_norm=0.2)
    model, c = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    assert pcfg == cfg
    toks = random_tokens(37, c.vocab_size, case)
    ref = plain.forward(pcfg, pw, toks)
    cache = model.new_cache(max_tokens=128, page_size=16)
    s = cache.acquire()
    got = [model.step(cache, [s], toks[:20], counts=[20], want=list(range(20))),
           model.step(cache, [s], toks[20:31], counts=[11], want=list(range(11)))]
    got += [model.step(cache, [s], [t]) for t in toks[31:]]
    mc.rows_close(torch.cat(got), ref, 5e-5, cfg)
