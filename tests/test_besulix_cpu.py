"""Besulix through the engine's host logic on the CPU (the product's model, cache, step function and generation loop
over the plain torch kernels of tests/ref_ops.py), against the plain implementation in tests/plain."""
import pytest
import torch

from trapetum_amd.config import BesulixConfig, ConfigError
from trapetum_amd.engine.generate import generate

from . import besulix_tiny as bt
from . import model_cases as mc
from .cpu_engine import load_cpu_model
from .plain import besulix_plain as plain
from .tiny import random_tokens

TOL = 2e-5


@pytest.fixture(scope="module", params=["P", "Q"])
def m(request, tmp_path_factory):
    folder = bt.make_folder(tmp_path_factory.mktemp("b"), request.param)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, TOL


@pytest.fixture(scope="module")
def sharp(tmp_path_factory):
    folder = bt.make_folder(tmp_path_factory.mktemp("b"), "S")
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    return model, cfg, pcfg, pw, 4e-3


def test_layout_cache_and_states(m):
    model, cfg, pcfg, _, _ = m
    names = set(model.tensor_layout())
    assert {"embed", "embed.norm", "head", "final.norm"} <= names
    cache = model.new_cache(max_tokens=64, page_size=16)
    states = model.entry_state_specs()
    for i, layer in enumerate(pcfg["layers"]):
        mx = layer["mixer"]
        assert f"l{i}.norm1" in names and (f"l{i}.norm2" in names) == (layer["mlp"] is not None)
        if layer["type"] == "mlstm":
            assert {f"l{i}.mix.i.b", f"l{i}.mix.f", f"l{i}.mix.norm", f"l{i}.mix.g"} <= names and cache.site(i) is None
            want = {"mixer.memory": (mx["heads"], mx["dim"], mx["vdim"]), "mixer.normalizer": (mx["heads"], mx["dim"]),
                    "mixer.maximum": (mx["heads"],)}
        else:
            a, r = mx["left"], mx["right"]
            assert {f"l{i}.mix.left.q.b", f"l{i}.mix.left.temp", f"l{i}.mix.left.sink", f"l{i}.mix.right.mu.w", f"l{i}.mix.right.w2",
                    f"l{i}.mix.right.u"} <= names
            want = {"mixer.right.memory": (r["heads"], r["dim"], r["dim"]), "mixer.right.shift": (cfg.hidden_size,)}
            row = max(a["dim"], a["vdim"])               # keys and values share rows of the larger size
            spec = cache.site(i).spec
            assert list(spec.tensors) == [("k", (a["kv_heads"], row)), ("v", (a["kv_heads"], row))]
            assert spec.window == a["mask"]["size"]      # nothing before a chunk's first position is ever read again
        assert {k: v.shape for k, v in states[i].items()} == want
        assert all(v.dtype == "float32" for v in states[i].values())


def test_config_errors():
    for path, value, match in [(("layers", 0, "mixer", "left", "kv_heads"), 3, "no multiple"),
                               (("layers", 0, "mixer", "left", "rot", "dims"), 18, "exceeds dim"),
                               (("layers", 0, "mixer", "left", "vdim"), 23, "even"),
                               (("layers", 0, "mixer", "left", "mask", "size"), 0, "positive"),
                               (("layers", 1, "mixer", "gate_cap"), 0.0, "positive"),
                               (("layers", 0, "mlp", "kind"), "moe", "dense"),
                               (("layers", 0, "mlp", "limit"), -1.0, "positive"),
                               (("layers", 0, "type"), "other", "mlstm and parallel")]:
        bad = bt.config_p()
        at = bad
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = value
        with pytest.raises(ConfigError, match=match):
            BesulixConfig.from_dict(bad)
    for key, where in (("norm", None), ("right_scale", ("layers", 0, "mixer")), ("limit", ("layers", 0, "mlp"))):
        d = bt.config_p()
        at = d
        for k in where or ():
            at = at[k]
        del at[key]
        with pytest.raises(ConfigError, match=key):
            BesulixConfig.from_dict(d)


def test_the_checkpoint_gives_the_decay_rank(tmp_path):
    """No configuration key names the channels between the decay's two products: a folder's shapes decide."""
    from safetensors.torch import load_file, save_file
    folder = bt.make_folder(tmp_path, "Q")
    path = f"{folder}/model.safetensors"
    t = load_file(path)
    g = torch.Generator().manual_seed(5)
    for rank in (3, 11):
        t["l1.mix.right.w1"] = (torch.randn(rank, 50, generator=g) * 0.2).to(torch.bfloat16)
        t["l1.mix.right.w2"] = (torch.randn(16, rank, generator=g) * 0.2).to(torch.bfloat16)
        save_file(t, path)
        model, cfg = load_cpu_model(folder)
        pcfg, pw = plain.read_folder(folder)
        toks = random_tokens(9, cfg.vocab_size, rank)
        cache = model.new_cache(max_tokens=64, page_size=16)
        got = model.step(cache, [cache.acquire()], toks, counts=[9], want=list(range(9)))
        mc.rows_close(got, plain.forward(pcfg, pw, toks), TOL, rank)


def test_whole_and_token_by_token(m):
    mc.whole_and_token_by_token(m, n=40)


def test_prompt_then_decode(m):
    mc.prompt_then_decode(m, n=50, tail=30)


def test_portions(m):
    mc.portions(m)


def test_unequal_batches_and_reuse(m):
    mc.unequal_batches_and_reuse(m)


def test_slot_after_a_longer_sequence(m):
    mc.slot_after_a_longer_sequence(m)


def test_sharp_scores_at_chunk_edges(sharp):
    mc.sharp_scores_far_keys(sharp, n=100)


def test_an_early_token_decides(tmp_path):
    """With decays and forget gates close to one, the logits at the end of a sequence change when an early token
    changes, by as much as the plain implementation says: what the recurrent states took from it is carried through a
    prompt and through decoded tokens.  A state lost on the way would leave no difference at all."""
    folder = bt.make_long_memory_folder(tmp_path)
    model, cfg = load_cpu_model(folder)
    pcfg, pw = plain.read_folder(folder)
    bt.early_token_decides(model, cfg, pcfg, pw, 2e-3)


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
    import random

    from trapetum_amd.weights import write_model_folder

    from .besulix_random import draw
    rng = random.Random(700 + case)
    cfg = draw(rng)
    folder = str(tmp_path)
    write_model_folder(BesulixConfig.from_dict(cfg), folder, seed=case, sigma=0.1, sigma_norm=0.2)
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
