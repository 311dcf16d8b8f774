"""Cases that every design's model must pass on the CPU engine and on the GPU: whole prompts against token by token,
prompt then decoding, portions, unequal batches on reused slots and pages, sharp scores on far keys.  `m` is
(model, cfg, plain config, plain weights, tolerance); the plain implementation is chosen by the design's name."""
import torch

from .plain import besulix_plain, golepel_plain, lutovik_plain, vogunex_plain
from .tiny import random_tokens, rel_l2
from . import trace_schedules as ts

PLAIN = {"Besulix": besulix_plain, "Golepel": golepel_plain, "Lutovik": lutovik_plain, "Vogunex": vogunex_plain}


# ---- cases: `m` is (model, cfg, pcfg, pw, tol) ------------------------------------------------------------------------
def reference(m, toks):
    """The plain implementation's logits for the whole sequence, by the design config.json names."""
    return PLAIN[m[2]["architecture"]].forward(m[2], m[3], toks)


class Rounded(float):
    """A tolerance for an engine that rounds activations to bfloat16.  Rounding turns a router's close call between
    two experts now and then, and the row's logits then differ by tenths although nothing is wrong: the typical row
    is held to the tolerance, and one row in ten may lie beyond four times it."""


def rows_close(got, ref, tol, what=None):
    errs = [rel_l2(got[i], ref[i]) for i in range(ref.shape[0])]
    if isinstance(tol, Rounded):
        ordered = sorted(errs)
        assert ordered[len(errs) // 2] < tol, (what, ordered[len(errs) // 2])
        beyond = [i for i, e in enumerate(errs) if e >= 4 * tol]
        assert len(beyond) <= max(1, len(errs) // 10), (what, beyond)
    else:
        for i, e in enumerate(errs):
            assert e < 3 * tol, (what, i, e)


def whole_and_token_by_token(m, n=70, page=16):
    model, cfg, _, _, tol = m
    toks = random_tokens(n, cfg.vocab_size, 3)
    ref = reference(m, toks)
    cache = model.new_cache(max_tokens=4 * page * (-(-n // page)), page_size=page)
    s = cache.acquire()
    got = model.step(cache, [s], toks, counts=[n], want=list(range(n)))
    rows_close(got, ref, tol, "whole")
    cache.release(s)
    s = cache.acquire()                                 # the same slot and pages again, from the first token on one by one
    got = torch.cat([model.step(cache, [s], [t]) for t in toks])
    rows_close(got, ref, tol, "one by one")
    cache.release(s)


def prompt_then_decode(m, n=90, tail=40, page=16):
    model, cfg, _, _, tol = m
    toks = random_tokens(n, cfg.vocab_size, 4)
    ref = reference(m, toks)
    cache = model.new_cache(max_tokens=2 * n, page_size=page)
    s = cache.acquire()
    rows = [model.step(cache, [s], toks[:n - tail], counts=[n - tail], want=list(range(n - tail)))]
    rows += [model.step(cache, [s], [t]) for t in toks[n - tail:]]
    rows_close(torch.cat(rows), ref, tol)
    cache.release(s)


def portions(m, sizes=((2,), (3, 1, 7), (16, 2), (5, 33))):
    """A prompt cut into portions of several sizes, down to two tokens: a portion sees the cached positions and its own."""
    model, cfg, _, _, tol = m
    requests = {"a": random_tokens(61, cfg.vocab_size, 21), "b": random_tokens(18, cfg.vocab_size, 22)}
    ref = {rid: reference(m, t) for rid, t in requests.items()}
    for cut in sizes:
        steps = ts.chunked(requests, list(cut))
        cache = model.new_cache(max_tokens=ts.held_tokens(steps, 16), page_size=16)
        got = ts.collect(steps, ts.run_on_model(model, cache, steps), cfg.vocab_size)
        rows_close(torch.cat([torch.from_numpy(got[rid]) for rid in requests]), torch.cat([ref[rid] for rid in requests]), tol, cut)


def unequal_batches_and_reuse(m):
    """Batches of unequal requests, one after another on the same few slots and pages, against each request alone."""
    model, cfg, _, _, tol = m
    lens = [37, 1, 12, 50, 3, 2, 19]
    requests = {f"r{i}": random_tokens(n, cfg.vocab_size, 30 + i) for i, n in enumerate(lens)}
    ref = {rid: reference(m, t) for rid, t in requests.items()}
    steps = ts.batches(requests, 3, prefill_fraction=0.6)
    cache = model.new_cache(max_tokens=ts.held_tokens(steps, 16), max_slots=3, page_size=16)
    got = ts.collect(steps, ts.run_on_model(model, cache, steps), cfg.vocab_size)
    rows_close(torch.cat([torch.from_numpy(got[rid]) for rid in requests]), torch.cat([ref[rid] for rid in requests]), tol, "batches")
    assert cache.live_slots() == [] and cache.tokens_held() == 0
    steps = ts.joining(requests, every=2, burst=3)      # requests join a running batch; some go on by a few tokens
    cache = model.new_cache(max_tokens=ts.held_tokens(steps, 16), page_size=16)
    got = ts.collect(steps, ts.run_on_model(model, cache, steps), cfg.vocab_size)
    rows_close(torch.cat([torch.from_numpy(got[rid]) for rid in requests]), torch.cat([ref[rid] for rid in requests]), tol, "joining")


def slot_after_a_longer_sequence(m):
    """A slot that held a long sequence is given back and taken by a short one: neither the pages' old rows nor the
    convolutions' old states may reach the new sequence's first tokens."""
    model, cfg, _, _, tol = m
    cache = model.new_cache(max_tokens=128, max_slots=1, page_size=16)
    long_one = random_tokens(100, cfg.vocab_size, 41)
    s = cache.acquire()
    model.step(cache, [s], long_one, counts=[100], want=[99])
    cache.release(s)
    got, ref, fresh = [], [], []
    for n in (1, 2, 5, 9):
        toks = random_tokens(n, cfg.vocab_size, 42 + n)
        s2 = cache.acquire()
        assert s2 == s
        got += [model.step(cache, [s2], [t]) for t in toks]
        ref.append(reference(m, toks))
        cache.release(s2)
        unused = model.new_cache(max_tokens=128, max_slots=1, page_size=16)
        s3 = unused.acquire()
        fresh += [model.step(unused, [s3], [t]) for t in toks]
    # the same steps in a cache that nothing has used give the same bits: nothing of the slot's past is read
    assert torch.equal(torch.cat(got), torch.cat(fresh))
    if isinstance(tol, Rounded):
        # single tokens after one another hand a router's turned close call on to the few tokens that follow: the typical row is held
        errs = sorted(rel_l2(a, b) for a, b in zip(torch.cat(got), torch.cat(ref)))
        assert errs[len(errs) // 2] < tol, errs
    else:
        rows_close(torch.cat(got), torch.cat(ref), tol)


def sharp_scores_far_keys(m, n=150, page=16):
    """Scores so sharp that a softmax picks single keys, anywhere in a long sequence: whole, decoded and in portions
    that end on, one before and one after a page's border."""
    model, cfg, _, _, tol = m
    toks = random_tokens(n, cfg.vocab_size, 51)
    ref = reference(m, toks)
    for first in (n, page * 4, page * 4 - 1, page * 4 + 1):
        cache = model.new_cache(max_tokens=2 * n, page_size=page)
        s = cache.acquire()
        rows = [model.step(cache, [s], toks[:first], counts=[first], want=list(range(first)))]
        at = first
        if first < n:                                   # a portion of two pages and one row, then one by one
            k = min(2 * page + 1, n - at)
            rows.append(model.step(cache, [s], toks[at:at + k], counts=[k], want=list(range(k))))
            at += k
        rows += [model.step(cache, [s], [t]) for t in toks[at:]]
        rows_close(torch.cat(rows), ref, tol, first)
        cache.release(s)
