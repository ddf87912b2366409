"""Ways of cutting the same requests into steps, and a driver that replays them.

A trace is a list of steps in trace_run's format. ``replay`` drives the
engine's own step function and cache manager in-process and returns the logits
by (request, position); ``plain_logits`` gives the same from the plain
implementation, whole sequences at once.
"""

from __future__ import annotations

import os
import random

import torch


def whole(requests):
    """Each request alone, in one step, logits everywhere."""
    steps = []
    for i, (rid, toks) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def tail_one_by_one(requests, tail=32):
    """Most of the request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for p in range(head, len(toks)):
            steps.append({"entries": [{"id": rid, "tokens": toks[p: p + 1], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return _number(steps)


def portions(requests, sizes=(24, 7, 2, 16, 3, 2, 31, 5)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        p, i = 0, 0
        while p < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - p)
            steps.append({"entries": [{"id": rid, "tokens": toks[p: p + n], "want": list(range(n))}], "end": []})
            p += n
            i += 1
        steps[-1]["end"] = [rid]
    return _number(steps)


def mixed(requests, seed=0, max_live=4, decode_tail=8):
    """Up to ``max_live`` requests at once: portions of some beside single tokens of others.

    Each request is fed in portions of random size until ``decode_tail`` tokens
    remain, which come one per step. A finished request ends at once and the
    next one starts, so its pages are taken by later tokens of other requests.
    """
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            toks = requests[rid]
            p = live[rid]
            left = len(toks) - p
            if rng.random() < 0.2 and len(live) > 1 and entries:
                continue  # a request may sit a step out
            if left <= decode_tail:
                n = 1
            else:
                n = min(left - decode_tail, rng.choice((2, 3, 5, 9, 17, 30)))
            entries.append({"id": rid, "tokens": toks[p: p + n], "want": list(range(n))})
            live[rid] = p + n
            if p + n == len(toks):
                ended.append(rid)
        for rid in ended:
            del live[rid]
        if entries:
            steps.append({"entries": entries, "end": ended})
    return _number(steps)


def random_trace(requests, rng, max_live):
    """Steps drawn at random: requests enter while others run, portions from a few tokens to
    hundreds beside single tokens, requests that sit a step out, tails of 0 to 40 tokens decoded one
    by one, logits wanted at some places only."""
    waiting = list(requests.items())
    live: dict[str, int] = {}
    steps = []
    sizes = rng.choice([(2, 3, 5, 9, 17, 30), (1, 2, 64, 128, 257), (2, 40, 300, 600), (16, 32, 48, 512)])
    tail = {rid: rng.choice((0, 1, 4, 12, 40)) for rid in requests}
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            toks = requests[rid]
            p = live[rid]
            left = len(toks) - p
            if rng.random() < 0.2 and entries:
                continue
            n = 1 if left <= tail[rid] else min(left - tail[rid], rng.choice(sizes))
            want = [i for i in range(n) if n <= 4 or rng.random() < 0.3 or i == n - 1]
            entries.append({"id": rid, "tokens": toks[p: p + n], "want": want})
            live[rid] = p + n
            if p + n == len(toks):
                ended.append(rid)
        for rid in ended:
            del live[rid]
        if entries:
            steps.append({"entries": entries, "end": ended})
    return _number(steps)


def _number(steps):
    for i, s in enumerate(steps):
        s["step"] = i
    return steps


def peak_tokens(steps, unit=64):
    """Most tokens live requests hold at any time, each rounded up to ``unit``."""
    held: dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // unit) * unit for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


def replay(loaded, steps, check_cache=True, page_users=None, poison_freed=False):
    """Run the steps through ``loaded.runner``; returns {(request, position): logits row}.
    ``page_users`` (a dict) receives, per page of the first cache group, the requests that held it.
    ``poison_freed``: the pages a request gives back are filled with NaN (keys) and infinities
    (values) before anyone takes them again, and so are all pages before the first step."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    runner, cache = loaded.runner, loaded.cache
    pos: dict[str, int] = {}
    out = {}

    def poison(group, pages):
        for i, store in enumerate(group.storage):  # keys, values (or whatever streams the cache has)
            store[:, pages] = float("nan") if i % 2 == 0 else float("inf")

    if poison_freed:
        for g in cache.groups:
            poison(g, slice(None))
    for s in steps:
        entries = []
        for e in s["entries"]:
            if not cache.has(e["id"]):
                cache.admit(e["id"])
                pos[e["id"]] = 0
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = runner.step(entries)
        if logits is not None:
            logits = logits.float().cpu()
            row = 0
            for e in s["entries"]:
                for w in e["want"]:
                    out[(e["id"], pos[e["id"]] + w)] = logits[row]
                    row += 1
            assert row == logits.shape[0]
        for e in s["entries"]:
            pos[e["id"]] += len(e["tokens"])
            if page_users is not None and cache.groups:
                for page in cache.block_table(0, e["id"]):
                    if page >= 0:
                        page_users.setdefault(page, set()).add(e["id"])
        for rid in s["end"]:
            held = [[p for p in g.tables[rid] if p >= 0] for g in cache.groups]
            cache.release(rid)
            if poison_freed:
                for g, pages in zip(cache.groups, held):
                    poison(g, torch.tensor(pages, dtype=torch.long, device=g.storage[0].device))
        if check_cache:
            cache.check()
    assert not cache.live_requests()
    return out


def plain_logits(folder, requests, device="cpu", positions=None):
    """The plain implementation's logits by (request, position), float64 arithmetic. ``device``:
    where torch runs it (models of a real width take minutes on the host); ``positions``: keep
    these only, per request."""
    from plain import qwen3_plain as P

    cfg, w = P.read_model(folder, device=device)
    out = {}
    for rid, toks in requests.items():
        logits = P.forward(cfg, w, toks).float().cpu()
        for p in (range(len(toks)) if positions is None else positions[rid]):
            out[(rid, p)] = logits[p]
    return out


def make_requests(vocab, lengths, seed=0):
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


# (rms, worst) of every bfloat16 comparison of the run, in units of the logits' deviation
MEASURED_NOISE: list = []


def compare_rounding_noise(got, want, rms_bound=0.015, worst_bound=0.08):
    """bfloat16 against the float64 plain implementation, in units of the logits' own spread.
    Activations are rounded to 8 bits of mantissa some seven times per layer, which leaves an
    error that behaves like noise: its root mean square is about 1 % of the logits' standard
    deviation and its largest value over some 10^5 logits five times that. A fault in a page, a
    mask or a portion's edge moves the logits of the positions it touches by a sizeable part of
    their standard deviation, so the worst error is bounded at 8 % of it and the rms at 1.5 %."""
    keys = sorted(want)
    assert set(got) == set(want), f"{len(set(want) - set(got))} positions are missing"
    w = torch.stack([want[k].double() for k in keys])
    err = torch.stack([got[k].double() for k in keys]) - w
    std = float(w.std())
    rms = float(err.pow(2).mean().sqrt())
    per_pos = err.abs().amax(dim=1)
    worst = float(per_pos.max())
    where = keys[int(per_pos.argmax())]
    over = [keys[i] for i in torch.nonzero(per_pos >= worst_bound * std).flatten().tolist()]
    assert worst < worst_bound * std, (
        f"largest error {worst:.4f} at (request, position) {where}; logit deviation {std:.3f}; "
        f"first position over the bound: {over[0]}")
    assert rms < rms_bound * std, f"rms error {rms:.4f} against a logit deviation of {std:.3f}"
    MEASURED_NOISE.append((rms / std, worst / std, os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]))
    return rms / std, worst / std


def plain_logprobs(cfg, weights, prompt, tokens):
    """The plain implementation's log-probability of each of ``tokens`` following ``prompt`` (and
    each other), how far each lies below the best token of its place, and the logits' deviation."""
    from plain import qwen3_plain as P

    logits = P.forward(cfg, weights, list(prompt) + list(tokens))[len(prompt) - 1: -1].double()
    picked = logits[range(len(tokens)), list(tokens)]
    logprobs = torch.log_softmax(logits, dim=-1)[range(len(tokens)), list(tokens)]
    return logprobs.tolist(), (logits.max(dim=-1).values - picked).tolist(), float(logits.std())


def compare_logprobs(got, want, std, rms_bound=0.015, worst_bound=0.08):
    """Log-probabilities of given tokens, engine against plain (or graph against eager), by the
    measure of ``compare_rounding_noise``: in units of the logits' deviation ``std``."""
    err = torch.tensor(got, dtype=torch.float64) - torch.tensor(want, dtype=torch.float64)
    assert err.numel() and err.numel() == len(want)
    rms, worst = float(err.pow(2).mean().sqrt()), float(err.abs().max())
    assert worst < worst_bound * std, f"largest log-probability error {worst:.4f} at token {int(err.abs().argmax())}; logit deviation {std:.3f}"
    assert rms < rms_bound * std, f"rms log-probability error {rms:.4f} against a logit deviation of {std:.3f}"
    MEASURED_NOISE.append((rms / std, worst / std, os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]))


def check_tokens_chosen_in_bfloat16(cfg, weights, prompt, tokens, bound=0.08):
    """Tokens an engine chose greedily in bfloat16, judged by the plain implementation given the
    same context: each is the plain model's best token or lies below it by less than the
    rounding noise of two logits (``bound`` of the logits' deviation). A wrong cache or mask
    picks tokens far below the best."""
    _, below_best, std = plain_logprobs(cfg, weights, prompt, tokens)
    worst = max(below_best)
    assert worst < bound * std, f"token {below_best.index(worst)} lies {worst:.4f} below the plain model's best; deviation {std:.3f}"


def compare(got, want, atol, rtol):
    assert set(got) == set(want), f"{len(set(want) - set(got))} positions are missing"
    worst, where, first = 0.0, None, None
    for key in sorted(want):
        err = (got[key].double() - want[key].double()).abs()
        bound = atol + rtol * want[key].double().abs()
        excess = float((err - bound).max())
        if excess > 0 and first is None:
            first = (key, float(err.max()))
        if excess > worst:
            worst, where = excess, (key, float(err.max()))
    assert where is None, (
        f"first mismatch at (request, position) {first[0]} with max abs error {first[1]:.3e}; "
        f"worst at {where[0]} with {where[1]:.3e}"
    )
