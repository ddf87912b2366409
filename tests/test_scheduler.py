"""The scheduler's decisions, with no model: the reference's own vectors
(tests/cpu/test_scheduler.py:22-222), what happens when pages run out, finish reasons."""

import pytest
import torch

from qwen3_runtime_amd.cache import CacheManager
from qwen3_runtime_amd.config.engine import EngineConfig
from qwen3_runtime_amd.engine.request import Phase, Request
from qwen3_runtime_amd.engine.scheduler import Scheduler
from qwen3_runtime_amd.parts.plan import CacheSpec
from qwen3_runtime_amd.sampling.params import SamplingParams


def scheduler(num_pages=64, page_size=16, max_seqs=4, budget=512, eos=None, max_len=100_000):
    cfg = EngineConfig(page_size=page_size, num_pages=num_pages, max_num_seqs=max_seqs,
                       max_num_batched_tokens=budget, eos_token_id=eos, dtype="float32", device="cpu")
    cache = CacheManager([CacheSpec("paged_kv", heads=1, head_dim=8)], page_size=page_size, num_pages=num_pages,
                         max_requests=max(max_seqs, 16), device="cpu", dtype=torch.float32, allocate=False)
    return Scheduler(cfg, cache, max_len)


def run(s, batch, tokens):
    """What the engine does between schedule() and settle(): the tokens are stored."""
    for r in batch:
        s.cache.commit(r.request_id, r.grant)
    return s.settle(batch, tokens)


def test_first_portion_reserves_only_its_pages():
    s = scheduler(num_pages=513, budget=512)
    req = Request(list(range(8192)), max_tokens=1)
    s.add(req)
    batch = s.schedule()
    assert batch == [req] and req.grant == 512
    assert len(s.cache.block_table(0, req.request_id)) == 32 and s.cache.num_free_pages == 481
    assert req.phase == Phase.RUNNING


def test_budget_cuts_a_prompt_into_portions():
    s = scheduler(num_pages=256, budget=128)
    req = Request(list(range(300)), max_tokens=1)
    s.add(req)
    sizes = []
    for _ in range(3):
        batch = s.schedule()
        sizes.append(req.grant)
        run(s, batch, [None if sum(sizes) < 300 else 5])
    assert sizes == [128, 128, 44]
    assert req.phase == Phase.DONE and req.finish_reason == "length"
    assert s.cache.num_free_pages == 256


def test_two_prompts_share_the_budget():
    s = scheduler(num_pages=64, page_size=8, budget=10)
    a, b = Request(list(range(8)), 1), Request(list(range(8, 16)), 1)
    s.add(a), s.add(b)
    assert s.schedule() == [a, b]
    assert (a.grant, b.grant) == (8, 2)


def test_a_long_prompt_takes_the_whole_budget():
    s = scheduler(num_pages=2048, max_seqs=8, budget=2048)
    long, short = Request(list(range(9981)), 8), Request(list(range(16)), 8)
    s.add(long), s.add(short)
    for _ in range(2):
        batch = s.schedule()
        assert batch == [long] and long.grant == 2048
        run(s, batch, [None])


def test_decode_and_a_new_prompt_in_one_step():
    s = scheduler(num_pages=32, page_size=4, budget=16)
    d = Request(list(range(4)), max_tokens=4)
    s.add(d)
    run(s, s.schedule(), [99])
    p = Request(list(range(40)), max_tokens=1)
    s.add(p)
    batch = s.schedule()
    assert batch == [d, p] and (d.grant, p.grant) == (1, 15)


def test_portion_shrinks_to_the_free_pages():
    s = scheduler(num_pages=4, page_size=16, budget=512)
    a, b = Request(list(range(31)), 1), Request(list(range(40)), 1)
    s.add(a), s.add(b)
    assert s.schedule() == [a, b]
    assert (a.grant, b.grant) == (31, 32)
    assert len(s.cache.block_table(0, b.request_id)) == 2


def test_throughput_shape_two_waves_then_mixed():
    s = scheduler(num_pages=512, max_seqs=16, budget=2048)
    reqs = [Request(list(range(256)), max_tokens=128) for _ in range(16)]
    for r in reqs:
        s.add(r)
    first = s.schedule()
    assert len(first) == 8 and sum(r.grant for r in first) == 2048
    run(s, first, [1] * 8)
    second = s.schedule()
    assert sum(1 for r in second if r.grant == 1) == 8
    assert sum(r.grant for r in second) == 2048


def test_request_that_can_never_fit_is_refused():
    s = scheduler(num_pages=2, page_size=16)
    with pytest.raises(RuntimeError, match="needs 4 cache pages"):
        s.add(Request(list(range(48)), max_tokens=1))
    s = scheduler(num_pages=64, max_len=40)
    with pytest.raises(RuntimeError, match="limit of 40"):
        s.add(Request(list(range(30)), max_tokens=12))
    s.add(Request(list(range(30)), max_tokens=11))  # 40 positions are fed, the 41st token is only sampled


def test_pages_run_out_the_youngest_is_preempted_and_recomputed():
    s = scheduler(num_pages=4, page_size=4, budget=32)
    a, b = Request(list(range(8)), max_tokens=4), Request(list(range(8, 16)), max_tokens=4)
    s.add(a), s.add(b)
    run(s, s.schedule(), [11, 22])
    assert s.cache.num_free_pages == 0
    batch = s.schedule()                      # both want a fifth page; none is free
    assert s.num_preemptions == 1 and b.restarts == 1
    # a decodes with one of the two freed pages; b restarts at once with the other
    # (reference: tests/cpu/test_scheduler.py:115-131 expects a restarted request in this batch)
    assert batch == [a, b] and (a.grant, b.grant) == (1, 4)
    assert b.token_ids == list(range(8, 16)) + [22]          # keeps prompt and output
    assert b.holds_slot                                          # keeps its slot
    slot = s.cache.slots.slot(b.request_id)
    run(s, batch, [12, None])
    # b comes back: recomputes prompt + its one token in portions, samples only when caught up
    seen = []
    for _ in range(12):
        batch = s.schedule()
        toks = []
        for r in batch:
            end = s.cache.length(r.request_id) + r.grant
            toks.append(7 if end >= len(r.token_ids) else None)
            if r is b:
                seen.append((r.grant, toks[-1]))
        run(s, batch, toks)
        s.cache.check()
        if s.is_finished():
            break
    assert s.is_finished() and a.finish_reason == b.finish_reason == "length"
    assert len(a.output_tokens) == len(b.output_tokens) == 4
    assert seen[0] == (5, 7)                                   # the rest of its 9 tokens, then a sample
    assert s.num_preemptions >= 1
    assert s.cache.num_free_pages == 4 and s.cache.slots.num_free == 16


def test_running_request_without_a_page_sits_out_while_others_go_on():
    s = scheduler(num_pages=3, page_size=4, budget=32)
    a, b = Request(list(range(4)), max_tokens=8), Request(list(range(7)), max_tokens=2)
    s.add(a), s.add(b)
    run(s, s.schedule(), [1, 2])            # a holds 1 page (full), b holds 2 (7 of 8 slots)
    batch = s.schedule()
    assert batch == [b] and s.num_preemptions == 0   # a needs a new page and waits; b still has room
    run(s, batch, [3])
    assert b.phase == Phase.DONE
    assert s.schedule() == [a]


def test_portions_of_a_multiple_where_a_part_asks_for_it():
    """A mixer that works on blocks of 8 tokens: every portion but a request's last is a
    multiple of 8, whatever the token limit and the free pages would allow."""
    s = scheduler(num_pages=64, page_size=4, budget=21)
    s.portion_multiple = 8
    a, b = Request(list(range(30)), max_tokens=1), Request(list(range(9)), max_tokens=1)
    s.add(a), s.add(b)
    seen = []
    while not s.is_finished():
        batch = s.schedule()
        seen.append([(r.request_id - a.request_id, r.grant) for r in batch])
        run(s, batch, [5 if s.cache.length(r.request_id) + r.grant >= len(r.token_ids) else None for r in batch])
    # 21 tokens a step: 16 of a (not 21); b's 9 do not fit whole into the 5 (then 7) tokens left,
    # and a part of them would be no multiple of 8, so b waits; a's last 14 end it and need no rounding
    assert seen == [[(0, 16)], [(0, 14)], [(1, 9)]]


def test_nothing_running_and_no_page_is_an_error():
    s = scheduler(num_pages=2, page_size=4, budget=32)
    s.add(Request(list(range(5)), max_tokens=2))
    s.cache.admit("squatter")
    s.cache.reserve("squatter", 8)
    s.cache.commit("squatter", 8)   # stored tokens: pages held only ahead of the books would go back
    with pytest.raises(RuntimeError, match="cannot get a cache page"):
        s.schedule()


def test_slots_limit_residents_and_keep_arrival_order():
    s = scheduler(num_pages=64, page_size=4, max_seqs=2, budget=64)
    s.cache.slots = type(s.cache.slots)(2)
    reqs = [Request([1, 2, 3], max_tokens=2) for _ in range(3)]
    for r in reqs:
        s.add(r)
    assert s.schedule() == reqs[:2]
    run(s, reqs[:2], [5, 5])
    assert s.schedule() == reqs[:2]
    run(s, reqs[:2], [5, 5])
    assert s.schedule() == [reqs[2]]


@pytest.mark.parametrize("ignore_eos,min_tokens,tokens,reason,n_out", [
    (True, 0, [9, 9, 9], "length", 3),        # stop ids do not count unless asked (engine default)
    (False, 0, [4, 9, 4], "stop", 2),         # eos
    (False, 0, [4, 77, 4], "stop", 2),        # a stop id of the request
    (False, 3, [9, 9, 4], "length", 3),       # min_tokens holds the stop back, then length wins
    (False, 2, [9, 9, 9], "stop", 2),
])
def test_finish_reasons(ignore_eos, min_tokens, tokens, reason, n_out):
    # reference: qwen3_runtime/engine/scheduler.py:106-122
    s = scheduler(eos=9)
    req = Request([1, 2], max_tokens=3, ignore_eos=ignore_eos, stop_token_ids=(77,),
                  sampling=SamplingParams(min_tokens=min_tokens))
    s.add(req)
    for tok in tokens:
        if req.phase == Phase.DONE:
            break
        run(s, s.schedule(), [tok])
    assert req.finish_reason == reason and req.num_output_tokens == n_out
    assert s.is_finished() and s.cache.num_free_pages == 64


def test_request_validation_and_forced_tokens():
    with pytest.raises(ValueError):
        Request([], 4)
    with pytest.raises(ValueError):
        Request([1], 0)
    r = Request([1, 2], 4, forced_tokens=[5, 6])
    assert r.forced_next() == 5
    r.token_ids += [5, 6]
    assert r.forced_next() is None
    assert Request([1], 1, sampling=SamplingParams(seed=3)).seed == 3


def test_sampling_params_validation():
    # reference: qwen3_runtime/sampling_params.py:31-43
    for bad in (dict(temperature=float("nan")), dict(top_p=0.0), dict(top_p=1.5), dict(min_p=-0.1),
                dict(min_p=1.1), dict(min_tokens=-1), dict(repetition_penalty=0.0),
                dict(repetition_penalty=float("inf"))):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    assert SamplingParams().is_greedy() and SamplingParams(temperature=-1.0).is_greedy()
    assert not SamplingParams(temperature=0.5).is_greedy()
    assert SamplingParams(presence_penalty=0.1).has_penalties() and not SamplingParams().has_penalties()


def test_a_windowed_model_serves_requests_longer_than_its_pool():
    """One group of caches with a window of 12 tokens and a pool of five pages of four: a request of
    200 tokens is admitted (its window's pages are all it ever needs at once), its prompt is cut to
    what the pool holds, pages behind the window come back as it goes, and it ends."""
    cfg = EngineConfig(page_size=4, num_pages=5, max_num_seqs=2, max_num_batched_tokens=64, dtype="float32",
                       device="cpu")
    cache = CacheManager([CacheSpec("paged_kv", heads=1, head_dim=8, window=12)], page_size=4, num_pages=5,
                         max_requests=4, device="cpu", dtype=torch.float32, allocate=False)
    s = Scheduler(cfg, cache, 100_000)
    req = Request(list(range(150)), max_tokens=50)
    s.add(req)
    grants = []
    while not s.is_finished():
        batch = s.schedule()
        assert batch == [req] and 1 <= req.grant <= 20
        grants.append(req.grant)
        caught_up = cache.length(req.request_id) + req.grant >= len(req.token_ids)
        run(s, batch, [7 if caught_up else None])
        cache.check()
        assert len(grants) < 400
    assert req.finish_reason == "length" and len(req.output_tokens) == 50
    assert max(grants) > 1 and cache.num_free_pages == 5
    # a model that keeps every key refuses the same request in the same pool
    with pytest.raises(RuntimeError, match="needs 50 cache pages"):
        scheduler(num_pages=5, page_size=4).add(Request(list(range(150)), max_tokens=50))


def test_pages_held_ahead_do_not_change_what_a_prompt_is_offered():
    """A replayed decode step reserves the page of its request's next token while the device runs.
    In a pool at its peak such a page must not shorten a queued prompt's portion: the plan is the
    one made with the books as the last step left them."""
    def plan(reserve_ahead):
        s = scheduler(num_pages=4, page_size=4, budget=32)
        a = Request(list(range(4)), max_tokens=8)
        s.add(a)
        run(s, s.schedule(), [9])                       # a holds one page, full; its next token needs a second
        if reserve_ahead:
            s.cache.reserve(a.request_id, 1)            # what the step function does ahead of the books
        b = Request(list(range(100, 108)), max_tokens=2)
        s.add(b)
        batch = s.schedule()
        s.cache.check()
        return [(r is a, r.grant) for r in batch], s.cache.num_free_pages

    assert plan(True) == plan(False) == ([(True, 1), (False, 8)], 0)
