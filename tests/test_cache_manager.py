"""The cache manager on the host: no page lost, held twice or freed twice, under
random orders of requests; the reference's own allocation vectors; windows; slots."""

import random

import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from qwen3_runtime_amd.cache import CacheFull, CacheManager, PagePool, StateSlots
from qwen3_runtime_amd.parts.plan import CacheSpec

FULL = CacheSpec("paged_kv", heads=2, head_dim=16)


def manager(num_pages, page_size, specs=(FULL,), max_requests=8, allocate=False):
    return CacheManager(list(specs), page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                        device="cpu", dtype=torch.float32, allocate=allocate)


def advance(m, rid, n):
    m.reserve(rid, n)
    m.commit(rid, n)


# --- the reference's vectors (tests/cpu/test_block_manager.py:7-80) -------------------------
def test_first_portion_takes_only_its_own_pages():
    m = manager(64, 16)
    m.admit("r")
    m.reserve("r", 512)                       # of an 8,192-token prompt
    assert len(m.block_table(0, "r")) == 32 and m.num_free_pages == 32


def test_second_portion_appends_and_keeps_the_prefix():
    m = manager(64, 16)
    m.admit("r")
    advance(m, "r", 512)
    first = list(m.block_table(0, "r"))
    m.reserve("r", 512)
    assert m.block_table(0, "r")[:32] == first and len(m.block_table(0, "r")) == 64 and m.num_free_pages == 0


def test_max_reservable_is_held_plus_free_minus_start():
    m = manager(2, 16)
    m.admit("r")
    assert m.max_reservable_tokens("r", 512) == 32
    advance(m, "r", 32)
    assert m.max_reservable_tokens("r", 512) == 0
    with pytest.raises(CacheFull):
        m.reserve("r", 1)
    m.check()


def test_slots_are_page_times_size_plus_offset():
    m = manager(4, 4)
    m.admit("r")
    m.reserve("r", 6)
    assert m.block_table(0, "r") == [0, 1]
    assert m.token_slots(0, "r", 0, 6).tolist() == [0, 1, 2, 3, 4, 5]


def test_decoding_takes_a_page_only_when_crossing_one():
    m = manager(4, 4)
    m.admit("r")
    advance(m, "r", 4)
    assert len(m.block_table(0, "r")) == 1
    advance(m, "r", 1)
    assert len(m.block_table(0, "r")) == 2
    advance(m, "r", 1)
    assert len(m.block_table(0, "r")) == 2


def test_trim_gives_back_pages_reserved_and_not_stored():
    """Pages taken ahead for a step that then does not come: back to the pool, stored tokens
    untouched, and the epoch says that tables handed out before are void."""
    window = CacheSpec("paged_kv", heads=1, head_dim=8, window=6)
    m = manager(6, 4, [FULL, window])
    m.admit("a")
    m.admit("b")
    advance(m, "a", 8)          # two pages in the full group; the window group has given one back
    advance(m, "b", 3)
    m.reserve("a", 1)           # the page of token 8, ahead of its step
    m.reserve("b", 6)           # two pages more, ahead
    held = {rid: [list(m.block_table(g, rid)) for g in range(2)] for rid in "ab"}
    assert len(held["a"][0]) == 3 and len(held["b"][0]) == 3
    free_before, epoch = [g.pool.num_free for g in m.groups], m.epoch
    assert m.trim() == 2 * (1 + 2)
    m.check()
    assert [g.pool.num_free for g in m.groups] == [f + 3 for f in free_before] and m.epoch == epoch + 1
    for rid, n in (("a", 2), ("b", 1)):
        for g in range(2):
            assert m.block_table(g, rid) == held[rid][g][:n]
    assert m.length("a") == 8 and m.length("b") == 3
    with pytest.raises(AssertionError):
        m.commit("a", 1)        # the reservation is gone with the pages
    advance(m, "a", 1)
    assert m.trim() == 0 and m.epoch == epoch + 1
    m.check()


def test_release_returns_everything_and_freed_pages_come_out_last():
    m = manager(8, 16)
    m.admit("a")
    m.reserve("a", 32)
    assert m.num_free_pages == 6
    m.release("a")
    assert m.num_free_pages == 8 and not m.has("a")
    m.admit("b")
    m.reserve("b", 16)
    assert m.block_table(0, "b") == [2]        # first in, first out: pages 0 and 1 went to the back


def test_bytes_per_page_of_the_4b_shape():
    # reference: qwen3_runtime/engine/memory.py:8-14, tests/cpu/test_memory.py:16-19
    specs = [CacheSpec("paged_kv", heads=8, head_dim=128)] * 36
    assert CacheManager.bytes_per_page(specs, 16, 2) == 2_359_296


# --- misuse is caught where it happens ----------------------------------------------------------
def test_pool_refuses_double_free_and_foreign_free():
    pool = PagePool(3)
    p = pool.take("a")
    with pytest.raises(AssertionError, match="held by"):
        pool.give(p, "b")
    pool.give(p, "a")
    with pytest.raises(AssertionError, match="twice"):
        pool.give(p, "a")
    pool.check()


def test_commit_beyond_reservation_and_double_admit_are_errors():
    m = manager(4, 4)
    m.admit("r")
    with pytest.raises(AssertionError):
        m.admit("r")
    m.reserve("r", 3)
    with pytest.raises(AssertionError, match="reserved"):
        m.commit("r", 4)


def test_reserve_takes_pages_in_every_group_or_in_none():
    specs = [FULL, CacheSpec("paged_kv", heads=1, head_dim=8)]
    m = manager(4, 4, specs)
    assert len(m.groups) == 2
    m.admit("a")
    m.reserve("a", 12)
    m.admit("b")
    with pytest.raises(CacheFull):
        m.reserve("b", 8)
    assert all(len(m.block_table(g, "b")) == 0 for g in range(2))
    m.check()


# --- windows -----------------------------------------------------------------------------------------
def test_window_group_gives_back_pages_that_no_later_query_sees():
    specs = [FULL, CacheSpec("paged_kv", heads=2, head_dim=16, window=6)]
    m = manager(16, 4, specs)
    full, win = 0, 1
    assert m.groups[win].window == 6
    m.admit("r")
    advance(m, "r", 9)       # next query at 9 sees keys 4..9: page 0 (positions 0..3) is gone
    assert m.block_table(win, "r") == [-1, 1, 2]
    assert m.block_table(full, "r") == [0, 1, 2]
    for _ in range(40):
        advance(m, "r", 1)
    held = [p for p in m.block_table(win, "r") if p >= 0]
    assert len(held) <= 6 // 4 + 2
    assert len([p for p in m.block_table(full, "r") if p >= 0]) == 13
    m.check()
    with pytest.raises(AssertionError, match="given back"):
        m.token_slots(win, "r", 0, 1)
    m.release("r")
    assert all(g.pool.num_free == 16 for g in m.groups)


def test_window_pages_are_reused_by_the_same_request():
    m = manager(3, 4, [CacheSpec("paged_kv", heads=1, head_dim=8, window=4)])
    m.admit("r")
    for _ in range(100):       # 100 tokens through 3 pages of 4
        advance(m, "r", 1)
    m.check()
    assert m.length("r") == 100


# --- state slots ---------------------------------------------------------------------------------------
def test_state_slots_zero_on_take_and_keep_marked_tensors_over_restart():
    s = StateSlots(2)
    rec = s.add_tensor("recurrent", (3,), torch.float32)
    rng = s.add_tensor("draws", (1,), torch.int64, survives_restart=True)
    a = s.take("a")
    rec[a] = 5.0
    rng[a] = 7
    s.reset("a")
    assert rec[a].abs().sum() == 0 and int(rng[a]) == 7
    s.give("a")
    b = s.take("b")
    assert b == a and int(rng[b]) == 0
    s.take("c")
    with pytest.raises(CacheFull):
        s.take("d")
    with pytest.raises(AssertionError):
        s.give("zzz")


def test_state_caches_live_in_slots_and_restart_clears_them():
    specs = [FULL, CacheSpec("state", shape=(5,), dtype="float32")]
    m = manager(8, 4, specs, max_requests=2, allocate=True)
    m.admit("a")
    view = m.view(1, [None])
    assert view.state.shape == (2, 5)
    view.state[m.slots.slot("a")] = 3.0
    advance(m, "a", 6)
    m.restart("a")
    assert m.length("a") == 0 and m.num_free_pages == 8
    assert view.state[m.slots.slot("a")].abs().sum() == 0
    m.release("a")


def test_views_have_the_kernel_layout():
    m = manager(6, 8, [FULL, FULL], allocate=True)
    m.admit("a")
    m.reserve("a", 3)
    from qwen3_runtime_amd.parts.base import GroupView

    gv = [GroupView(8, None, None, None)]
    v0, v1 = m.view(0, gv), m.view(1, gv)
    assert v0.k.shape == (6, 2, 8, 16) and v0.v.shape == (6, 2, 16, 8)
    assert v0.k.data_ptr() != v1.k.data_ptr()
    table = np.empty((1, 4), dtype=np.int32)
    m.fill_tables(0, ["a"], table)
    assert table.tolist() == [[0, -1, -1, -1]]


# --- random orders ------------------------------------------------------------------------------------------
@settings(max_examples=60, deadline=None)
@given(seed=st.integers(0, 10_000), num_pages=st.integers(3, 24), page_size=st.sampled_from([1, 4, 8, 16]),
       window=st.sampled_from([None, 3, 17]))
def test_random_lifetimes_keep_every_page_accounted_for(seed, num_pages, page_size, window):
    rng = random.Random(seed)
    specs = [FULL] if window is None else [FULL, CacheSpec("paged_kv", heads=1, head_dim=8, window=window)]
    m = manager(num_pages, page_size, specs, max_requests=5)
    live, next_id = [], 0
    for _ in range(200):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            m.admit(next_id)
            live.append(next_id)
            next_id += 1
        elif op < 0.80 and live:
            rid = rng.choice(live)
            want = rng.choice([1, 1, 1, 2, 5, 13, 40])
            n = m.max_reservable_tokens(rid, want)
            assert 0 <= n <= want
            if n < want:
                with pytest.raises(CacheFull):
                    m.reserve(rid, want)
            if n:
                before = m.length(rid)
                m.reserve(rid, n)
                slots = m.token_slots(0, rid, before, n)
                assert len(set(slots.tolist())) == n
                m.commit(rid, n)
        elif op < 0.86 and live:
            rid = rng.choice(live)      # pages taken ahead, and given back before they are used
            ahead = m.max_reservable_tokens(rid, rng.choice([1, 9]))
            m.reserve(rid, ahead)
            if rng.random() < 0.5:
                lengths = {r: m.length(r) for r in live}
                m.trim()
                assert {r: m.length(r) for r in live} == lengths
                assert all(len(m.block_table(0, r)) == m.groups[0].pages_for(m.length(r)) for r in live)
        elif op < 0.9 and live:
            m.restart(rng.choice(live))
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            m.release(rid)
        m.check()
        # no slot of the cache is addressed by two live requests
        seen = set()
        for rid in live:
            pages = [p for p in m.block_table(0, rid) if p >= 0]
            assert not seen & set(pages)
            seen |= set(pages)
    for rid in live:
        m.release(rid)
    m.check()
    assert all(g.pool.num_free == num_pages for g in m.groups)
    assert m.slots.num_free == 5


# --- what a paged cache holds per token is the spec's to say ---------------------------------------
def test_streams_of_a_paged_cache_decide_storage_views_and_bytes():
    from qwen3_runtime_amd.parts.base import GroupView
    from qwen3_runtime_amd.parts.plan import PagedStream

    kv = CacheSpec("paged_kv", heads=2, head_dim=16, value_dim=24)          # values wider than keys
    latent = CacheSpec("paged", streams=(PagedStream("latent", 1, 40), PagedStream("rope_key", 1, 8, True)))
    assert kv.group_key() != FULL.group_key() and latent.group_key() != kv.group_key()
    # bytes: 2 * (16 + 24) elements per token for the first, 40 + 8 for the second
    assert CacheManager.bytes_per_page([kv, latent, FULL], 8, 2) == 8 * 2 * (80 + 48 + 64)
    m = manager(5, 8, [kv, latent, kv], allocate=True)
    assert len(m.groups) == 2
    views = [GroupView(8, None, None, None)] * 2
    a, b, c = (m.view(i, views) for i in range(3))
    assert a.k.shape == (5, 2, 8, 16) and a.v.shape == (5, 2, 24, 8) and a.pages["v"] is a.v
    assert b.k is None and b.pages["latent"].shape == (5, 1, 8, 40) and b.pages["rope_key"].shape == (5, 1, 8, 8)
    # two caches of one group have storage of their own
    a.k.fill_(1.0)
    assert float(c.k.abs().sum()) == 0.0 and c.k.shape == a.k.shape
    with pytest.raises(ValueError, match="names its streams"):
        CacheSpec("paged").page_streams()


def test_bytes_a_step_reads_follow_windows_and_states():
    specs = [FULL, CacheSpec("paged_kv", heads=1, head_dim=8, window=6), CacheSpec("state", shape=(5,), dtype="float32")]
    m = manager(8, 4, specs, allocate=True)
    # all keys and values of the full cache, at most six tokens of the windowed one, the state once per request
    assert m.bytes_read([10, 3], dtype_bytes=2) == (13 * 64 + (6 + 3) * 16) * 2 + 2 * 5 * 4


def test_a_window_group_needs_its_windows_pages_only():
    window = CacheSpec("paged_kv", heads=1, head_dim=8, window=6)
    m = manager(3, 4, [window])
    assert m.can_ever_hold(10_000) == (True, "")         # six positions touch at most three pages of four
    ok, why = manager(2, 4, [window]).can_ever_hold(100)
    assert not ok and "window 6" in why and "needs 3" in why
    assert manager(2, 4, [window]).can_ever_hold(8)[0]    # a short request needs its own length only
    ok, why = manager(3, 4, [window, FULL]).can_ever_hold(13)
    assert not ok and "needs 4 cache pages" in why        # the group that keeps every key decides
