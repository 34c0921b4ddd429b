"""The cache manager: block math, what is given back when, windows, state slots, and under
random orders of requests no page lost, held twice or freed twice."""

import random

import numpy as np
import pytest

from atom_amd.cache import CacheManager, GroupSpec, OutOfPages, OutOfSlots, PagePool, StateSlots


def test_pool_hands_out_lowest_first_and_refuses_double_free():
    pool = PagePool(4)
    assert [pool.take() for _ in range(3)] == [0, 1, 2]
    pool.give(1)
    pool.give(0)
    assert pool.take() == 0 and pool.take() == 1 and pool.take() == 3
    with pytest.raises(OutOfPages):
        pool.take()
    pool.give(2)
    with pytest.raises(AssertionError):
        pool.give(2)
    with pytest.raises(AssertionError):
        pool.give(7)


def test_state_slots():
    slots = StateSlots(2)
    a, b = slots.claim(), slots.claim()
    assert (a, b) == (0, 1)
    with pytest.raises(OutOfSlots):
        slots.claim()
    slots.release(a)
    with pytest.raises(AssertionError):
        slots.release(a)
    assert slots.claim() == 0


def test_block_counts_follow_the_reference():
    """4 tokens -> 1 block, 9 tokens -> 3 blocks at block size 4 (reference tests/test_block_manager.py:58-66)."""
    m = CacheManager([GroupSpec(4, 10)], 4)
    m.open("a")
    m.cover("a", 0, 4)
    assert len(m.block_table("a", 0)) == 1
    m.open("b")
    m.cover("b", 0, 9)
    assert len(m.block_table("b", 0)) == 3
    m.check()


def test_append_takes_a_block_exactly_when_a_token_starts_one():
    """The reference's may_append boundary (tests/test_block_manager.py:229-251): with block 4 a
    sequence of 4 tokens needs no new block for its tokens, the 5th token does."""
    m = CacheManager([GroupSpec(4, 10)], 2)
    m.open("a")
    m.cover("a", 0, 4)
    assert m.pages_missing("a", 3, 4) == [0]
    assert m.pages_missing("a", 4, 5) == [1]
    m.cover("a", 4, 5)
    assert len(m.block_table("a", 0)) == 2
    for n in (6, 7, 8):
        assert m.pages_missing("a", n - 1, n) == [0]
    assert m.pages_missing("a", 8, 9) == [1]
    assert m.pages_missing("a", 8, 8 + 5) == [2]        # several tokens at once (can_append with k)
    assert m.pages_missing("zzz", 0, 9) == [3]          # an unknown request counts from nothing


def test_cover_is_all_or_nothing_and_close_gives_everything_back():
    m = CacheManager([GroupSpec(4, 3)], 2)
    m.open("a")
    m.cover("a", 0, 8)
    m.open("b")
    assert not m.can_cover("b", 0, 5)
    with pytest.raises(OutOfPages):
        m.cover("b", 0, 5)
    assert m.block_table("b", 0) == [] and m.num_free_pages() == 1
    m.close("a")
    assert m.num_free_pages() == 3
    m.cover("b", 0, 5)
    assert m.block_table("b", 0) == [0, 1], "freed pages are used again, lowest first"
    m.check()


def test_reserve_holds_the_whole_prompt_only_where_every_key_is_kept():
    m = CacheManager([GroupSpec(4, 20), GroupSpec(4, 20, window=6)], 2)
    m.open("a")
    m.cover("a", 0, 4, reserve=18)
    assert len(m.block_table("a", 0)) == 5      # ceil(18 / 4) pages for the group that keeps all keys
    assert len(m.block_table("a", 1)) == 1      # the window group holds what the step needs
    m.check()


def test_slot_mapping():
    m = CacheManager([GroupSpec(4, 10)], 2)
    m.open("x")
    m.cover("x", 0, 2)         # takes page 0
    m.open("a")
    m.cover("a", 0, 10)        # pages 1, 2, 3
    assert m.slot_mapping("a", 0, 0, 10).tolist() == [4, 5, 6, 7, 8, 9, 10, 11, 12, 13]
    assert m.slot_mapping("a", 0, 7, 2).tolist() == [11, 12]
    assert m.slot_mapping("a", 0, 0, 10).dtype == np.int32


def test_window_group_gives_pages_back_as_the_window_passes():
    w, ps = 6, 4
    m = CacheManager([GroupSpec(ps, 5, window=w)], 1)
    m.open("a")
    n = 0
    for step in (3, 5, 1, 1, 8, 1, 1, 1, 2):
        m.cover("a", n, n + step)
        n += step
        m.commit("a", n)
        table = m.block_table("a", 0)
        first_needed = max(0, n - w + 1) // ps         # the next query sits at position n
        for idx, page in enumerate(table):
            assert (page >= 0) == (idx >= first_needed), (n, table)
        m.check()
    assert m.num_free_pages() >= 5 - (-(-(w + 8) // ps) + 1)
    m.close("a")
    assert m.num_free_pages() == 5


def test_window_group_never_needs_a_returned_page_again():
    m = CacheManager([GroupSpec(4, 8, window=4)], 1)
    m.open("a")
    m.cover("a", 0, 20)
    m.commit("a", 20)
    assert m.block_table("a", 0)[:4] == [-1, -1, -1, -1]
    m.cover("a", 20, 21)     # sees keys 17..20 only
    with pytest.raises(AssertionError):
        m.slot_mapping("a", 0, 3, 2)


def test_state_slot_held_from_open_to_close():
    m = CacheManager([GroupSpec(4, 4)], 2)
    assert m.open("a") == 0 and m.open("b") == 1
    assert not m.can_open()
    with pytest.raises(OutOfSlots):
        m.open("c")
    assert m.is_fresh("a")
    m.commit("a", 0)
    assert not m.is_fresh("a")
    m.close("a")
    assert m.open("c") == 0 and m.is_fresh("c")
    with pytest.raises(KeyError):
        m.open("c")


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    groups = [GroupSpec(4, 24), GroupSpec(8, 10, window=rng.choice([5, 16, 30])), GroupSpec(4, 12, window=9)]
    m = CacheManager(groups, 5)
    live: dict[int, int] = {}
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.can_open():
            m.open(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16, 33])
            cached = live[rid]
            reserve = cached + n + rng.choice([0, 0, 5, 20])
            before = [p.num_free for p in m.pools]
            if m.can_cover(rid, cached, cached + n, reserve):
                missing = m.pages_missing(rid, cached, cached + n, reserve)
                m.cover(rid, cached, cached + n, reserve)
                assert [b - p.num_free for b, p in zip(before, m.pools)] == missing
                for gi in range(len(groups)):
                    m.slot_mapping(rid, gi, cached, n)      # every new position has a page
                live[rid] = cached + n
                m.commit(rid, live[rid])
            else:
                with pytest.raises(OutOfPages):
                    m.cover(rid, cached, cached + n, reserve)
                assert [p.num_free for p in m.pools] == before
        elif live:
            rid = rng.choice(list(live))
            m.close(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.close(rid)
    m.check()
    assert all(p.num_free == g.num_pages for p, g in zip(m.pools, groups))
    assert m.slots.num_free == 5


def test_plan_groups_layers_by_window():
    import torch
    from atom_amd.cache import group_runs, plan_cache
    from atom_amd.config import build_model, model_config_from_dict
    from tiny import TINY_C

    model = build_model(model_config_from_dict(TINY_C))
    windows, run_group = group_runs(model)
    assert windows == [None, 40] and run_group == [0, 1, 1, 0]
    plan = plan_cache(model, 16, torch.bfloat16, num_pages=7)
    assert [g.num_pages for g in plan.groups] == [7, 7]
    assert plan.bytes_per_page == [2 * (2 * 2 * 64 * 16 * 2)] * 2     # two layers a group, K and V
    plan = plan_cache(model, 16, torch.bfloat16, budget_bytes=10 << 20, max_num_seqs=4, max_model_len=1024,
                      max_num_batched_tokens=64)
    per_req = -(-(40 + 64) // 16) + 1
    assert plan.groups[1].num_pages == 4 * per_req
    assert plan.groups[0].num_pages == ((10 << 20) - 4 * per_req * plan.bytes_per_page[1]) // plan.bytes_per_page[0]


# ------------------------------------------------------------------ prefix cache


def _run(m, rid, tokens, start=0):
    """Takes pages for ``tokens`` at ``start`` and notes them as run."""
    m.cover(rid, start, start + len(tokens))
    m.commit(rid, start + len(tokens), tokens)


def test_pool_prefers_pages_without_a_hash_then_the_oldest_hashed():
    """Free order of the reference's pool (tests/test_block_pool.py:26-60): vacant pages first, lowest id first;
    then hashed pages in the order they were released; a page that is handed out again forgets its hash."""
    pool = PagePool(4)
    pages = [pool.take() for _ in range(4)]
    pool.publish(1, 111, (1,))
    pool.publish(2, 222, (2,))
    for p in (2, 0, 1, 3):
        pool.give(p)
    assert pool.num_free == 4
    assert pool.find(222, (2,)) == 2 and pool.find(222, (9,)) is None, "a hash answers only for its own tokens"
    assert [pool.take() for _ in range(3)] == [0, 3, 2]     # vacant 0, 3, then 2 (released before 1)
    assert pool.find(222, (2,)) is None and pool.find(111, (1,)) == 1
    pool.share(1)                                            # found by content: held again, no longer evictable
    with pytest.raises(OutOfPages):
        pool.take()
    assert pool.refs(1) == 1 and pages == [0, 1, 2, 3]


def test_hash_is_published_only_after_the_step_and_chains_over_the_prefix():
    m = CacheManager([GroupSpec(4, 10)], 4, prefix_caching=True)
    prompt = [5, 6, 7, 8, 9, 10, 11, 12, 13]
    m.open("a")
    m.cover("a", 0, 9)
    m.open("b")
    assert m.match_prefix("b", prompt) == 0, "pages are taken but nothing has been run yet"
    m.commit("a", 9, prompt)
    m.close("b")
    m.open("b")
    assert m.match_prefix("b", prompt) == 8 and m.block_table("b", 0) == m.block_table("a", 0)[:2]
    m.open("c")
    assert m.match_prefix("c", [0, 0, 0, 0] + prompt[4:]) == 0, "same second page, other prefix: no hit"
    m.open("d")
    assert m.match_prefix("d", prompt[:8]) == 4, "the last token is always left to run"
    m.check()
    m.close("a")
    m.check()
    assert m.num_free_pages() == 10 - 2, "b still holds the two shared pages"
    for r in ("b", "c", "d"):
        m.close(r)
    assert m.num_free_pages() == 10
    m.open("e")
    assert m.match_prefix("e", prompt) == 8, "released pages stay findable until the pool needs them"
    m.check()


def test_prefix_cache_random_orders():
    rng = random.Random(5)
    m = CacheManager([GroupSpec(4, 24), GroupSpec(4, 24)], 4, prefix_caching=True)
    stems = [[rng.randrange(50) for _ in range(12)] for _ in range(3)]
    live = {}
    for step in range(400):
        if live and (len(live) == 4 or rng.random() < 0.4):
            rid = rng.choice(list(live))
            tokens, at = live[rid]
            if at >= len(tokens) or rng.random() < 0.1:
                m.close(rid)
                del live[rid]
            else:
                n = min(rng.choice([1, 1, 2, 5]), len(tokens) - at)
                if m.can_cover(rid, at, at + n):
                    _run(m, rid, tokens[at:at + n], at)
                    live[rid] = (tokens, at + n)
                else:
                    m.close(rid)
                    del live[rid]
        else:
            rid = f"r{step}"
            tokens = rng.choice(stems)[:rng.randrange(4, 13)] + [rng.randrange(50) for _ in range(rng.randrange(0, 9))]
            m.open(rid)
            hit = m.match_prefix(rid, tokens)
            assert hit % 4 == 0 and hit < len(tokens)
            for gi in range(2):
                assert len(m.block_table(rid, gi)) == hit // 4
            live[rid] = (tokens, hit)
        m.check()
    assert m.pools[0].hits > 20
    for rid in list(live):
        m.close(rid)
    m.check()
    assert m.num_free_pages(0) == 24 and m.num_free_pages(1) == 24


def test_prefix_cache_refuses_window_groups():
    with pytest.raises(ValueError):
        CacheManager([GroupSpec(4, 8, window=6)], 2, prefix_caching=True)


def test_a_page_is_named_only_when_all_its_tokens_are_known():
    """A token that ran before the host knew it (read on the device) keeps its page out of the prefix
    cache until ``amend`` tells its value."""
    mgr = CacheManager([GroupSpec(4, 8)], 2, prefix_caching=True)
    mgr.open("a")
    mgr.cover("a", 0, 7)
    mgr.commit("a", 7, [1, 2, 3, 4, 5, 6, 7])
    assert mgr.pools[0].hash_of(mgr.block_table("a", 0)[0]) is not None
    mgr.cover("a", 7, 8)
    mgr.commit("a", 8, [0], last_unknown=True)            # fills the second page, value unknown
    assert mgr.awaited_position("a") == 7
    assert mgr.pools[0].hash_of(mgr.block_table("a", 0)[1]) is None
    with pytest.raises(AssertionError):
        mgr.commit("a", 9, [0], last_unknown=True)         # never two at once
    with pytest.raises(AssertionError):
        mgr.amend("a", 6, 9)
    mgr.amend("a", 7, 8)
    assert mgr.awaited_position("a") is None
    assert mgr.pools[0].hash_of(mgr.block_table("a", 0)[1]) is not None
    mgr.close("a")
    mgr.open("b")
    assert mgr.match_prefix("b", [1, 2, 3, 4, 5, 6, 7, 8, 9]) == 8      # found under the amended token
    mgr.close("b")
    mgr.open("c")
    assert mgr.match_prefix("c", [1, 2, 3, 4, 5, 6, 7, 0, 9]) == 4      # not under the placeholder
    mgr.check()
