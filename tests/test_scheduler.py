"""The scheduler's decisions, on token lists alone (no model): admission, the token
budget and how prompts are cut, mixed batches, what happens when pages run out, and the
finishing rules.  Vectors marked (ref) are the reference's own
(tests/test_scheduler.py in ROCm/ATOM)."""

import pytest

from atom_amd.cache import CacheManager, GroupSpec
from atom_amd.config import Config, model_config_from_dict
from atom_amd.engine.scheduler import Scheduler
from atom_amd.engine.sequence import Sequence, SequenceStatus
from atom_amd.sampling import SamplingParams
from tiny import TINY_C


class FakeCore:
    """What the scheduler needs of the engine core: the cache manager and open/close."""

    def __init__(self, groups, slots, prefix_caching=False):
        self.manager = CacheManager(groups, slots, prefix_caching=prefix_caching)

    def open(self, rid):
        if rid not in self.manager:
            self.manager.open(rid)

    def match_prefix(self, rid, token_ids):
        return self.manager.match_prefix(rid, token_ids)

    def close(self, rid):
        if rid in self.manager:
            self.manager.close(rid)

    def resolve(self, rid, position, token):
        if rid in self.manager and self.manager.awaited_position(rid) == position:
            self.manager.amend(rid, position, token)


def make(blocks=100, block=4, window_group=None, prefix_caching=False, **kw):
    raw = {**TINY_C, "max_position_embeddings": 4096, "eos_token_id": 2}
    kw.setdefault("max_num_seqs", 4)
    kw.setdefault("max_num_batched_tokens", 64)
    kw.setdefault("max_model_len", 1024)
    cfg = Config("x", model_config=model_config_from_dict(raw), kv_cache_block_size=block, **kw)
    groups = [GroupSpec(block, blocks)]
    if window_group:
        groups.append(GroupSpec(block, window_group[1], window=window_group[0]))
    core = FakeCore(groups, cfg.max_num_seqs, prefix_caching)
    return Scheduler(cfg, core), core


def seq(tokens, **sp):
    return Sequence(list(tokens), SamplingParams(**sp))


def run(sched, batch, token=5):
    """Pretends the step ran: every final item samples ``token``."""
    sampled = {it.seq.id: (token(it.seq) if callable(token) else token) for it in batch.items if it.is_final}
    if sched.manager.prefix_caching:   # what the step function does after running the tokens
        for it in batch.items:
            sched.manager.commit(it.seq.id, it.start + it.num_tokens, it.seq.token_ids[it.start:it.start + it.num_tokens])
    return sched.postprocess(batch, sampled)


def test_budget_two_prompts_128_64():   # (ref) :236-254
    sched, _ = make(max_num_batched_tokens=192, blocks=100)
    sched.add(seq(range(128)))
    sched.add(seq(range(200, 328)))
    batch = sched.schedule()
    assert [it.num_tokens for it in batch.items] == [128, 64]
    assert [it.is_final for it in batch.items] == [True, False]


def test_budget_sliver_is_left_for_the_next_step():   # (ref) :256-278
    sched, _ = make(max_num_batched_tokens=200, blocks=400)
    for start in (0, 200, 400):
        sched.add(seq(range(start, start + 128)))
    batch = sched.schedule()
    assert [it.num_tokens for it in batch.items] == [128, 64]     # 8 tokens stay unspent
    assert len(sched.waiting) == 1


def test_prompt_cut_6_then_4():   # (ref) :280-314
    sched, _ = make(max_num_batched_tokens=6, blocks=100, block=4)
    s = seq(range(10))
    sched.add(s)
    b1 = sched.schedule()
    assert b1.entries()[0].tokens == list(range(6)) and b1.items[0].start == 0
    assert b1.entries()[0].want == []
    run(sched, b1)
    assert s.is_partial_prefill and s.num_cached_tokens == 6 and s.num_completion_tokens == 0
    b2 = sched.schedule()
    assert b2.entries()[0].tokens == list(range(6, 10)) and b2.items[0].start == 6
    assert b2.entries()[0].want == [3]
    run(sched, b2)
    assert not s.is_partial_prefill and s.num_cached_tokens == 10 and s.token_ids[-1] == 5


def test_chunking_off_is_all_or_nothing():
    sched, _ = make(max_num_batched_tokens=12, enable_chunked_prefill=False)
    sched.add(seq(range(8)))
    sched.add(seq(range(8)))
    assert [it.num_tokens for it in sched.schedule().items] == [8]
    sched2, _ = make(max_num_batched_tokens=12, enable_chunked_prefill=False)
    s = seq(range(20))
    sched2.add(s)
    assert sched2.schedule() is None
    assert sched2.take_rejected() == [s] and s.leave_reason.startswith("unschedulable")


def test_admission_respects_pages_and_blocks_the_queue():   # (ref) :316-321
    sched, _ = make(blocks=1, block=4)
    sched.add(seq([1, 2, 3, 4]))
    sched.add(seq([5, 6, 7, 8, 9]))     # two pages: can never run in a pool of one
    sched.add(seq([1, 2]))
    batch = sched.schedule()
    assert [it.num_tokens for it in batch.items] == [4]
    rejected = sched.take_rejected()
    assert len(rejected) == 1 and "cache pages" in rejected[0].leave_reason
    assert len(sched.waiting) == 1      # the short one waits behind: pages are taken


def test_too_long_prompt_is_rejected_not_hung():
    sched, _ = make(max_model_len=16)
    s = seq(range(17))
    sched.add(s)
    assert sched.schedule() is None
    assert sched.take_rejected() == [s] and "max_model_len" in s.leave_reason and s.is_finished
    assert sched.is_finished()


def test_max_num_seqs():
    sched, _ = make(max_num_seqs=2)
    for _ in range(3):
        sched.add(seq(range(4)))
    assert len(sched.schedule().items) == 2
    assert len(sched.waiting) == 1


def test_decode_and_prompt_share_one_step():
    sched, _ = make(max_num_batched_tokens=70)
    a = seq(range(8), max_tokens=10)
    sched.add(a)
    run(sched, sched.schedule())
    b = seq(range(100, 200), max_tokens=10)
    sched.add(b)
    batch = sched.schedule()
    kinds = [(it.seq.id, it.is_decode, it.num_tokens) for it in batch.items]
    # the decode token first; of the 69 tokens left the prompt gets 64 (a cut portion is floored to 64s)
    assert kinds == [(a.id, True, 1), (b.id, False, 64)]
    assert batch.entries()[0].tokens == [5] and batch.entries()[0].want == [0]
    assert batch.entries()[1].want == []
    run(sched, batch)
    batch = sched.schedule()
    assert [(it.is_decode, it.num_tokens, it.is_final) for it in batch.items] == [(True, 1, True), (False, 36, True)]
    run(sched, batch)
    batch = sched.schedule()
    assert [(it.is_decode, it.num_tokens) for it in batch.items] == [(True, 1), (True, 1)]


def test_decode_preemption():   # (ref) :332-346
    sched, core = make(blocks=2, block=4)
    s1, s2 = seq([1, 2, 3, 4], max_tokens=8), seq([5, 6, 7, 8], max_tokens=8)
    sched.add(s1)
    sched.add(s2)
    run(sched, sched.schedule(), token=9)
    batch = sched.schedule()
    assert {s1.status, s2.status} == {SequenceStatus.RUNNING, SequenceStatus.WAITING}
    assert s2.status == SequenceStatus.WAITING, "the last running request is the one preempted"
    assert [it.seq.id for it in batch.items] == [s1.id] and sched.total_preemptions == 1
    assert s2.num_cached_tokens == 0 and s2.id not in core.manager
    assert sched.waiting[0] is s2
    core.manager.check()


def test_preempted_request_prefills_prompt_plus_generated():
    sched, core = make(blocks=3, block=4, max_num_batched_tokens=64)
    s1, s2 = seq([1, 2, 3, 4], max_tokens=3), seq([5, 6, 7, 8], max_tokens=6)
    sched.add(s1)
    sched.add(s2)
    run(sched, sched.schedule(), token=9)        # both prompts; 2 pages held, 1 free
    run(sched, sched.schedule(), token=9)        # s1 takes the last page; s2 cannot: preempted
    assert s2.status == SequenceStatus.WAITING and s2.token_ids == [5, 6, 7, 8, 9]
    run(sched, sched.schedule(), token=9)        # s1 decodes (pool still full for s2)
    assert s1.is_finished and s1.leave_reason == "max_tokens"
    batch = sched.schedule()
    assert [it.seq.id for it in batch.items] == [s2.id]
    assert batch.entries()[0].tokens == [5, 6, 7, 8, 9] and not batch.items[0].is_decode
    assert batch.entries()[0].want == [4]
    run(sched, batch, token=9)
    assert s2.token_ids == [5, 6, 7, 8, 9, 9] and s2.num_cached_tokens == 5
    core.manager.check()


def test_lone_request_that_outgrows_the_pool_preempts_itself_then_is_rejected():
    sched, core = make(blocks=1, block=4)
    s = seq([1, 2, 3], max_tokens=10)
    sched.add(s)
    run(sched, sched.schedule())
    run(sched, sched.schedule())          # 4 tokens cached + 1 pending: needs a second page
    assert sched.schedule() is None       # preempted itself; now 5 tokens need 2 pages of a pool of 1
    out = sched.take_rejected()
    assert out == [s] and "cache pages" in s.leave_reason
    assert core.manager.num_free_pages() == 1 and sched.is_finished()


@pytest.mark.parametrize("kw,tokens,reason,count", [
    (dict(max_tokens=3), [7, 7, 7, 7], "max_tokens", 3),
    (dict(max_tokens=9), [7, 2, 7], "eos", 2),
    (dict(max_tokens=4, ignore_eos=True), [2, 2, 2, 2, 2], "max_tokens", 4),
])
def test_finish_reasons(kw, tokens, reason, count):   # (ref) :1110-1177
    sched, core = make()
    s = seq([1, 1, 1], **kw)
    sched.add(s)
    feed = iter(tokens)
    while not s.is_finished:
        run(sched, sched.schedule(), token=lambda _s: next(feed))
    assert s.leave_reason == reason and s.num_completion_tokens == count
    assert not sched.running and s.id not in core.manager


def test_stop_token_ids_and_stop_sequences():
    sched, _ = make()
    sched.stop_token_ids = {11}
    s = seq([1, 1], max_tokens=9)
    sched.add(s)
    feed = iter([7, 11])
    while not s.is_finished:
        run(sched, sched.schedule(), token=lambda _s: next(feed))
    assert s.leave_reason == "stop_11"
    s2 = Sequence([1, 1], SamplingParams(max_tokens=9), stop_token_sequences=[[8, 9]])
    sched.add(s2)
    feed = iter([8, 8, 9, 3])
    while not s2.is_finished:
        run(sched, sched.schedule(), token=lambda _s: next(feed))
    assert s2.leave_reason == "stop_sequence" and s2.completion_token_ids == [8, 8, 9]
    # a stop sequence wins over eos when both end at the same token
    s3 = Sequence([1], SamplingParams(max_tokens=9), stop_token_sequences=[[4, 2]])
    sched.add(s3)
    feed = iter([4, 2])
    while not s3.is_finished:
        run(sched, sched.schedule(), token=lambda _s: next(feed))
    assert s3.leave_reason == "stop_sequence"


def test_sequence_stops_at_max_model_len():
    sched, _ = make(max_model_len=6)
    s = seq([1, 1, 1, 1], max_tokens=50)
    sched.add(s)
    while not s.is_finished:
        run(sched, sched.schedule())
    assert s.leave_reason == "max_model_len" and s.num_tokens == 6


def test_long_prefill_threshold_caps_a_portion():
    sched, _ = make(max_num_batched_tokens=512, long_prefill_token_threshold=64, blocks=400)
    s = seq(range(200))
    sched.add(s)
    sizes = []
    while s.num_completion_tokens == 0:
        batch = sched.schedule()
        sizes.append(batch.items[0].num_tokens)
        run(sched, batch)
    assert sizes == [64, 64, 64, 8]


def test_whole_prompt_is_reserved_at_admission_where_all_keys_are_kept():
    sched, core = make(blocks=6, block=4, max_num_batched_tokens=8, window_group=(8, 20))
    a = seq(range(20))
    sched.add(a)
    sched.add(seq(range(8)))
    batch = sched.schedule()
    assert [it.num_tokens for it in batch.items] == [8]
    assert len(core.manager.block_table(a.id, 0)) == 5, "all five pages of the prompt are held from the start"
    assert len(core.manager.block_table(a.id, 1)) == 2, "the window group holds this step only"
    assert len(sched.waiting) == 1, "the second prompt waits: one free page is not enough for it"


def test_aborted_waiting_request_leaves_without_running():
    sched, _ = make()
    s = seq(range(4))
    s.status = SequenceStatus.ABORTED
    sched.add(s)
    assert sched.schedule() is None
    assert sched.take_rejected() == [s] and s.leave_reason == "aborted"


# ------------------------------------------------------------------ prefix cache


def test_new_request_starts_after_the_pages_that_hold_its_beginning():
    sched, core = make(blocks=20, block=4, prefix_caching=True)
    prompt = list(range(10, 20))
    a = seq(prompt, max_tokens=1)
    sched.add(a)
    batch = sched.schedule()
    assert [(it.start, it.num_tokens) for it in batch.items] == [(0, 10)]
    assert run(sched, batch) == [a]                      # finished; its two full pages stay findable
    b = seq(prompt + [99, 98], max_tokens=2)
    c = seq(prompt[:6] + [1, 2, 3], max_tokens=2)          # shares only the first page
    sched.extend([b, c])
    batch = sched.schedule()
    assert [(it.seq.id, it.start, it.num_tokens) for it in batch.items] == [(b.id, 8, 4), (c.id, 4, 5)]
    assert core.manager.block_table(b.id, 0)[0] == core.manager.block_table(c.id, 0)[0]   # one page, two holders
    run(sched, batch)
    core.manager.check()
    # the same prompt again: all but the last token's page comes from the cache, never the whole prompt
    d = seq(prompt[:8], max_tokens=1)
    sched.add(d)
    batch = sched.schedule()
    item = [it for it in batch.items if it.seq is d][0]
    assert (item.start, item.num_tokens) == (4, 4), "at least the last token is run"


def test_preempted_request_finds_its_own_pages_again():
    sched, core = make(blocks=6, block=4, prefix_caching=True, max_num_seqs=2)
    a, b = seq(range(100, 108), max_tokens=20, ignore_eos=True), seq(range(200, 208), max_tokens=20, ignore_eos=True)
    sched.extend([a, b])
    run(sched, sched.schedule())
    steps = 0
    while sched.total_preemptions == 0 and steps < 20:
        run(sched, sched.schedule())
        steps += 1
    assert sched.total_preemptions == 1 and b.status == SequenceStatus.WAITING
    core.manager.check()
    while a.status != SequenceStatus.FINISHED:
        run(sched, sched.schedule())
    batch = sched.schedule()
    item = [it for it in batch.items if it.seq is b][0]
    assert item.start >= 8, "the pages it filled before it was preempted are found by their content"


# ------------------------------------------------------------------ the step after a running one


def _decoding(sched, lengths, **sp):
    """Requests of these prompt lengths, prefilled and one token in."""
    seqs = [seq(range(10 * k, 10 * k + n), **sp) for k, n in enumerate(lengths)]
    for s in seqs:
        sched.add(s)
    run(sched, sched.schedule())
    return seqs


def test_schedule_ahead_takes_the_steady_decode_case():
    sched, core = make(blocks=40, block=4)
    a, b = _decoding(sched, [6, 9], max_tokens=8, ignore_eos=True)
    running = sched.schedule()
    assert [it.is_decode for it in running.items] == [True, True]
    ahead = sched.schedule_ahead(running)
    assert [(it.seq.id, it.start, it.num_tokens) for it in ahead.items] == [(a.id, 7, 1), (b.id, 10, 1)]
    assert a.awaits_token and b.awaits_token and a.num_tokens == 8 and a.num_cached_tokens == 7
    entries = ahead.entries({a.id: 0, b.id: 1})
    assert [(e.tokens, e.feed) for e in entries] == [([Sequence.PLACEHOLDER], 0), ([Sequence.PLACEHOLDER], 1)]
    # the running batch's tokens arrive: the placeholders become them, nothing else moves
    sched.postprocess(running, {a.id: 31, b.id: 32})
    assert a.token_ids[-1] == 31 and b.token_ids[-1] == 32 and not a.awaits_token
    assert a.num_tokens == 8 and a.num_cached_tokens == 7 and a.num_completion_tokens == 2
    sched.postprocess(ahead, {a.id: 41, b.id: 42})
    assert a.token_ids[-2:] == [31, 41] and a.num_cached_tokens == 8
    core.manager.check()


def test_schedule_ahead_leaves_out_what_finishes_by_its_count_and_drops_what_finished_meanwhile():
    sched, core = make(blocks=40, block=4)
    a, b, c = _decoding(sched, [5, 6, 7], max_tokens=9)
    a.max_tokens = 3                       # one token in; the running batch gives the second, the next the third
    running = sched.schedule()
    ahead = sched.schedule_ahead(running)
    assert [it.seq.id for it in ahead.items] == [a.id, b.id, c.id]
    done = sched.postprocess(running, {a.id: 9, b.id: 2, c.id: 9})      # b samples eos (2)
    assert [s.id for s in done] == [b.id] and b.leave_reason == "eos" and b.id not in core.manager
    running2 = ahead
    ahead2 = sched.schedule_ahead(running2)
    assert ahead2 is None                  # b is in the running batch but runs no more: not the steady case
    done = sched.postprocess(running2, {a.id: 9, b.id: 77, c.id: 9})
    assert [s.id for s in done] == [a.id] and a.leave_reason == "max_tokens"
    assert b.token_ids[-1] == 2 and b.num_completion_tokens == 2          # the token sampled for b after eos is dropped
    batch = sched.schedule()
    assert [it.seq.id for it in batch.items] == [c.id]
    assert sched.schedule_ahead(batch) is not None
    core.manager.check()


def test_schedule_ahead_skips_a_request_at_its_last_token():
    sched, core = make(blocks=40, block=4)
    a, b = _decoding(sched, [5, 6], max_tokens=5, ignore_eos=True)
    a.max_tokens = 2
    running = sched.schedule()
    ahead = sched.schedule_ahead(running)
    assert [it.seq.id for it in ahead.items] == [b.id] and a.awaits_token
    done = sched.postprocess(running, {a.id: 7, b.id: 8})
    assert [s.id for s in done] == [a.id] and a.token_ids[-1] == 7 and a.leave_reason == "max_tokens"
    core.manager.check()


def test_schedule_ahead_with_nothing_left_to_run_leaves_placeholders_that_postprocess_fills():
    """Every request of the running batch reaches its token count in it and nobody waits: the effects of the
    running batch are applied, nothing is scheduled, and the tokens still land where they belong."""
    sched, core = make(blocks=40, block=4)
    (a,) = _decoding(sched, [6], max_tokens=2, ignore_eos=True)
    running = sched.schedule()
    assert [it.seq.id for it in running.items] == [a.id]
    assert sched.schedule_ahead(running) is None
    assert a.awaits_token and a.num_cached_tokens == 7      # not "nothing changed": the request ends in a placeholder
    done = sched.postprocess(running, {a.id: 55})
    assert [s.id for s in done] == [a.id] and a.leave_reason == "max_tokens"
    assert a.token_ids[-1] == 55 and not a.awaits_token and a.num_completion_tokens == 2
    assert a.id not in core.manager and sched.schedule() is None
    core.manager.check()


def test_schedule_ahead_admits_and_continues_prompts():
    """What a step scheduled ahead may hold besides decode tokens: a request admitted meanwhile, the next
    portion of an unfinished prompt; a prompt that ends in the running batch decodes in the next."""
    sched, core = make(blocks=40, block=4)
    a, = _decoding(sched, [6], max_tokens=9)
    running = sched.schedule()
    new = seq(range(50, 55))
    sched.add(new)                                  # arrives while the batch runs
    ahead = sched.schedule_ahead(running)
    assert [(it.seq.id, it.start, it.num_tokens, it.is_decode) for it in ahead.items] == [(a.id, 7, 1, True), (new.id, 0, 5, False)]
    assert a.awaits_token and not new.awaits_token
    entries = ahead.entries({a.id: 0})
    assert [(e.tokens, e.feed) for e in entries] == [([Sequence.PLACEHOLDER], 0), (list(range(50, 55)), None)]
    sched.postprocess(running, {a.id: 5})
    assert a.token_ids[-1] == 5 and not a.awaits_token
    # the prompt ended in the batch that is now running: its first token too is read on the device
    running = ahead
    ahead = sched.schedule_ahead(running)
    assert [(it.seq.id, it.start, it.is_decode) for it in ahead.items] == [(a.id, 8, True), (new.id, 5, True)]
    assert ahead.entries({a.id: 0, new.id: 1})[1].feed == 1
    sched.postprocess(running, {a.id: 6, new.id: 7})
    sched.postprocess(ahead, {a.id: 8, new.id: 9})
    assert a.token_ids[-3:] == [5, 6, 8] and new.token_ids[-2:] == [7, 9]
    core.manager.check()
    # an unfinished prompt goes on with its next portion, beside a request that decodes
    sched, core = make(blocks=100, block=4, max_num_batched_tokens=65)
    d, = _decoding(sched, [6], max_tokens=9, ignore_eos=True)
    long = seq(range(150))
    sched.add(long)
    running = sched.schedule()
    assert [(it.num_tokens, it.is_final) for it in running.items] == [(1, True), (64, False)]
    ahead = sched.schedule_ahead(running)
    assert [(it.seq.id, it.start, it.num_tokens, it.is_final) for it in ahead.items] == [(d.id, 7, 1, True), (long.id, 64, 64, False)]
    assert d.awaits_token and long.is_partial_prefill and not long.awaits_token and long.num_cached_tokens == 64
    sched.postprocess(running, {d.id: 4})
    third = sched.schedule_ahead(ahead)
    assert [(it.start, it.num_tokens, it.is_final) for it in third.items] == [(8, 1, True), (128, 22, True)]
    sched.postprocess(ahead, {d.id: 4})
    sched.postprocess(third, {d.id: 4, long.id: 3})
    assert long.num_completion_tokens == 1 and long.num_cached_tokens == 150
    core.manager.check()


def test_schedule_ahead_declines_and_changes_nothing():
    # a request reaches its token count in the running batch while another waits for its place
    sched, core = make(blocks=40, block=4, max_num_seqs=2)
    a, b = _decoding(sched, [6, 7], max_tokens=9)
    a.max_tokens = 2
    sched.add(seq(range(50, 55)))
    running = sched.schedule()
    before = (a.num_tokens, b.num_tokens, b.num_cached_tokens, core.manager.num_free_pages(0))
    assert sched.schedule_ahead(running) is None
    assert (a.num_tokens, b.num_tokens, b.num_cached_tokens, core.manager.num_free_pages(0)) == before
    assert not a.awaits_token and not b.awaits_token
    # ... but a full house whose requests all go on keeps the waiting request out, so decoding runs ahead
    sched, core = make(blocks=40, block=4, max_num_seqs=2)
    a, b = _decoding(sched, [6, 7], max_tokens=9)
    sched.add(seq(range(50, 55)))
    running = sched.schedule()
    assert [it.is_decode for it in sched.schedule_ahead(running).items] == [True, True]
    # no page for the next token: left to the ordinary path, which preempts
    sched, core = make(blocks=4, block=4)
    a, b = _decoding(sched, [7, 7], max_tokens=9, ignore_eos=True)
    running = sched.schedule()                      # positions 7: the last slots of the second pages
    before = (a.num_tokens, a.num_cached_tokens, core.manager.num_free_pages(0))
    assert sched.schedule_ahead(running) is None
    assert (a.num_tokens, a.num_cached_tokens, core.manager.num_free_pages(0)) == before and not a.awaits_token
    # a request of the running batch was aborted meanwhile
    sched, core = make(blocks=40, block=4)
    a, b = _decoding(sched, [6, 7], max_tokens=9)
    running = sched.schedule()
    sched.abort(b.id)
    assert sched.schedule_ahead(running) is None and not a.awaits_token


# ------------------------------------------------------------------ the delay factor, abort, the next batch


class FakeClock:
    def __init__(self):
        self.now = 1000.0

    def __call__(self):
        return self.now


def test_delay_factor_holds_new_prompts_while_requests_run():
    """atom/model_engine/scheduler.py:2761-2777: with requests running, a waiting prompt is admitted only
    once the oldest waiting request has waited longer than delay_factor times the last prompt step's
    latency; with nothing running it is admitted at once."""
    clock = FakeClock()
    sched, _ = make(scheduler_delay_factor=2.0)
    sched.clock = clock
    first = seq(range(10), max_tokens=50, ignore_eos=True)
    first.arrive_time = clock.now
    sched.add(first)
    batch = sched.schedule()                      # nothing runs: admitted whatever the delay says
    assert [it.seq for it in batch.items] == [first]
    sched.postprocess(batch, {first.id: 5}, step_seconds=0.5)    # the last prompt step took 0.5 s
    late = seq(range(20, 30), max_tokens=5, ignore_eos=True)
    late.arrive_time = clock.now
    sched.add(late)
    clock.now += 0.9                              # waited 0.9 s <= 2.0 * 0.5 s
    batch = sched.schedule()
    assert [it.seq for it in batch.items] == [first] and batch.items[0].is_decode
    sched.postprocess(batch, {first.id: 5}, step_seconds=0.01)   # a decode step does not change the latency
    clock.now += 0.2                              # 1.1 s > 1.0 s
    batch = sched.schedule()
    assert [it.seq for it in batch.items] == [first, late]
    # without a delay factor the prompt would have gone in at once
    sched0, _ = make()
    a, b = seq(range(10), max_tokens=50, ignore_eos=True), seq(range(20, 30), max_tokens=5, ignore_eos=True)
    sched0.add(a)
    run(sched0, sched0.schedule())
    sched0.add(b)
    assert [it.seq for it in sched0.schedule().items] == [a, b]


def test_abort_of_waiting_and_running_requests_frees_pages():
    """atom/model_engine/scheduler.py:1195-1197, 2284-2285; engine_utility.py:219-229."""
    sched, core = make(blocks=20, block=4, max_num_seqs=2)
    a, b, c = (seq(range(k, k + 9), max_tokens=30, ignore_eos=True) for k in (0, 100, 200))
    sched.extend([a, b, c])
    run(sched, sched.schedule())                  # a and b run, c waits (two slots)
    assert a.status == b.status == SequenceStatus.RUNNING and c.status == SequenceStatus.WAITING
    used = core.manager.pools[0].num_pages - core.manager.pools[0].num_free
    assert used == 6
    assert sched.abort(c.id) and sched.abort(a.id) and not sched.abort(10 ** 9)
    assert not sched.abort(a.id), "a request is aborted once"
    batch = sched.schedule()
    gone = sched.take_rejected()
    assert {s.id for s in gone} == {a.id, c.id}
    assert all(s.leave_reason == "aborted" and s.leave_time > 0 for s in gone)
    assert a.num_completion_tokens == 1, "what it had generated stays"
    assert [it.seq for it in batch.items] == [b]
    assert list(sched.running) == [b] and not sched.waiting
    assert a.id not in core.manager and c.id not in core.manager
    assert core.manager.pools[0].num_pages - core.manager.pools[0].num_free == 3
    core.manager.check()
    # an aborted request whose step is still running: that step's result is dropped
    run(sched, batch)
    batch = sched.schedule()
    sched.abort(b.id)
    assert sched.postprocess(batch, {b.id: 7}) == []
    assert sched.schedule() is None
    assert [s.id for s in sched.take_rejected()] == [b.id] and sched.is_finished()
    assert core.manager.pools[0].num_free == core.manager.pools[0].num_pages


def test_next_batch_info():
    """atom/model_engine/scheduler.py:2724-2759, for steps that hold both kinds."""
    sched, _ = make(max_num_batched_tokens=64, max_num_seqs=4)
    assert sched.get_next_batch_info() == (False, 0, 0)
    sched.add(seq(range(100), max_tokens=9, ignore_eos=True))
    sched.add(seq(range(30), max_tokens=9, ignore_eos=True))
    assert sched.get_next_batch_info() == (True, 64, 1)
    batch = sched.schedule()
    assert (batch.total_tokens, len(batch.items)) == (64, 1)
    run(sched, batch)
    assert sched.get_next_batch_info() == (True, 36, 1)      # 36 left of the first; 28 of the second are a sliver
    batch = sched.schedule()
    assert (batch.total_tokens, len(batch.items)) == (36, 1)
    run(sched, batch)
    assert sched.get_next_batch_info() == (True, 31, 2)      # one decodes, the other's 30 tokens
    batch = sched.schedule()
    assert (batch.total_tokens, len(batch.items)) == (31, 2)
    run(sched, batch)
    assert sched.get_next_batch_info() == (False, 2, 2)
