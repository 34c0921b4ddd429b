"""The engine's bookkeeping without a GPU: the step function, the cache manager and the
model assembly run with plain PyTorch stand-ins for the kernels (``plain_kernels``) and
must reproduce the plain implementation under every way of cutting the work.  What is
tested here is paging, batching and metadata; the kernels themselves are tested on the GPU."""

import pytest
import torch

import replay
from helpers import make_core, oracle_logits, random_ids
from plain_kernels import PlainKernels
from tiny import CONFIGS

LENGTHS = {"A": [5, 17, 33, 70], "B": [1, 9, 40, 71], "C": [3, 50, 120, 64, 95, 31]}


def _requests(which, seed=0):
    return {f"r{k}": random_ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


@pytest.mark.parametrize("which", ["A", "B", "C"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut):
    requests = _requests(which)
    oracle = {rid: oracle_logits(which, ids) for rid, ids in requests.items()}
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 64) // 16)
    core = make_core(which, "float32", PlainKernels(), "cpu", num_pages=pages, page_size=16)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, "float32", f"{which}/{cut}")
    assert not core.manager.live_requests()
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


def test_small_pages_and_reuse():
    """Config B with its own page size of 8 and a pool so small that pages are used again."""
    requests = _requests("B", seed=3)
    oracle = {rid: oracle_logits("B", ids) for rid, ids in requests.items()}
    steps = replay.mixed(requests, seed=4, max_live=2)
    pages = -(-replay.peak_tokens(steps, 8) // 8)
    core = make_core("B", "float32", PlainKernels(), "cpu", num_pages=pages, page_size=8)
    used = set()
    from atom_amd.engine.core import StepEntry
    results = {}
    for s in steps:
        logits = core.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        results[s["step"]] = logits
        for rid in core.manager.live_requests():
            used.update(p for p in core.manager.block_table(rid, 0) if p >= 0)
        for rid in s["end"]:
            core.close(rid)
    assert sum(len(v) for v in requests.values()) > pages * 8, "the pool must be smaller than what runs through it"
    replay.check(steps, results, requests, oracle, "float32", "B/reuse")


def test_layer_order_is_data():
    """A layer run twice (each run with its own cache) and a run that reads another run's cache."""
    order = [(0, None), (1, None), (1, None), (2, 1)]
    ids = random_ids("B", 45, 9)
    want = oracle_logits("B", ids, order=order)
    core = make_core("B", "float32", PlainKernels(), "cpu", order=order)
    requests = {"x": ids}
    steps = replay.portions(requests, seed=1)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, {"x": want}, "float32", "order")
    plain = oracle_logits("B", ids)
    assert (plain - want).abs().max() > 1e-3, "the changed order must change the result"


def test_a_mixer_may_refuse_a_page_size():
    """What a page size must be is the mixers' to say: the cache plan asks each of them."""
    from atom_amd.parts.attention import GroupedQueryAttention

    core = make_core("A", "float32", PlainKernels(), "cpu", page_size=6)     # attention takes any positive size
    ids = random_ids("A", 20, 1)
    from atom_amd.engine.core import StepEntry
    logits = core.step([StepEntry("a", ids, [19])])
    assert replay.first_bad({19: logits[0]}, oracle_logits("A", ids), "float32") is None

    class Picky(GroupedQueryAttention):
        def page_size_problem(self, page_size):
            return None if page_size % 32 == 0 else "this mixer's kernels read 32 keys at a time"

    core.model.blocks[1].mixer.__class__ = Picky
    try:
        with pytest.raises(ValueError, match="pages of 16 tokens do not suit layer 1 .Picky.: this mixer's kernels"):
            from atom_amd.cache.storage import plan_cache
            plan_cache(core.model, 16, torch.float32, num_pages=4)
        plan_cache(core.model, 64, torch.float32, num_pages=4)
    finally:
        core.model.blocks[1].mixer.__class__ = GroupedQueryAttention


def test_step_rejects_bad_input():
    core = make_core("A", "float32", PlainKernels(), "cpu")
    from atom_amd.engine.core import StepEntry
    with pytest.raises(ValueError):
        core.step([StepEntry("a", [CONFIGS["A"]["vocab_size"]], [0])])
    with pytest.raises(ValueError):
        core.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(ValueError):
        core.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(ValueError):
        core.step([StepEntry("a", list(range(129)), [])])   # 128 positions
    assert not core.manager.live_requests()


# ------------------------------------------------------------------ steps launched before the last one's tokens are read


def _engine(deferred, which="B", **kw):
    from helpers import tiny_folder
    from tiny import PAGE
    from atom_amd import LLMEngine

    kw.setdefault("num_kvcache_blocks", 64)
    kw.setdefault("max_num_seqs", 4)
    return LLMEngine(tiny_folder(which), dtype="fp32", ops=PlainKernels(), device="cpu",
                     kv_cache_block_size=PAGE[which], deferred_output=deferred, **kw)


def _same(a, b):
    assert [o["token_ids"] for o in a] == [o["token_ids"] for o in b]
    assert [o["finish_reason"] for o in a] == [o["finish_reason"] for o in b]
    for x, y in zip(a, b):
        assert (x["logprobs"] is None) == (y["logprobs"] is None)
        if x["logprobs"]:
            assert x["logprobs"] == pytest.approx(y["logprobs"], abs=1e-5)


def _idle(llm):
    llm.core.manager.check()
    assert llm.is_finished() and not llm.core.manager.live_requests()
    assert all(pool.num_free == pool.num_pages for pool in llm.core.manager.pools)


def test_steps_launched_ahead_change_no_token():
    """Greedy, seeded temperature and log-probabilities; requests of different lengths that leave at
    different times; more requests than run at once; so few pages that requests are preempted."""
    from atom_amd import SamplingParams

    prompts = [random_ids("B", n, 7 + n) for n in (9, 40, 23, 5, 31, 12)]
    params = [SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True),
              SamplingParams(temperature=0.7, max_tokens=20, ignore_eos=True, seed=5),
              SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True, logprobs=True),
              SamplingParams(temperature=1.0, top_k=5, max_tokens=9, ignore_eos=True, seed=2),
              SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True),
              SamplingParams(temperature=0.0, max_tokens=15, ignore_eos=True)]
    for kw in ({}, {"max_num_seqs": 2}, {"num_kvcache_blocks": 12}):
        plain, ahead = _engine(False, **kw), _engine(True, **kw)
        _same(plain.generate(prompts, params), ahead.generate(prompts, params))
        _idle(ahead)
        if "num_kvcache_blocks" in kw:
            assert ahead.scheduler.total_preemptions > 0
        else:
            assert ahead.core.steps_run == plain.core.steps_run     # counts decide these ends: no step is wasted


def test_a_request_that_ends_on_a_token_is_run_once_more_and_that_result_dropped():
    from atom_amd import SamplingParams

    prompts = [random_ids("B", n, 3 * n) for n in (9, 17, 26)]
    sp = SamplingParams(temperature=0.0, max_tokens=14, ignore_eos=True)
    free = _engine(False).generate(prompts, sp)
    eos = free[1]["token_ids"][4]
    sp = SamplingParams(temperature=0.0, max_tokens=14)
    plain, ahead = _engine(False, eos_token_id=eos), _engine(True, eos_token_id=eos)
    a, b = plain.generate(prompts, sp), ahead.generate(prompts, sp)
    _same(a, b)
    assert b[1]["finish_reason"] == "eos" and len(b[1]["token_ids"]) <= 5
    _idle(ahead)
    plain, ahead = _engine(False, eos_token_id=eos), _engine(True, eos_token_id=eos)
    _same(plain.generate(prompts[1:2], sp), ahead.generate(prompts[1:2], sp))
    assert ahead.core.steps_run == plain.core.steps_run + 1
    _idle(ahead)


def test_pages_filled_by_steps_launched_ahead_are_found_under_their_real_tokens():
    """The prefix cache names a page only once the token that a step read on the device is known."""
    from atom_amd import SamplingParams

    prompt = random_ids("B", 13, 1)
    sp = SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True)
    ahead = _engine(True)
    first = ahead.generate([prompt], sp)[0]["token_ids"]
    longer = prompt + first + random_ids("B", 6, 2)
    hits_before = ahead.core.manager.pools[0].hits
    again = ahead.generate([longer], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))[0]
    assert ahead.core.manager.pools[0].hits - hits_before == (len(prompt) + len(first) - 1) // 8
    fresh = _engine(False, enable_prefix_caching=False).generate(
        [longer], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))[0]
    assert again["token_ids"] == fresh["token_ids"]
    _idle(ahead)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_steps_launched_ahead_under_random_load(seed):
    """Requests of random lengths and token counts arrive while others run, some end on a token, the pool
    is small enough to preempt, prompts share beginnings (prefix cache): with and without steps
    launched ahead every request gets the same tokens, and the cache's books stay right after every step."""
    import random
    from atom_amd import SamplingParams

    rng = random.Random(seed)
    shared = random_ids("A", 24, 500 + seed)
    arrivals = []
    for k in range(14):
        body = random_ids("A", rng.randrange(1, 30), 600 + 20 * seed + k)
        prompt = (shared[:rng.choice([0, 16, 24])] + body)[:60]
        sp = SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8]), max_tokens=rng.randrange(1, 40), seed=k,
                            ignore_eos=rng.random() < 0.5)
        arrivals.append((rng.randrange(0, 25), prompt, sp))
    arrivals.sort(key=lambda a: a[0])

    def run(deferred):
        llm = _engine(deferred, "A", num_kvcache_blocks=6, max_num_seqs=3, eos_token_id=7, max_model_len=128,
                      stop_token_ids=list(range(0, 256, 16)))
        seqs, outputs, pending, step = {}, {}, list(arrivals), 0
        while pending or not llm.is_finished():
            while pending and pending[0][0] <= step:
                _, prompt, sp = pending.pop(0)
                seq = llm.add_request(prompt, sp)[0]
                seqs[seq.id] = len(seqs)
            for seq in llm.step():
                outputs[seqs[seq.id]] = (seq.completion_token_ids, seq.leave_reason)
            llm.core.manager.check()
            step += 1
            assert step < 2000
        _idle(llm)
        return outputs, llm

    waited, _ = run(False)
    ahead, llm = run(True)
    assert len(waited) == len(arrivals) and ahead == waited
    reasons = [reason for _, reason in ahead.values()]
    assert any(r.startswith("stop_") or r == "eos" for r in reasons) and "max_tokens" in reasons
    assert llm.scheduler.total_preemptions > 0 and llm.core.manager.pools[0].hits > 0


# ------------------------------------------------------------------ options of the entry point


def test_unknown_engine_option_is_an_error():
    from atom_amd import LLMEngine
    from helpers import tiny_folder

    with pytest.raises(TypeError, match="max_num_seq"):
        LLMEngine(tiny_folder("A"), dtype="fp32", ops=PlainKernels(), device="cpu", max_num_seq=4)


def test_n_samples_fan_out():
    """``n`` sequences of one prompt (atom/model_engine/llm_engine.py:584-720): distinct seeds give distinct
    continuations at a temperature, the same as separate requests with those seeds give; greedy gives n equal
    ones; the later sequences find the prompt's full pages in the prefix cache."""
    from atom_amd import SamplingParams

    prompt = random_ids("B", 35, 3)
    llm = _engine(True, enable_prefix_caching=True, max_num_batched_tokens=40)
    outs = llm.generate([prompt], SamplingParams(temperature=0.9, max_tokens=10, ignore_eos=True, seed=11, n=3))
    assert len(outs) == 3
    texts = [tuple(o["token_ids"]) for o in outs]
    assert len(set(texts)) == 3, "three seeds, three continuations"
    _idle(llm)
    hits = llm.core.manager.pools[0].hits
    assert hits >= 4, "the second and third sequence take the prompt's pages from the prefix cache"
    singles = _engine(True)
    for k, want in enumerate(texts):
        got = singles.generate([prompt], SamplingParams(temperature=0.9, max_tokens=10, ignore_eos=True, seed=11 + k))
        assert tuple(got[0]["token_ids"]) == want
    same = llm.generate([prompt], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True, n=2))
    assert same[0]["token_ids"] == same[1]["token_ids"]


class _WordTokenizer:
    """Token k is the text "wk "."""

    def encode(self, text, add_special_tokens=True):
        return [int(w[1:]) for w in text.split()]

    def decode(self, ids):
        return "".join(f"w{t} " for t in ids)


def test_stop_strings_end_a_request():
    """atom/model_engine/llm_engine.py:661-671, scheduler.py:2296-2312: a stop string is a token sequence;
    a request ends when its output ends in one."""
    from atom_amd import LLMEngine, SamplingParams
    from helpers import tiny_folder
    from tiny import PAGE

    def make():
        return LLMEngine(tiny_folder("B"), tokenizer=_WordTokenizer(), dtype="fp32", ops=PlainKernels(), device="cpu",
                         kv_cache_block_size=PAGE["B"], num_kvcache_blocks=64, max_num_seqs=4)

    prompt = "w5 w17 w200 w3 w9"
    free = make().generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))[0]
    ids = free["token_ids"]
    assert len(ids) == 12 and free["text"] == "".join(f"w{t} " for t in ids)
    stop = f"w{ids[5]} w{ids[6]}"
    first = next(k for k in range(1, 12) if ids[k - 1:k + 1] == ids[5:7])
    out = make().generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True,
                                                   stop_strings=[stop, "w310 w310"]))[0]
    assert out["finish_reason"] == "stop_sequence"
    assert out["token_ids"] == ids[:first + 1]


def test_abort_through_the_engine():
    from atom_amd import SamplingParams

    llm = _engine(True, max_num_seqs=2)    # the third request waits
    sp = SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True)
    keep = llm.add_request(random_ids("B", 12, 1), sp)[0]
    gone = llm.add_request(random_ids("B", 20, 2), sp)[0]
    never = llm.add_request(random_ids("B", 9, 3), sp)[0]
    finished = []
    for _ in range(6):
        finished += llm.step()
    assert gone.num_completion_tokens >= 3
    assert llm.abort(gone.id) and llm.abort(never.id) is True
    while not llm.is_finished():
        finished += llm.step()
    reasons = {s.id: s.leave_reason for s in finished}
    assert reasons == {keep.id: "max_tokens", gone.id: "aborted", never.id: "aborted"}
    assert 3 <= gone.num_completion_tokens < 30 and not gone.awaits_token and never.num_completion_tokens == 0
    assert keep.num_completion_tokens == 30
    # the request that stayed is not disturbed: the same tokens as alone
    alone = _engine(True).generate([keep.token_ids[:12]], sp)[0]
    assert alone["token_ids"] == keep.completion_token_ids
    _idle(llm)


def test_a_request_turned_away_while_steps_run_ahead_still_comes_back():
    """A request that can never run (longer than max_model_len) arrives while decode steps are launched ahead of
    each other: it is handed back at once, not when the engine runs dry."""
    from atom_amd import SamplingParams

    llm = _engine(True, max_model_len=64)
    sp = SamplingParams(temperature=0.0, max_tokens=25, ignore_eos=True)
    keep = llm.add_request(random_ids("B", 12, 1), sp)[0]
    for _ in range(4):
        llm.step()
    assert llm.steps_launched_ahead >= 2
    huge = llm.add_request(random_ids("B", 100, 2), sp)[0]
    back = []
    for _ in range(3):
        back += llm.step()
    assert [s.id for s in back] == [huge.id] and huge.leave_reason.startswith("unschedulable")
    while not llm.is_finished():
        llm.step()
    assert keep.num_completion_tokens == 25
    _idle(llm)
