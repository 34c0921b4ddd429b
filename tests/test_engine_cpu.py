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
