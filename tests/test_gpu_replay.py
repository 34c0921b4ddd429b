"""The engine on the GPU against the plain implementation, in float32 and bfloat16:
each request alone and whole; most of it in one step and the last 32 tokens one by one;
in portions of changing size, down to two tokens; and mixed, up to four live requests
with so few pages that they are used again.  Once in process on ``EngineCore`` and once
through ``bin/trace_run``."""

import pytest

import replay
from helpers import gpu_ops, make_core, oracle_logits, random_ids, tiny_folder
from tiny import CONFIGS

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 33, 100, 128, 64], "B": [1, 9, 40, 71, 200, 256, 130], "C": [3, 50, 600, 320, 95, 31, 257, 1000],
           "D": [2, 70, 700, 129, 33, 400], "E": [4, 37, 150, 64, 210]}


def _requests(which, seed=0):
    return {f"r{k}": random_ids(which, n, seed * 100 + k) for k, n in enumerate(LENGTHS[which])}


_ORACLE = {}


def _oracle(which, requests):
    for rid, ids in requests.items():
        key = (which, tuple(ids))
        if key not in _ORACLE:
            _ORACLE[key] = oracle_logits(which, ids)
    return {rid: _ORACLE[(which, tuple(ids))] for rid, ids in requests.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
def test_cuts_match_plain(which, cut, dtype):
    requests = _requests(which)
    oracle = _oracle(which, requests)
    steps = getattr(replay, cut)(requests)
    pages = -(-replay.peak_tokens(steps, 64) // 16)
    core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=pages, page_size=16)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, dtype, f"{which}/{cut}/{dtype}")
    assert all(pool.num_free == pool.num_pages for pool in core.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_own_page_size_and_reuse(dtype):
    """Config B with pages of 8 tokens; two live requests at a time through a pool that holds
    far less than what runs through it."""
    requests = _requests("B", seed=3)
    oracle = _oracle("B", requests)
    steps = replay.mixed(requests, seed=4, max_live=2)
    pages = -(-replay.peak_tokens(steps, 8) // 8)
    assert sum(len(v) for v in requests.values()) > 1.5 * pages * 8
    core = make_core("B", dtype, gpu_ops(), "cuda:0", num_pages=pages, page_size=8)
    results = replay.run_in_process(core, steps)
    replay.check(steps, results, requests, oracle, dtype, f"B/page8/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_float32_cuts_agree_closely(dtype):
    """The same request whole and in portions: the two runs of the engine agree far more closely
    than either agrees with the reference (the key order inside a row's sums is the same)."""
    ids = random_ids("C", 500, 77)
    requests = {"x": ids}
    core = make_core("C", dtype, gpu_ops(), "cuda:0", num_pages=64, page_size=16)
    a = replay.collect(replay.whole(requests), replay.run_in_process(core, replay.whole(requests)))["x"]
    steps = replay.portions(requests, seed=5)
    b = replay.collect(steps, replay.run_in_process(core, steps))["x"]
    worst = max(float((a[p] - b[p]).abs().max()) for p in a)
    scale = max(float(a[p].abs().max()) for p in a)
    assert worst <= (1e-5 if dtype == "float32" else 3e-2) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "C", "D"])
def test_trace_run_program(which, dtype, tmp_path):
    """``bin/trace_run`` itself: mixed trace, pool sized by --max-tokens, logits read from files."""
    requests = _requests(which, seed=1)
    if which == "C":
        requests = dict(list(requests.items())[:6])
    oracle = _oracle(which, requests)
    steps = replay.mixed(requests, seed=2)
    out = replay.run_program(tiny_folder(which), dtype, steps, str(tmp_path / "out"),
                             replay.peak_tokens(steps, 64), CONFIGS[which]["vocab_size"])
    replay.check(steps, out, requests, oracle, dtype, f"trace_run/{which}/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program_with_its_own_page_size(dtype, tmp_path):
    """``bin/trace_run --block-size 8``: config B's own pages through the program, two live requests at a
    time in a pool that holds far less than what runs through it."""
    requests = _requests("B", seed=5)
    oracle = _oracle("B", requests)
    steps = replay.mixed(requests, seed=6, max_live=2)
    peak = replay.peak_tokens(steps, 64)
    assert sum(len(v) for v in requests.values()) > 1.3 * peak      # pages are used again
    out = replay.run_program(tiny_folder("B"), dtype, steps, str(tmp_path / "out"), peak, CONFIGS["B"]["vocab_size"],
                             extra=["--block-size", "8"])
    replay.check(steps, out, requests, oracle, dtype, f"trace_run/B/page8/{dtype}")


def test_trace_run_wants_nothing(tmp_path):
    """Steps that want nothing write no file; a request may sit out steps and go on later."""
    ids = random_ids("A", 40, 5)
    other = random_ids("A", 20, 6)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids[:20], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": other, "want": [19]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "a", "tokens": ids[20:], "want": [0, 19]}], "end": ["a"]},
    ]
    out = replay.run_program(tiny_folder("A"), "float32", steps, str(tmp_path / "o"), 128, CONFIGS["A"]["vocab_size"])
    assert sorted(out) == [1, 2]
    want = oracle_logits("A", ids)
    assert replay.first_bad({20: out[2][0], 39: out[2][1]}, want, "float32") is None
    assert replay.first_bad({19: out[1][0]}, oracle_logits("A", other), "float32") is None
