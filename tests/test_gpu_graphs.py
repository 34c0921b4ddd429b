"""Decode-only steps replayed as HIP graphs: the same traces as the eager engine against the
plain implementation, and a graph replayed several times, with eager steps of other requests
between the replays, against the eager result of the same step."""

import pytest
import torch

import replay
from helpers import gpu_ops, make_core, oracle_logits, random_ids
from atom_amd.engine.core import StepEntry

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [40, 17, 90, 128], "B": [1, 9, 71, 200, 130], "C": [50, 600, 95, 257], "D": [45, 500, 130, 260], "E": [33, 150, 64, 210]}


def _requests(which):
    return {f"g{k}": random_ids(which, n, 900 + k) for k, n in enumerate(LENGTHS[which])}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("cut", ["tail", "mixed"])
def test_graph_cuts_match_plain(which, cut, dtype):
    requests = _requests(which)
    oracle = {rid: oracle_logits(which, ids) for rid, ids in requests.items()}
    steps = replay.tail(requests) if cut == "tail" else replay.mixed(requests, seed=8, decode_tail=20)
    pages = -(-replay.peak_tokens(steps, 64) // 16)
    core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=pages, page_size=16, graph_sizes=[1, 2, 4])
    assert core.graphs is not None
    results = replay.run_in_process(core, steps)
    assert core.graphs.replays >= 20, "the decode steps of this trace should have been replayed graphs"
    replay.check(steps, results, requests, oracle, dtype, f"graph/{which}/{cut}/{dtype}")


ORDERS = {"C": [(0, None), (1, None), (1, None), (2, 1), (3, 0)],   # a windowed and a full run that read
          "D": [(0, None), (1, None), (1, None), (0, 0)]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["C", "D"])
@pytest.mark.parametrize("cut", ["tail", "mixed"])
def test_an_order_whose_runs_share_and_read_caches(which, cut, dtype):
    """The running order as data, on the GPU kernels and through replayed graphs: a layer run twice, each run
    with a cache of its own, and runs that read an earlier run's cache and write none (in the decode steps of
    few rows that is the kernel that norms, rotates, writes and attends in one, with its write switched off)."""
    order = ORDERS[which]
    requests = _requests(which)
    oracle = {rid: oracle_logits(which, ids, order=order) for rid, ids in requests.items()}
    first = next(iter(requests))
    assert (oracle_logits(which, requests[first]) - oracle[first]).abs().max() > 1e-3, "the order must matter"
    steps = replay.tail(requests) if cut == "tail" else replay.mixed(requests, seed=11, decode_tail=20)
    pages = -(-replay.peak_tokens(steps, 64) // 16)
    core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=pages, page_size=16, graph_sizes=[1, 2, 4],
                     order=order)
    assert core.graphs is not None
    results = replay.run_in_process(core, steps)
    assert core.graphs.replays >= 20
    replay.check(steps, results, requests, oracle, dtype, f"order/{which}/{cut}/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_that_do_not_divide_the_longest_context(dtype):
    """Pages of 24 tokens and 2,048 positions: the graphs' block tables name more positions than the rotation
    tables hold, which must refuse no capture and change no logit."""
    which = "D"
    requests = {f"q{k}": random_ids(which, n, 300 + k) for k, n in enumerate([50, 131, 75])}
    oracle = {rid: oracle_logits(which, ids) for rid, ids in requests.items()}
    steps = replay.tail(requests)
    pages = -(-replay.peak_tokens(steps, 72) // 24)
    core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=pages, page_size=24, graph_sizes=[1, 2])
    assert core.graphs is not None and core.graphs.widths[0] * 24 > 2048
    results = replay.run_in_process(core, steps)
    assert core.graphs.replays >= 90
    replay.check(steps, results, requests, oracle, dtype, f"page24/{dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["B", "C", "D"])
def test_steps_with_prompt_portions_replayed_as_graphs(which, dtype):
    """Steps as a scheduler under a small budget makes them (one or two prompt portions beside single tokens)
    run as replayed graphs of fixed shape, padded in both parts, and give the plain implementation's logits."""
    lengths = {"B": [30, 71, 200, 130, 12, 90], "C": [50, 400, 95, 257, 31, 140], "D": [45, 300, 130, 260, 20]}[which]
    requests = {f"m{k}": random_ids(which, n, 500 + k) for k, n in enumerate(lengths)}
    oracle = {rid: oracle_logits(which, ids) for rid, ids in requests.items()}
    steps = replay.scheduled(requests, seed=3, max_live=4, budget=100)
    pages = -(-replay.peak_tokens(steps, 64) // 16)
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model
    from helpers import tiny_folder

    model, _ = load_model(tiny_folder(which), dtype=TORCH_DTYPES[dtype], device="cuda:0")
    core = build_core(model, gpu_ops(), dtype=TORCH_DTYPES[dtype], device="cuda:0", page_size=16, num_pages=pages,
                      max_num_seqs=8, graph_sizes=[1, 2, 4, 8], graph_prefill_sizes=[48, 128])
    results = replay.run_in_process(core, steps)
    mixed = sum(1 for s in steps if any(len(e["tokens"]) > 1 for e in s["entries"]))
    assert mixed >= 6 and core.graphs.mixed_replays == mixed, "every step with a prompt portion fits a bucket here"
    assert {shape[0] for shape in core.graphs.captured} >= {0, 48, 128}
    replay.check(steps, results, requests, oracle, dtype, f"mixed graph/{which}/{dtype}", every=False)
    # the same steps eagerly: the same logits within rounding
    eager = build_core(model, gpu_ops(), dtype=TORCH_DTYPES[dtype], device="cuda:0", page_size=16, num_pages=pages,
                       max_num_seqs=8)
    plain = replay.run_in_process(eager, steps)
    tol = (1e-5 if dtype == "float32" else 3e-2)
    for k in results:
        scale = float(plain[k].abs().max())
        assert float((results[k] - plain[k]).abs().max()) <= tol * scale, f"step {k}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("live,bucket", [(3, 4), (27, 32)])
def test_replays_agree_with_eager(dtype, live, bucket):
    """Requests decode together through one graph (with padding rows) for 12 steps; in between, another
    request runs eager prompt portions.  An eager engine runs the same steps.  With 27 rows the bfloat16
    products inside the graph are the BLAS library's, with 3 the engine's own."""
    which = "C"
    prompts = {f"p{k}": random_ids(which, n, 40 + k) for k, n in enumerate(([33, 70, 150] * 9)[:live])}
    tails = {rid: random_ids(which, 12, 60 + k) for k, rid in enumerate(prompts)}
    other = random_ids(which, 200, 99)

    def run(graph_sizes):
        core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=64 + 12 * live, page_size=16,
                         max_num_seqs=max(live + 1, bucket), graph_sizes=graph_sizes)
        for rid, ids in prompts.items():
            core.step([StepEntry(rid, ids, [])])
        outs = []
        for t in range(12):
            logits = core.step([StepEntry(rid, [tails[rid][t]], [0]) for rid in prompts])
            outs.append(logits.cpu())
            core.step([StepEntry("other", other[16 * t:16 * t + 16], [15])])   # eager work between replays
            torch.cuda.synchronize()
        return outs, core

    eager, _ = run(None)
    graphed, core = run([bucket])
    assert core.graphs.replays == 12
    scale = max(float(e.abs().max()) for e in eager)
    tol = 1e-5 if dtype == "float32" else 2e-2
    for t, (e, g) in enumerate(zip(eager, graphed)):
        assert torch.isfinite(g).all()
        assert float((e - g).abs().max()) <= tol * scale, f"replay {t} differs from the eager step"


def test_stateful_mixer_is_not_graphed():
    """A model is replayed only if all its mixers declare themselves graph safe."""
    from atom_amd.parts.base import Mixer

    assert Mixer.graph_safe is False
    core = make_core("A", "float32", gpu_ops(), "cuda:0", graph_sizes=[1, 2])
    assert core.graphs is not None and core.graphs.usable
    core.model.blocks[0].mixer.graph_safe = False
    try:
        from atom_amd.engine.graphs import DecodeGraphs

        assert not DecodeGraphs(core, [1, 2], 128).usable
    finally:
        del core.model.blocks[0].mixer.graph_safe


@pytest.mark.parametrize("graph_sizes", [None, [4]])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_read_on_the_device(dtype, graph_sizes):
    """A step whose entries name rows of the sampler's output instead of tokens gives the logits of the
    step that is handed the same tokens by the host; rows are taken in any order, and a step may mix both."""
    which = "B"
    prompts = {f"f{k}": random_ids(which, n, 70 + k) for k, n in enumerate([20, 9, 33])}
    nxt = {"f0": 5, "f1": 300, "f2": 17}

    def run(fed: dict):
        core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=32, page_size=8, graph_sizes=graph_sizes)
        for rid, ids in prompts.items():
            core.step([StepEntry(rid, ids, [])])
        core.sampled[:4] = torch.tensor([nxt["f2"], 0, nxt["f0"], nxt["f1"]], dtype=torch.int32, device="cuda:0")
        rows = {"f2": 0, "f0": 2, "f1": 3}
        entries = [StepEntry(rid, [0] if rid in fed else [nxt[rid]], [0], None, rows[rid] if rid in fed else None)
                   for rid in prompts]
        out = core.step(entries).cpu()
        if graph_sizes:
            assert core.graphs.replays == 1
        return out

    given = run({})
    assert torch.equal(run({"f0", "f1", "f2"}), given)
    assert torch.equal(run({"f1"}), given)
    # and beside a prompt portion, where the step is not a graph's
    core = make_core(which, dtype, gpu_ops(), "cuda:0", num_pages=32, page_size=8, graph_sizes=graph_sizes)
    core.step([StepEntry("f0", prompts["f0"], [])])
    core.sampled[1] = nxt["f0"]
    mixed = core.step([StepEntry("f0", [0], [0], None, 1), StepEntry("f2", prompts["f2"], [])])
    torch.testing.assert_close(mixed.cpu()[0], given[0], rtol=0, atol=(1e-4 if dtype == "float32" else 3e-2) * float(given.abs().max()))
    with pytest.raises(ValueError):
        core.step([StepEntry("f0", [0, 0], [0], None, 1)])
