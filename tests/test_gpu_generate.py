"""Generation through the entry points on the GPU: greedy against the plain implementation,
long decoding, the first tokens of a sequence, seeded temperature sampling that does not
depend on the batch, page pressure with preemption, and the command line."""

import os
import subprocess
import sys

import pytest
import torch

import plain_model as pm
from helpers import gpu_ops, oracle_weights, random_ids, tiny_folder
from tiny import CONFIGS, PAGE
from atom_amd import LLMEngine, SamplingParams
from replay import ROOT

pytestmark = pytest.mark.gpu


def engine(which, dtype, **kw):
    kw.setdefault("kv_cache_block_size", PAGE[which])
    kw.setdefault("num_kvcache_blocks", 64)
    kw.setdefault("max_num_seqs", 4)
    return LLMEngine(tiny_folder(which), dtype=dtype, ops=gpu_ops(), **kw)


def check_greedy(which, dtype, prompts, outs):
    """Every generated token is the plain implementation's argmax, or, in bfloat16, a token whose
    plain logit is within rounding of the best."""
    cfg, tensors = oracle_weights(which)
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for step, token in enumerate(out["token_ids"]):
            logits = pm.qwen3_logits(cfg, tensors, ids)[-1]
            best = int(logits.argmax())
            slack = 0.0 if dtype == "fp32" else 0.03 * float(logits.abs().max())
            assert token == best or float(logits[best] - logits[token]) <= slack, \
                f"{which}/{dtype}: token {step} of a {len(prompt)}-token prompt is {token}, plain says {best}"
            ids.append(token)


@pytest.mark.parametrize("which,dtype", [("A", "fp32"), ("B", "fp32"), ("B", "bf16"), ("C", "fp32"), ("C", "bf16"),
                                         ("D", "fp32"), ("D", "bf16")])
def test_greedy_generation_matches_plain(which, dtype):
    lens = {"A": (5, 17, 33), "B": (1, 9, 40, 71), "C": (3, 50, 120), "D": (4, 70, 300)}[which]
    prompts = [random_ids(which, n, 40 + n) for n in lens]
    llm = engine(which, dtype, max_num_batched_tokens=16 if which == "B" else 64)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8 if which == "A" else 12, ignore_eos=True))
    assert [o["num_tokens_input"] for o in outs] == list(lens)
    assert all(o["finish_reason"] == "max_tokens" and o["ttft"] > 0 and o["latency"] >= o["ttft"] for o in outs)
    check_greedy(which, dtype, prompts, outs)
    llm.core.manager.check()
    assert all(p.num_free == p.num_pages for p in llm.core.manager.pools)


def test_long_decoding_past_the_window_and_many_pages():
    """200 decoded tokens in float32: every token is the plain argmax; the window layers' pages go back meanwhile."""
    prompt = random_ids("C", 30, 7)
    llm = engine("C", "fp32", num_kvcache_blocks=20)
    out = llm.generate([prompt], SamplingParams(temperature=0.0, max_tokens=200, ignore_eos=True))[0]
    assert out["num_tokens_output"] == 200
    check_greedy("C", "fp32", [prompt], [out])


@pytest.mark.parametrize("live", [40, 100])
def test_many_requests_decode_together(live):
    """40 and 100 live requests in bfloat16: decode steps of 17 to 64 and of 65 to 128 rows (the product
    kernels for those row counts, the graph buckets above 32); every token is the plain argmax within rounding."""
    prompts = [random_ids("B", 3 + (7 * k) % 40, 300 + k) for k in range(live)]
    llm = engine("B", "bf16", max_num_seqs=128, num_kvcache_blocks=1024,
                 cudagraph_capture_sizes=[1, 2, 4, 8, 16, 32, 48, 64, 128])
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True))
    assert llm.core.graphs.replays >= 3
    picks = list(range(0, live, 7))
    check_greedy("B", "bf16", [prompts[k] for k in picks], [outs[k] for k in picks])
    llm.core.manager.check()
    assert not llm.core.manager.live_requests()


def test_first_tokens_of_a_sequence():
    """Prompts of one and two tokens: the first position has a single key, itself."""
    for which in ("A", "B"):
        for dtype in ("fp32", "bf16"):
            prompts = [[3], [7, 250 % CONFIGS[which]["vocab_size"]], [0]]
            outs = engine(which, dtype).generate(prompts, SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True))
            check_greedy(which, dtype, prompts, outs)


def test_seeded_temperature_sampling_is_reproducible_and_batch_independent():
    prompts = [random_ids("B", n, 60 + n) for n in (9, 40, 71)]
    sp = [SamplingParams(temperature=0.7, max_tokens=12, ignore_eos=True, seed=100 + k) for k in range(3)]
    together = engine("B", "fp32", max_num_batched_tokens=16).generate(prompts, sp)
    again = engine("B", "fp32", max_num_batched_tokens=64).generate(prompts, sp)
    assert [o["token_ids"] for o in together] == [o["token_ids"] for o in again]
    alone = engine("B", "fp32").generate([prompts[1]], sp[1])[0]
    assert alone["token_ids"] == together[1]["token_ids"], "a request's draws do not depend on its batch-mates"
    other = engine("B", "fp32").generate([prompts[1]], SamplingParams(temperature=0.7, max_tokens=12, ignore_eos=True, seed=999))[0]
    assert other["token_ids"] != alone["token_ids"]
    greedy = engine("B", "fp32").generate([prompts[1]], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))[0]
    topk1 = engine("B", "fp32").generate([prompts[1]], SamplingParams(temperature=0.7, top_k=1, max_tokens=12, ignore_eos=True))[0]
    assert topk1["token_ids"] == greedy["token_ids"], "top_k = 1 is greedy"


def test_sampled_tokens_follow_the_plain_race():
    """With the engine's own noise fed to the plain race, every sampled token is reproduced."""
    from plain_kernels import exponential_noise_row
    cfg, tensors = oracle_weights("B")
    prompt = random_ids("B", 20, 5)
    out = engine("B", "fp32").generate([prompt], SamplingParams(temperature=0.7, max_tokens=6, ignore_eos=True, seed=42))[0]
    ids = list(prompt)
    for k, token in enumerate(out["token_ids"]):
        logits = pm.qwen3_logits(cfg, tensors, ids)[-1:]
        noise = exponential_noise_row(42, k, cfg["vocab_size"]).unsqueeze(0)
        assert int(pm.exponential_race(logits, torch.tensor([0.7]), noise)[0]) == token
        ids.append(token)


def test_page_pressure_preempts_and_still_matches():
    """Six requests through a pool that cannot hold them all: some are preempted, prefilled again with
    what they had generated, and still produce the plain implementation's tokens."""
    prompts = [random_ids("B", n, 80 + n) for n in (30, 25, 41, 12, 36, 19)]
    llm = engine("B", "fp32", num_kvcache_blocks=14, max_num_seqs=4, max_num_batched_tokens=64)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))
    assert llm.scheduler.total_preemptions > 0, "the pool was meant to be too small"
    assert all(o["finish_reason"] == "max_tokens" and o["num_tokens_output"] == 20 for o in outs)
    check_greedy("B", "fp32", prompts, outs)
    llm.core.manager.check()


def test_stop_on_eos_and_logprobs():
    cfg, tensors = oracle_weights("B")
    prompt = random_ids("B", 9, 3)
    free = engine("B", "fp32").generate([prompt], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True, logprobs=True))[0]
    eos = free["token_ids"][3]
    first = free["token_ids"].index(eos)
    llm = engine("B", "fp32", eos_token_id=eos)
    out = llm.generate([prompt], SamplingParams(temperature=0.0, max_tokens=10))[0]
    assert out["finish_reason"] == "eos" and out["token_ids"] == free["token_ids"][:first + 1]
    lp = torch.log_softmax(pm.qwen3_logits(cfg, tensors, prompt)[-1], dim=-1)[free["token_ids"][0]]
    assert abs(free["logprobs"][0] - float(lp)) < 1e-4
    rejected = llm.generate([list(range(300))], SamplingParams(max_tokens=2))[0]
    assert rejected["finish_reason"].startswith("unschedulable")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_steps_launched_ahead_change_no_token(dtype):
    """The next decode step is launched before the host reads the last one's tokens (the default): the
    same tokens as with a wait after every step, for requests that leave by count or on a token, with
    graphs and without."""
    prompts = [random_ids("B", n, 11 * n) for n in (9, 40, 23, 5)]
    params = [SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True),
              SamplingParams(temperature=0.7, max_tokens=20, ignore_eos=True, seed=5),
              SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True, logprobs=True),
              SamplingParams(temperature=0.0, max_tokens=16, ignore_eos=True)]
    waited = engine("B", dtype, deferred_output=False).generate(prompts, params)
    check_greedy("B", dtype, [prompts[0], prompts[3]], [waited[0], waited[3]])
    eos = waited[3]["token_ids"][6]
    for kw in ({}, {"enforce_eager": True}):
        llm = engine("B", dtype, **kw)
        assert llm.deferred_output
        ahead = llm.generate(prompts, params)
        assert [o["token_ids"] for o in ahead] == [o["token_ids"] for o in waited]
        # (without graphs the keys of a decode step are split over another number of waves: other rounding)
        loose = dtype == "bf16" and bool(kw)
        assert ahead[2]["logprobs"] == pytest.approx(waited[2]["logprobs"], abs=3e-2 if loose else 1e-5)
        if not kw:
            assert llm.core.graphs.replays > 10
        llm.core.manager.check()
        assert not llm.core.manager.live_requests()
    # a request that ends on a token: one more step runs for it and is dropped
    params[3] = SamplingParams(temperature=0.0, max_tokens=16)
    a = engine("B", dtype, deferred_output=False, eos_token_id=eos).generate(prompts, params)
    llm = engine("B", dtype, eos_token_id=eos)
    b = llm.generate(prompts, params)
    assert [o["token_ids"] for o in a] == [o["token_ids"] for o in b] and b[3]["finish_reason"] == "eos"
    assert len(b[3]["token_ids"]) <= 7
    llm.core.manager.check()
    assert llm.is_finished() and not llm.core.manager.live_requests()


def test_steps_launched_ahead_under_random_load_on_the_gpu():
    """Requests of random lengths and token counts arrive while others run, some end on a token, the pool is
    small enough to preempt, prompts share beginnings (prefix cache).  In 32-bit a row's logits do not depend on
    the batch to the bit, so with and without steps launched ahead every request gets the same tokens."""
    import random

    rng = random.Random(3)
    shared = random_ids("A", 24, 700)
    arrivals = []
    for k in range(12):
        body = random_ids("A", rng.randrange(1, 30), 800 + k)
        prompt = (shared[:rng.choice([0, 16, 24])] + body)[:60]
        sp = SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8]), max_tokens=rng.randrange(1, 40), seed=k,
                            ignore_eos=rng.random() < 0.5)
        arrivals.append((rng.randrange(0, 25), prompt, sp))
    arrivals.sort(key=lambda a: a[0])

    def run(deferred):
        llm = engine("A", "fp32", num_kvcache_blocks=6, max_num_seqs=3, eos_token_id=7, max_model_len=128,
                     stop_token_ids=list(range(0, 256, 16)), deferred_output=deferred)
        seqs, outputs, pending, step = {}, {}, list(arrivals), 0
        while pending or not llm.is_finished():
            while pending and pending[0][0] <= step:
                _, prompt, sp = pending.pop(0)
                seqs[llm.add_request(prompt, sp)[0].id] = len(seqs)
            for seq in llm.step():
                outputs[seqs[seq.id]] = (seq.completion_token_ids, seq.leave_reason)
            llm.core.manager.check()
            step += 1
            assert step < 2000
        assert not llm.core.manager.live_requests()
        return outputs, llm

    waited, _ = run(False)
    ahead, llm = run(True)
    assert len(waited) == len(arrivals) and ahead == waited
    assert llm.scheduler.total_preemptions > 0 and llm.core.graphs.replays > 10


def test_mark_trace_names_the_operations_in_a_profile():
    """With mark_trace the steps' spans hold one span per operation, and the tokens do not change."""
    from atom_amd.kernels.hip import HipKernels

    prompt = random_ids("B", 20, 5)
    sp = SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True)
    plain_run = engine("B", "bf16").generate([prompt], sp)[0]["token_ids"]
    llm = LLMEngine(tiny_folder("B"), dtype="bf16", ops=HipKernels("cuda:0"), mark_trace=True, enforce_eager=True,
                    kv_cache_block_size=PAGE["B"], num_kvcache_blocks=64, max_num_seqs=4)
    with torch.profiler.profile(activities=[torch.profiler.ProfilerActivity.CPU]) as prof:
        marked_run = llm.generate([prompt], sp)[0]["token_ids"]
    assert marked_run == plain_run
    names = {e.key for e in prof.key_averages()}
    for span in ("rope_cache", "paged_attention", "rmsnorm", "linear", "linear_silu", "embedding", "sample"):
        assert span in names, (span, sorted(n for n in names if not n.startswith("aten::")))
    assert any(n.startswith("prefill[bs=1 tok=20") for n in names) and any(n.startswith("decode[bs=1") for n in names)


def test_command_line():
    cmd = [sys.executable, "-m", "atom_amd.examples.simple_inference", "--model", tiny_folder("A"), "--temperature", "0",
           "--max-tokens", "8", "--block_size", "16", "--num-kvcache-blocks", "32", "--max-num-seqs", "4", "--dtype", "fp32",
           "--seed", "3"]
    res = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert res.stdout.count("Completion:") == 3 and res.stdout.count("finish_reason=max_tokens") == 3
    import random, re
    rng = random.Random(3)
    prompts = [[rng.randrange(256) for _ in range(n)] for n in (5, 17, 33)]
    shown = [eval(m) for m in re.findall(r"Completion: (\[.*?\])", res.stdout)]
    check_greedy("A", "fp32", prompts, [{"token_ids": ids} for ids in shown])


def test_profile_offline_command(tmp_path):
    """The offline profiling command (atom/examples/profile_offline.py:12-117): a warm-up, then --bs equal random
    prompts between start_profile and stop_profile; the trace holds the steps' spans and this library's kernels."""
    import json
    from atom_amd.examples import profile_offline
    out = str(tmp_path / "traces")
    outputs = profile_offline.main(["--model", tiny_folder("C"), "--dtype", "bf16", "--block_size", str(PAGE["C"]),
                                    "--num-kvcache-blocks", "64", "--max-num-seqs", "4", "--input-length", "40",
                                    "--output-length", "5", "--bs", "3", "--random-input", "--torch-profiler-dir", out])
    assert len(outputs) == 3 and all(o["num_tokens_input"] == 40 and o["num_tokens_output"] == 5 for o in outputs)
    with open(os.path.join(out, "trace.json")) as f:
        names = {e.get("name", "") for e in json.load(f)["traceEvents"]}
    assert any(n.startswith("prefill[bs=3") for n in names) and any(n.startswith("decode[bs=3") for n in names)
    assert any("attention" in n and "kernel" in n for n in names), "no kernel of this library in the trace"


@pytest.mark.parametrize("which,dtype", [("A", "fp32"), ("B", "fp32"), ("B", "bf16")])
def test_prefix_cache_reuses_pages_and_changes_nothing(which, dtype):
    """Requests that begin alike: with the prefix cache the later ones start after the pages that hold
    their beginning; the tokens are those of an engine without it (and of the plain implementation)."""
    stem = random_ids(which, 70, 3)
    prompts = [stem, stem + random_ids(which, 9, 4), stem[:41] + random_ids(which, 20, 5), stem]
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    outs = {}
    for caching in (True, False):
        llm = engine(which, dtype, enable_prefix_caching=caching, max_num_seqs=2)
        assert llm.core.prefix_caching == caching
        outs[caching] = [llm.generate([p], sp)[0] for p in prompts[:2]] + llm.generate(prompts[2:], sp)
        llm.core.manager.check()
        pool = llm.core.manager.pools[0]
        assert pool.num_free == pool.num_pages
        if caching:
            page = PAGE[which]
            # the 2nd finds the 1st's prompt pages, the 3rd 41 tokens' worth, the 4th all but its last page
            assert pool.hits >= (70 // page) + (41 // page) + (69 // page)
        else:
            assert pool.hits == 0
    if dtype == "fp32":
        assert [o["token_ids"] for o in outs[True]] == [o["token_ids"] for o in outs[False]]
    check_greedy(which, dtype, prompts, outs[True])


def test_prefix_cache_is_off_where_a_window_gives_pages_back():
    llm = engine("C", "fp32", enable_prefix_caching=True)
    assert not llm.core.prefix_caching


def test_default_cache_sizing_fills_the_allowed_memory_and_generates():
    """``num_kvcache_blocks=-1`` (the default): the pool takes what ``gpu_memory_utilization`` leaves after the
    weights, the decode graphs and a margin (atom/model_engine/model_runner.py:1591-1611); graphs are
    captured; generation matches the plain implementation."""
    import torch

    torch.cuda.empty_cache()
    free, total = torch.cuda.mem_get_info()
    want_pool = 4 << 30
    util = min(1.0, (total - free + int(total * 0.02) + want_pool + (1 << 30)) / total)
    llm = LLMEngine(tiny_folder("D"), dtype="bf16", ops=gpu_ops(), gpu_memory_utilization=util, max_num_seqs=8,
                    max_model_len=512, cudagraph_capture_sizes=[1, 2, 4, 8], cudagraph_prefill_sizes=[])
    plan = llm.core.plan
    assert llm.config.num_kvcache_blocks == -1 and llm.config.kv_cache_block_size == 16
    assert plan.groups[0].num_pages > 8 * 512 // 16, "the pool must hold more than every slot's longest request"
    assert 0.7 * want_pool <= plan.total_bytes() <= want_pool + (1 << 30)
    free_after, _ = torch.cuda.mem_get_info()
    assert total - free_after <= util * total, "weights, cache and graphs stay inside the allowed share"
    assert llm.core.graphs is not None and sorted(llm.core.graphs.captured) == [(0, 0, n) for n in (1, 2, 4, 8)]
    prompts = [random_ids("D", n, 60 + n) for n in (5, 90, 33)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    assert llm.core.graphs.replays > 0
    check_greedy("D", "bf16", prompts, outs)
    del llm
    torch.cuda.empty_cache()
