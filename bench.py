#!/usr/bin/python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 8b|4b|32b]

The default run has the layer sizes of Qwen3-8B (36 layers, hidden 4096, 32/8 heads of
128, intermediate 12288, vocabulary 151936) with seeded random bfloat16 weights, 8
sequences of 2,048 random prompt tokens each, and times K decode steps through the
engine's own step loop (scheduler, step function, sampler).  ``value`` is decoded tokens
a second.  It also times one 2,048-token prefill and decoding at batch 1 and 64, and
prints one JSON line.  More than one GPU is not built: ``--gpus N>1`` says so and exits 2.

With no ``--shape`` the same run goes on to the other shapes' workloads (below), the reference's two
single-stream pairs, and the 8B shape at 16,384 and 32,768 tokens of context, and adds their records
under ``shapes`` (their headline numbers also under ``points``).

``--shape 4b`` runs the Qwen3-4B shape (hidden 2560 under 32 heads of 128, tied head) on its
workload: 32 requests with prompts of 64 to 3,072 tokens through the scheduler, prompt portions
of 512 tokens beside the running requests' decode tokens, 128 output tokens each.
``--shape 32b`` runs the Qwen3-32B shape (64 layers, 65 GB of weights) on its workload:
8,192-token prompts prefilled in portions, then 16 requests decoding 256 tokens, with the
cache pool sized from the memory that is left (``num_kvcache_blocks=-1``).  Each prints one
JSON line of the same form.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12                       # bytes/s, MI355X HBM3E
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense flop/s

QWEN3_8B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36, hidden_size=4096,
    num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=40960, tie_word_embeddings=False,
    attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")


QWEN3_4B = dict(QWEN3_8B, hidden_size=2560, intermediate_size=9728, tie_word_embeddings=True)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
SHAPES = {"8b": ("Qwen3-8B", QWEN3_8B, 2), "4b": ("Qwen3-4B", QWEN3_4B, 3), "32b": ("Qwen3-32B", QWEN3_32B, 4)}


def weight_bytes(c: dict, layers: int, elem: int = 2) -> int:
    """Bytes of every weight a decode step reads once: the layers' matrices and the head."""
    h, d = c["hidden_size"], c["head_dim"]
    hq, hkv, inter = c["num_attention_heads"], c["num_key_value_heads"], c["intermediate_size"]
    per_layer = h * (hq + 2 * hkv) * d + hq * d * h + 2 * inter * h + inter * h
    norms = (2 * h + 2 * d) * 4 // elem
    return (layers * (per_layer + norms) + c["vocab_size"] * h) * elem


def kv_bytes_per_token(c: dict, layers: int, elem: int = 2) -> int:
    return 2 * layers * c["num_key_value_heads"] * c["head_dim"] * elem


def prefill_flops(c: dict, layers: int, tokens: int) -> float:
    h, d = c["hidden_size"], c["head_dim"]
    hq, hkv, inter = c["num_attention_heads"], c["num_key_value_heads"], c["intermediate_size"]
    per_layer = h * (hq + 2 * hkv) * d + hq * d * h + 3 * inter * h
    gemm = 2.0 * tokens * layers * per_layer
    attn = layers * 2.0 * 2.0 * hq * d * tokens * (tokens + 1) / 2     # QK^T and PV over the causal half
    head = 2.0 * c["vocab_size"] * h
    return gemm + attn + head


def flat_config(name: str, raw: dict, layers: int, **more) -> dict:
    """Every size of the run, flat (at most 20 keys)."""
    cfg = {"model": f"{name} shape, random weights", "parallelism": "single GPU", "layers": layers,
           "layers_of_model": raw["num_hidden_layers"], "hidden_size": raw["hidden_size"],
           "num_attention_heads": raw["num_attention_heads"], "num_key_value_heads": raw["num_key_value_heads"],
           "head_dim": raw["head_dim"], "intermediate_size": raw["intermediate_size"], "vocab_size": raw["vocab_size"],
           "tied_head": raw["tie_word_embeddings"], "kv_block_size": 16}
    cfg.update(more)
    assert len(cfg) <= 20
    return cfg


class ByteCounter:
    """Wraps the step function: adds up what every step has to read at least, the weights once and the
    cache of the requests in it, and the steps' matrix-product flops."""

    def __init__(self, core, raw, layers):
        self.core, self.inner = core, core.step
        self.weights = weight_bytes(raw, layers)
        self.kv = kv_bytes_per_token(raw, layers)
        h, d = raw["hidden_size"], raw["head_dim"]
        hq, hkv, inter = raw["num_attention_heads"], raw["num_key_value_heads"], raw["intermediate_size"]
        self.flops_per_token = 2.0 * layers * (h * (hq + 2 * hkv) * d + hq * d * h + 3 * inter * h)
        self.head_flops = 2.0 * raw["vocab_size"] * h
        self.attn_flops_per_pair = 4.0 * layers * hq * d
        self.reset()
        core.step = self.step

    def reset(self):
        self.bytes = self.flops = 0.0
        self.steps = self.tokens = 0

    def step(self, entries):
        for e in entries:
            before = self.core.num_cached(e.req_id)
            n = len(e.tokens)
            self.bytes += (before + n) * self.kv
            self.flops += n * self.flops_per_token + len(e.want) * self.head_flops
            self.flops += self.attn_flops_per_pair * (n * before + n * (n + 1) / 2)
            self.tokens += n
        self.bytes += self.weights
        self.steps += 1
        return self.inner(entries)


def run_mixed(llm, args, name, raw, layers, gen, requests: int) -> dict:
    """Continuous batching under load: every step holds the running requests' decode tokens and, under a
    budget of 512 + N tokens, the next portion of a waiting prompt."""
    import torch
    from atom_amd import SamplingParams

    vocab = raw["vocab_size"]
    sp = SamplingParams(temperature=0.0, max_tokens=128, ignore_eos=True)
    warm = [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in (700, 90)]
    llm.generate(warm, SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))   # untimed: first-use work
    lens = torch.randint(64, 3073, (requests,), generator=gen).tolist()
    prompts = [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in lens]
    counter = ByteCounter(llm.core, raw, layers)
    torch.cuda.synchronize()
    t = time.perf_counter()
    outs = llm.generate(prompts, sp)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t
    assert all(o["num_tokens_output"] == 128 for o in outs)
    out_tokens = 128 * requests
    return {
        "metric": f"output tok/s of {requests} mixed requests, prompt portions of 512 beside decodes ({name}, bf16)",
        "value": round(out_tokens / elapsed, 1), "unit": "tokens/s", "n_gpus": 1, "steps": counter.steps, "warmup": 0,
        "ms_per_step": round(elapsed / counter.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: seeded uniform random token ids and prompt lengths, seeded random N(0, 0.02) weights",
        "config": flat_config(name, raw, layers, global_batch=requests, seq_len=3072, prompt_tokens=sum(lens),
                              output_tokens=out_tokens, portion=512, max_model_len=llm.config.max_model_len,
                              hip_graphs=not args.enforce_eager),
        "roofline": {"bound": "hbm", "achieved": round(counter.bytes / elapsed / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(counter.bytes / elapsed / HBM_PEAK, 4)},
        "mfma_frac": round(counter.flops / elapsed / MFMA_PEAK["bf16"], 4),
        "total_tok_s": round((sum(lens) + out_tokens) / elapsed, 1), "seconds": round(elapsed, 3),
        "preemptions": llm.scheduler.total_preemptions, "steps_launched_ahead": llm.steps_launched_ahead,
        "graph_replays": llm.core.graphs.replays if llm.core.graphs else 0,
        "mean_ttft_ms": round(1e3 * sum(o["ttft"] for o in outs) / len(outs), 1),
        "mean_tpot_ms": round(1e3 * sum(o["tpot"] for o in outs) / len(outs), 2),
    }


def run_single(llm, args, name, raw, layers, gen, pairs) -> dict:
    """One request at a time: time to the first token, time per output token and output tokens a second as
    the reference prints them for its single-stream runs (atom/model_engine/llm_engine.py:735-744: TTFT =
    first token - arrival, TPOT = (leave - first token) / (output tokens - 1)), for its own input / output lengths
    (recipes/Qwen3-8B-FP8.md:69-73: 18 / 80 and 549 / 256)."""
    import torch
    from atom_amd import SamplingParams

    vocab = raw["vocab_size"]
    llm.generate([torch.randint(0, vocab, (64,), generator=gen).tolist()],
                 SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))   # untimed: first-use work
    rows = {}
    for isl, osl in pairs:
        best = None
        for _ in range(3):
            p = torch.randint(0, vocab, (isl,), generator=gen).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            out = llm.generate([p], SamplingParams(temperature=0.0, max_tokens=osl, ignore_eos=True))[0]
            torch.cuda.synchronize()
            wall = time.perf_counter() - t
            if best is None or wall < best[0]:
                best = (wall, out)
        wall, out = best
        rows[f"isl{isl}_osl{osl}"] = {"ttft_ms": round(out["ttft"] * 1e3, 2), "tpot_ms": round(out["tpot"] * 1e3, 3),
                                      "output_tok_s": round(osl / wall, 1)}
        print(f"[bench] single stream, {isl} in / {osl} out: {rows[f'isl{isl}_osl{osl}']}", file=sys.stderr, flush=True)
    isl, osl = pairs[-1]
    last = rows[f"isl{isl}_osl{osl}"]
    return {
        "metric": f"single-stream output tok/s, {isl} tokens in / {osl} out ({name}, bf16)",
        "value": last["output_tok_s"], "unit": "tokens/s", "n_gpus": 1, "steps": osl, "warmup": 0,
        "ms_per_step": last["tpot_ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: seeded uniform random token ids, seeded random N(0, 0.02) weights",
        "config": flat_config(name, raw, layers, global_batch=1, seq_len=isl + osl, hip_graphs=not args.enforce_eager,
                              deferred_output=not args.no_deferred_output),
        "single_stream": rows,
    }


def run_long(llm, args, name, raw, layers, gen, batch: int = 16, prompt_len: int = 8192, out_tokens: int = 256) -> dict:
    """Long prompts prefilled in portions of the token budget, then the whole batch decodes."""
    import torch
    from atom_amd import SamplingParams

    vocab = raw["vocab_size"]
    llm.generate([torch.randint(0, vocab, (600,), generator=gen).tolist()],
                 SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))            # untimed: first-use work
    sp = SamplingParams(temperature=0.0, max_tokens=out_tokens, ignore_eos=True)
    for _ in range(batch):
        llm.add_request(torch.randint(0, vocab, (prompt_len,), generator=gen).tolist(), sp)
    counter = ByteCounter(llm.core, raw, layers)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while any(s.num_completion_tokens == 0 for s in llm.seqs.values()):
        llm.step()
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    prefill_steps, prefill_flops = counter.steps, counter.flops
    print(f"[bench] {batch} prompts of {prompt_len} tokens prefilled in {t_prefill:.2f} s, {prefill_steps} steps",
          file=sys.stderr, flush=True)
    for _ in range(args.warmup):
        llm.step()
    torch.cuda.synchronize()
    assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
    steps = min(args.steps, out_tokens - args.warmup - batch - 8)
    counter.reset()
    t = time.perf_counter()
    for _ in range(steps):
        llm.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t
    assert len(llm.scheduler.running) == batch, "a request finished inside the timed steps"
    step_bytes = counter.bytes / counter.steps
    while not llm.is_finished():
        llm.step()
    llm.seqs.clear()
    pool = llm.core.plan.groups[0]
    return {
        "metric": f"decode tok/s at batch {batch} after {prompt_len}-token prompts ({name}, bf16)",
        "value": round(batch * steps / elapsed, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic: seeded uniform random token ids, seeded random N(0, 0.02) weights",
        "config": flat_config(name, raw, layers, global_batch=batch, seq_len=prompt_len, max_model_len=llm.config.max_model_len,
                              portion=llm.config.max_num_batched_tokens, cache_pages=pool.num_pages,
                              cache_gb=round(llm.core.plan.total_bytes() / 1e9, 1), hip_graphs=not args.enforce_eager),
        "prefill": {"value": round(batch * prompt_len / t_prefill, 1), "tokens": batch * prompt_len,
                    "ms": round(t_prefill * 1e3, 1), "frac": round(prefill_flops / t_prefill / MFMA_PEAK["bf16"], 4)},
        "roofline": {"bound": "hbm", "achieved": round(step_bytes * steps / elapsed / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(step_bytes * steps / elapsed / HBM_PEAK, 4)},
    }


def make_engine(args, shape_key: str, *, max_seqs: int, max_model_len: int, pages: int, budget: int, layers=None):
    """The engine on a shape's sizes with seeded random weights; returns (engine, name, raw config, layers, generator)."""
    import torch

    from atom_amd import LLMEngine
    from atom_amd.config import model_config_from_dict

    name, shape, seed = SHAPES[shape_key]
    raw = dict(shape)
    layers = layers or raw["num_hidden_layers"]
    raw["num_hidden_layers"] = layers
    t0 = time.time()
    llm = LLMEngine(f"{name.lower()}-random", model_config=model_config_from_dict(raw), load_dummy="random", seed=seed,
                    dtype="bf16", max_model_len=max_model_len, kv_cache_block_size=16, num_kvcache_blocks=pages,
                    max_num_seqs=max_seqs, max_num_batched_tokens=budget, enforce_eager=args.enforce_eager,
                    deferred_output=not args.no_deferred_output,
                    cudagraph_capture_sizes=[s for s in (1, 2, 4, 8, 16, 32, 48, 64, 128, 256) if s <= max_seqs])
    torch.cuda.synchronize()
    print(f"[bench] {name} shape ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    raw["num_hidden_layers"] = SHAPES[shape_key][1]["num_hidden_layers"]
    return llm, name, raw, layers, torch.Generator().manual_seed(seed)


def release(llm) -> None:
    """Gives an engine's device memory (weights, cache, graphs) back before the next one is built."""
    import gc

    import torch

    if llm.core.graphs is not None:
        llm.core.graphs.captured.clear()
    llm.core = llm.model = llm.scheduler = llm.sampler = None
    gc.collect()
    torch.cuda.empty_cache()


def time_prefill(llm, raw, layers, gen, tokens: int, repeats: int = 3) -> dict:
    """One prompt of ``tokens`` tokens through ``generate`` with one output token: the best of ``repeats``."""
    import torch
    from atom_amd import SamplingParams

    sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
    vocab = raw["vocab_size"]
    llm.generate([torch.randint(0, vocab, (tokens,), generator=gen).tolist()], sp)   # warm-up: library autotuning
    times = []
    for _ in range(repeats):
        p = torch.randint(0, vocab, (tokens,), generator=gen).tolist()
        torch.cuda.synchronize()
        t = time.perf_counter()
        llm.generate([p], sp)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
    best = min(times)
    flops = prefill_flops(raw, layers, tokens)
    return {"value": round(tokens / best, 1), "tokens": tokens, "ms": round(best * 1e3, 3),
            "frac": round(flops / best / MFMA_PEAK["bf16"], 4)}


def time_decode(llm, args, raw, gen, batch: int, context: int, steps: int, warmup: int):
    """``batch`` requests of ``context`` random prompt tokens, prefilled untimed, then ``steps`` timed decode steps
    through the engine's own loop.  Returns (seconds, context length at the first timed step)."""
    import torch
    from atom_amd import SamplingParams

    # prompts are admitted over several steps, so the first requests are some tokens ahead of the last
    # when all decode: leave room, so that none finishes (and the batch does not shrink) while timed
    admission_steps = -(-batch * context // llm.config.max_num_batched_tokens) + batch
    sp = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, seed=1,
                        max_tokens=steps + warmup + admission_steps + 2, ignore_eos=True)
    for _ in range(batch):
        llm.add_request(torch.randint(0, raw["vocab_size"], (context,), generator=gen).tolist(), sp)
    while any(s.num_completion_tokens == 0 for s in llm.seqs.values()):   # prompts, untimed
        llm.step()
    for _ in range(warmup):
        llm.step()
    torch.cuda.synchronize()
    assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
    start_ctx = next(iter(llm.seqs.values())).num_tokens
    t = time.perf_counter()
    for _ in range(steps):
        llm.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t
    assert len(llm.scheduler.running) == batch, "a request finished inside the timed steps"
    while not llm.is_finished():
        llm.step()
    llm.seqs.clear()
    return elapsed, start_ctx


def decode_roofline(raw, layers, batch, ctx0, steps, elapsed) -> dict:
    step_bytes = weight_bytes(raw, layers) + batch * (ctx0 + steps / 2) * kv_bytes_per_token(raw, layers)
    achieved = step_bytes * steps / elapsed
    return {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK, 4)}


def run_long_context(args, contexts=(16384, 32768), batch: int = 8, prefill_tokens: int = 16384) -> dict:
    """The 8B shape far from the headline's context: decode at ``batch`` requests of 16,384 and 32,768 tokens each,
    and one prompt of 16,384 tokens prefilled in one step."""
    longest = max(contexts)
    max_model_len = longest + 1024
    llm, name, raw, layers, gen = make_engine(args, "8b", max_seqs=batch, max_model_len=max_model_len,
                                              pages=batch * max_model_len // 16, budget=16384)
    out = {"config": flat_config(name, raw, layers, global_batch=batch, seq_len=longest, max_model_len=max_model_len,
                                 hip_graphs=not args.enforce_eager), "decode": {}}
    steps = min(args.steps, 32)
    for context in contexts:
        elapsed, ctx0 = time_decode(llm, args, raw, gen, batch, context, steps, args.warmup)
        roof = decode_roofline(raw, layers, batch, ctx0, steps, elapsed)
        out["decode"][f"ctx{context}"] = {"value": round(batch * steps / elapsed, 1), "ms_per_step": round(elapsed / steps * 1e3, 4),
                                          "roofline": roof}
        print(f"[bench] decode batch {batch} at context {context}: {elapsed / steps * 1e3:.3f} ms/step, "
              f"{roof['frac']} of the HBM peak", file=sys.stderr, flush=True)
    last = out["decode"][f"ctx{longest}"]
    out["ms_per_step"], out["roofline"] = last["ms_per_step"], last["roofline"]
    out["prefill"] = time_prefill(llm, raw, layers, gen, prefill_tokens, repeats=2)
    print(f"[bench] prefill {out['prefill']}", file=sys.stderr, flush=True)
    release(llm)
    return out


def graph_time(fn, variants, reps: int = 3) -> float:
    """Microseconds a call of ``fn(v)`` takes, from a HIP graph that calls it once for every v in ``variants``
    (different weights, so that no call finds its operands in a cache), replayed ``reps`` times."""
    import torch

    stream, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        for v in variants[:2]:
            fn(v)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for v in variants:
                fn(v)
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * len(variants))


def run_products(args) -> dict:
    """The four matrix products of a layer of the chosen shape, alone, at the given numbers of rows: the engine's
    ``linear`` (whatever kernel it picks, a product left as a sum of slices counted as it is) beside the BLAS
    library's.  No model is built."""
    import torch
    from atom_amd.kernels.hip import HipKernels

    name, raw, _ = SHAPES[args.shape or "8b"]
    h, d = raw["hidden_size"], raw["head_dim"]
    hq, hkv, inter = raw["num_attention_heads"], raw["num_key_value_heads"], raw["intermediate_size"]
    products = [("qkv", (hq + 2 * hkv) * d, h), ("o", h, hq * d), ("gate_up", 2 * inter, h), ("down", h, inter)]
    ops = HipKernels("cuda:0")
    rows = [int(v) for v in args.products.split(",")]
    table = {}
    for label, n, k in products:
        copies = max(2, int(2e9 // (n * k * 2)))
        ws = [torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        for m in rows:
            x = torch.randn(m, k, device="cuda:0", dtype=torch.bfloat16)
            ours = graph_time(lambda w: ops.linear(x, w, None, defer=True), ws)
            lib = graph_time(lambda w: torch.nn.functional.linear(x, w), ws)
            flops = 2.0 * m * n * k
            table[f"{label}_m{m}"] = {"us": round(ours, 1), "library_us": round(lib, 1),
                                      "tflops": round(flops / ours / 1e6, 1), "weights_gb_s": round(n * k * 2 / ours / 1e3, 1)}
            print(f"[bench] {label:8s} [{n} x {k}] {m:5d} rows: {ours:7.1f} us ({flops / ours / 1e6:6.1f} TFLOP/s, weights at "
                  f"{n * k * 2 / ours / 1e6:4.2f} TB/s); BLAS library {lib:7.1f} us", file=sys.stderr, flush=True)
        del ws
    return {"metric": f"matrix products of a layer alone ({name} shape, bf16)", "unit": "us", "n_gpus": 1, "dtype": "bf16",
            "products": table}


def run_attention(args) -> dict:
    """Prefill attention alone: one request brings T tokens behind C cached ones, for every "T,C" pair given."""
    import torch
    from atom_amd.kernels.hip import AttentionMeta, HipKernels

    name, raw, _ = SHAPES[args.shape or "8b"]
    hq, hkv, d, page = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"], 16
    ops, dev = HipKernels("cuda:0"), "cuda:0"
    table = {}
    for pair in args.attention.split(";"):
        t, cached = (int(v) for v in pair.split(","))
        ctx = t + cached
        pages = -(-ctx // page)
        q = torch.randn(t, hq, d, device=dev, dtype=torch.bfloat16)
        kc = torch.randn(pages, hkv, page, d, device=dev, dtype=torch.bfloat16)
        vc = torch.randn(pages, hkv, d, page, device=dev, dtype=torch.bfloat16)
        out = torch.empty_like(q)

        def tiles_of(rows):
            starts = sorted(range(0, t, rows), reverse=True)
            return torch.tensor([(0, r0) for r0 in starts], dtype=torch.int32, device=dev).view(-1, 2)

        short, tall = ops.attention_tile_rows(torch.bfloat16, d, page, hq // hkv, t)
        meta = AttentionMeta(token_seq=torch.zeros(t, dtype=torch.int32, device=dev),
                             positions=torch.arange(cached, ctx, dtype=torch.int32, device=dev),
                             block_tables=torch.arange(pages, dtype=torch.int32, device=dev).view(1, -1),
                             cu_seqlens_q=torch.tensor([0, t], dtype=torch.int32, device=dev),
                             context_lens=torch.tensor([ctx], dtype=torch.int32, device=dev), num_seqs=1, num_tokens=t,
                             max_q_len=t, max_context_len=ctx, page_size=page, num_prefill=1,
                             prefill_tiles=tiles_of(short), rows_per_tile=short,
                             tiles_by_rows={tall: tiles_of(tall)} if tall else None)
        us = graph_time(lambda _: ops.paged_attention(q, kc, vc, out, meta, d ** -0.5), [0] * 8)
        flops = 4.0 * (t * cached + t * (t + 1) / 2) * d * hq
        table[f"t{t}_c{cached}"] = {"us": round(us, 1), "tflops": round(flops / us / 1e6, 1),
                                    "frac": round(flops / us / 1e6 / (MFMA_PEAK["bf16"] / 1e12), 4)}
        print(f"[bench] prefill attention, {t} tokens behind {cached} cached: {us:8.1f} us, {flops / us / 1e6:6.1f} TFLOP/s",
              file=sys.stderr, flush=True)
    return {"metric": f"prefill attention alone ({name} heads, bf16)", "unit": "us", "n_gpus": 1, "dtype": "bf16",
            "attention": table}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", choices=sorted(SHAPES), default=None,
                    help="8b: decode at batch 8 (and 1, 64) and a 2,048-token prefill; 4b: 32 mixed requests; "
                         "32b: 8,192-token prompts in portions, then decode at batch 16 with the cache sized from memory; "
                         "not given: the 8b run, and the other shapes' workloads beside it under 'shapes'")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--max-model-len", type=int, default=None,
                    help="positions a request may reach (default: 4096, or twice a longer --context)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--points", type=str, default="1,64", help="other decode batch sizes to time")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--mixed", type=int, default=0, metavar="N",
                    help="the mixed workload with N requests on the chosen shape (what --shape 4b runs with 32)")
    ap.add_argument("--decode", action="store_true",
                    help="the prefill and decode points (what --shape 8b runs) on the chosen shape, whatever its own workload")
    ap.add_argument("--single", type=str, default="", metavar="ISL,OSL[;ISL,OSL]",
                    help="one request at a time: TTFT, TPOT and output tok/s, e.g. '18,80;549,256' (the reference's own pairs)")
    ap.add_argument("--products", type=str, default="", metavar="ROWS[,ROWS]",
                    help="no model: the four products of a layer of the shape alone at these numbers of rows, the "
                         "engine's kernels beside the BLAS library's")
    ap.add_argument("--attention", type=str, default="", metavar="T,C[;T,C]",
                    help="no model: prefill attention alone, T tokens of one request behind C cached ones")
    ap.add_argument("--budget", type=int, default=None,
                    help="the scheduler's token budget of a step (mixed: 512 + N by default, so that portions stay 512)")
    ap.add_argument("--temperature", type=float, default=0.0, help="of the decode steps' sampling (0: greedy)")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--enforce-eager", action="store_true")
    ap.add_argument("--no-deferred-output", action="store_true",
                    help="read every step's tokens before the next step is launched")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not built")
        return 2

    import logging

    logging.basicConfig(level=logging.INFO, stream=sys.stderr, format="[bench] %(name)s: %(message)s")
    logging.getLogger("atom_amd").setLevel(logging.INFO if args.shape == "32b" else logging.WARNING)
    # no shape named, nothing else asked for: the headline run and every other shape's workload beside it
    everything = all(getattr(args, k) == ap.get_default(k) for k in vars(args) if k not in ("gpus", "steps", "warmup"))
    if args.products or args.attention:
        print(json.dumps(run_products(args) if args.products else run_attention(args)), flush=True)
        return 0
    args.shape = args.shape or "8b"
    line = run_shape(args)
    if everything:
        line["shapes"] = shapes = {}
        for key, sub in (("qwen3_4b_mixed", dict(shape="4b")), ("qwen3_32b_long", dict(shape="32b")),
                         ("qwen3_8b_single", dict(shape="8b", single="18,80;549,256"))):
            sub_args = argparse.Namespace(**{**vars(args), **sub, "steps": min(args.steps, 32) if key == "qwen3_32b_long" else args.steps})
            shapes[key] = run_shape(sub_args)
        shapes["qwen3_8b_long_context"] = run_long_context(args)
        # the same numbers flat, beside the headline's other points
        pts = line["points"]
        pts["mixed_4b_output_tok_s"] = shapes["qwen3_4b_mixed"]["value"]
        pts["decode_32b_b16_ctx8192"] = shapes["qwen3_32b_long"]["value"]
        pts["prefill_32b_tok_s"] = shapes["qwen3_32b_long"]["prefill"]["value"]
        for pair, row in shapes["qwen3_8b_single"]["single_stream"].items():
            pts[f"single_{pair}_ttft_ms"], pts[f"single_{pair}_tpot_ms"] = row["ttft_ms"], row["tpot_ms"]
        for ctx, row in shapes["qwen3_8b_long_context"]["decode"].items():
            pts[f"decode_b8_{ctx}"] = row["value"]
            line["points_roofline"][f"decode_b8_{ctx}"] = row["roofline"]["frac"]
        pts["prefill_16384_tok_s"] = shapes["qwen3_8b_long_context"]["prefill"]["value"]
    print(json.dumps(line), flush=True)
    return 0


def run_shape(args) -> dict:
    """One shape's workload on an engine of its own; returns the record of that run."""
    mixed_requests = 0 if (args.single or args.decode) else (args.mixed or (32 if args.shape == "4b" else 0))
    plain = bool(args.single) or args.decode
    long_run = args.shape == "32b" and not mixed_requests and not plain
    points = sorted({int(x) for x in args.points.split(",") if x} | {args.batch})
    if long_run:
        max_seqs, max_model_len, pages, budget = 16, args.max_model_len or 8192 + 512, -1, 4096
    else:
        max_seqs = max(points + [mixed_requests])
        max_model_len = args.max_model_len or max(4096, 2 * args.context)
        pages, budget = max_seqs * max_model_len // 16, (512 + mixed_requests if mixed_requests else 16384)
    budget = args.budget or budget
    llm, name, raw, layers, gen = make_engine(args, args.shape, max_seqs=max_seqs, max_model_len=max_model_len,
                                              pages=pages, budget=budget, layers=args.layers)
    try:
        if args.single:
            pairs = [tuple(int(v) for v in pair.split(",")) for pair in args.single.split(";")]
            return run_single(llm, args, name, raw, layers, gen, pairs)
        if mixed_requests:
            return run_mixed(llm, args, name, raw, layers, gen, mixed_requests)
        if long_run:
            return run_long(llm, args, name, raw, layers, gen)
        return run_points(llm, args, name, raw, layers, gen, points, max_model_len)
    finally:
        release(llm)


def run_points(llm, args, name, raw, layers, gen, points, max_model_len) -> dict:
    """A prefill of ``--context`` tokens and decode at every batch size of ``points``."""
    prefill = None
    if not args.no_prefill:
        prefill = time_prefill(llm, raw, layers, gen, args.context)
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    results = {}
    for b in points:
        steps = args.steps
        elapsed, ctx0 = time_decode(llm, args, raw, gen, b, args.context, steps, args.warmup)
        results[b] = (elapsed, ctx0, steps)
        print(f"[bench] decode batch {b}: {b * steps / elapsed:.1f} tok/s, {elapsed / steps * 1e3:.3f} ms/step",
              file=sys.stderr, flush=True)

    def roofline(b):
        elapsed, ctx0, steps = results[b]
        return decode_roofline(raw, layers, b, ctx0, steps, elapsed)

    elapsed, ctx0, steps = results[args.batch]
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({name}, bf16); prefill tok/s at {args.context} tokens and "
                  f"batch {'/'.join(str(b) for b in points if b != args.batch)} alongside",
        "value": round(args.batch * steps / elapsed, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": round(elapsed / steps * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: seeded uniform random token ids, seeded random N(0, 0.02) weights",
        "config": flat_config(name, raw, layers, global_batch=args.batch, seq_len=args.context,
                              max_model_len=max_model_len, decode_steps=steps, hip_graphs=not args.enforce_eager,
                              deferred_output=not args.no_deferred_output),
        "roofline": roofline(args.batch),
        "points": {f"decode_b{b}": round(b * results[b][2] / results[b][0], 2) for b in points if b != args.batch},
        # the same fraction of the HBM peak for the other batch sizes
        "points_roofline": {f"decode_b{b}": roofline(b)["frac"] for b in points if b != args.batch},
    }
    if prefill:
        line["prefill"] = prefill
    return line


if __name__ == "__main__":
    sys.exit(main())
