#!/usr/bin/python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

The default run has the layer sizes of Qwen3-8B (36 layers, hidden 4096, 32/8 heads of
128, intermediate 12288, vocabulary 151936) with seeded random bfloat16 weights, 8
sequences of 2,048 random prompt tokens each, and times K decode steps through the
engine's own step loop (scheduler, step function, sampler).  ``value`` is decoded tokens
a second.  It also times one 2,048-token prefill and decoding at batch 1 and 64, and
prints one JSON line.  More than one GPU is not built: ``--gpus N>1`` says so and exits 2.
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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--max-model-len", type=int, default=None,
                    help="positions a request may reach (default: 4096, or twice a longer --context)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--points", type=str, default="1,64", help="other decode batch sizes to time")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--mixed", type=int, default=0, metavar="N",
                    help="instead: N requests with prompts of 64..3072 tokens through the scheduler, prompt portions of "
                         "512 tokens beside running decodes, 128 output tokens each; prints its own line")
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

    import torch

    from atom_amd import LLMEngine, SamplingParams
    from atom_amd.config import model_config_from_dict

    raw = dict(QWEN3_8B)
    full_layers = raw["num_hidden_layers"]
    layers = args.layers or full_layers
    raw["num_hidden_layers"] = layers
    cfg = model_config_from_dict(raw)
    points = sorted({int(x) for x in args.points.split(",") if x} | {args.batch})
    points = [p for p in points]
    max_seqs = max(points + [args.mixed])
    max_model_len = args.max_model_len or max(4096, 2 * args.context)
    block = 16
    t0 = time.time()
    llm = LLMEngine("qwen3-8b-random", model_config=cfg, load_dummy="random", seed=2, dtype="bf16",
                    max_model_len=max_model_len, kv_cache_block_size=block,
                    num_kvcache_blocks=max_seqs * max_model_len // block, max_num_seqs=max_seqs,
                    max_num_batched_tokens=16384, enforce_eager=args.enforce_eager,
                    deferred_output=not args.no_deferred_output)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    gen = torch.Generator().manual_seed(2)
    vocab = raw["vocab_size"]

    def prompt():
        return torch.randint(0, vocab, (args.context,), generator=gen).tolist()

    def sync():
        torch.cuda.synchronize()

    if args.mixed:
        # continuous batching under load: every step holds the running requests' decode tokens and, under a
        # budget of 512 + N tokens, the next portion of a waiting prompt
        llm.scheduler.max_num_batched_tokens = 512 + args.mixed
        lens = torch.randint(64, 3073, (args.mixed,), generator=gen).tolist()
        sp = SamplingParams(temperature=0.0, max_tokens=128, ignore_eos=True)
        prompts = [torch.randint(0, vocab, (n,), generator=gen).tolist() for n in lens]
        sync()
        t = time.perf_counter()
        outs = llm.generate(prompts, sp)
        sync()
        elapsed = time.perf_counter() - t
        assert all(o["num_tokens_output"] == 128 for o in outs)
        print(json.dumps({"workload": "mixed", "requests": args.mixed, "prompt_tokens": sum(lens),
                          "output_tokens": 128 * args.mixed, "seconds": round(elapsed, 3),
                          "output_tok_s": round(128 * args.mixed / elapsed, 1),
                          "total_tok_s": round((sum(lens) + 128 * args.mixed) / elapsed, 1),
                          "steps": llm.core.steps_run, "preemptions": llm.scheduler.total_preemptions,
                          "mean_ttft_ms": round(1e3 * sum(o["ttft"] for o in outs) / len(outs), 1),
                          "mean_tpot_ms": round(1e3 * sum(o["tpot"] for o in outs) / len(outs), 2)}), flush=True)
        return 0

    # ---- prefill of one 2,048-token prompt
    prefill = None
    if not args.no_prefill:
        sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
        llm.generate([prompt()], sp)            # warm-up: library autotuning, first-use allocations
        times = []
        for _ in range(3):
            p = prompt()
            sync()
            t = time.perf_counter()
            llm.generate([p], sp)
            sync()
            times.append(time.perf_counter() - t)
        best = min(times)
        flops = prefill_flops(raw, layers, args.context)
        prefill = {"value": round(args.context / best, 1), "tokens": args.context, "ms": round(best * 1e3, 3),
                   "frac": round(flops / best / MFMA_PEAK["bf16"], 4)}
        print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode at each batch size
    def decode(batch: int, steps: int, warmup: int):
        # prompts are admitted over several steps, so the first requests are some tokens ahead of the last
        # when all decode: leave room, so that none finishes (and the batch does not shrink) while timed
        admission_steps = -(-batch * args.context // 16384) + 1
        sp = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k, seed=1,
                            max_tokens=steps + warmup + admission_steps + 2, ignore_eos=True)
        for _ in range(batch):
            llm.add_request(prompt(), sp)
        while any(s.num_completion_tokens == 0 for s in llm.seqs.values()):   # prompts, untimed
            llm.step()
        for _ in range(warmup):
            llm.step()
        sync()
        assert len(llm.scheduler.running) == batch and not llm.scheduler.waiting
        start_ctx = next(iter(llm.seqs.values())).num_tokens
        t = time.perf_counter()
        for _ in range(steps):
            llm.step()
        sync()
        elapsed = time.perf_counter() - t
        assert len(llm.scheduler.running) == batch, "a request finished inside the timed steps"
        while not llm.is_finished():
            llm.step()
        llm.seqs.clear()
        return elapsed, start_ctx

    results = {}
    for b in points:
        steps = args.steps
        elapsed, ctx0 = decode(b, steps, args.warmup)
        results[b] = (elapsed, ctx0, steps)
        print(f"[bench] decode batch {b}: {b * steps / elapsed:.1f} tok/s, {elapsed / steps * 1e3:.3f} ms/step",
              file=sys.stderr, flush=True)

    elapsed, ctx0, steps = results[args.batch]
    per_step = elapsed / steps
    mean_ctx = ctx0 + steps / 2
    step_bytes = weight_bytes(raw, layers) + args.batch * mean_ctx * kv_bytes_per_token(raw, layers)
    achieved = step_bytes / per_step
    line = {
        "metric": "decode tok/s at batch 8 (Qwen3-8B, bf16); prefill tok/s at 2048 tokens and batch 1/64 alongside",
        "value": round(args.batch * steps / elapsed, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": round(per_step * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic: seeded uniform random token ids, seeded random N(0, 0.02) weights",
        "config": {"model": "Qwen3-8B shape, random weights", "global_batch": args.batch, "seq_len": args.context,
                   "parallelism": "single GPU", "layers": layers, "layers_of_model": full_layers,
                   "hidden_size": raw["hidden_size"], "num_attention_heads": raw["num_attention_heads"],
                   "num_key_value_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
                   "intermediate_size": raw["intermediate_size"], "vocab_size": vocab,
                   "max_model_len": max_model_len, "kv_block_size": block, "decode_steps": steps,
                   "hip_graphs": not args.enforce_eager, "deferred_output": not args.no_deferred_output},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": {f"decode_b{b}": round(b * results[b][2] / results[b][0], 2) for b in points if b != args.batch},
    }
    if prefill:
        line["prefill"] = prefill
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
