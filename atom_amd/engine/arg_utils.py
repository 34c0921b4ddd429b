"""Engine arguments: a dataclass, its command-line flags and the engine it creates, with
ATOM's names, defaults and meanings (atom/model_engine/arg_utils.py:33-626) for what this
engine has.  Flags of subsystems that are not built (tensor/pipeline/data parallelism,
speculative decoding, expert parallelism, servers, quantized caches) are absent.  Every
long flag is accepted in kebab- and snake-case (atom/utils/arg_parser.py:17-44)."""

from __future__ import annotations

import argparse
import json
import sys
from dataclasses import dataclass, fields


class FlexibleArgumentParser(argparse.ArgumentParser):
    """``--max-model-len`` and ``--max_model_len`` are the same flag."""

    def parse_args(self, args=None, namespace=None):
        if args is None:
            args = sys.argv[1:]
        fixed = []
        for a in args:
            if a.startswith("--"):
                key, eq, val = a.partition("=")
                a = "--" + key[2:].replace("_", "-") + eq + val
            fixed.append(a)
        return super().parse_args(fixed, namespace)


def parse_size_list(text: str) -> list[int]:
    return [int(x) for x in json.loads(text)] if text else []


@dataclass
class EngineArgs:
    model: str = "Qwen/Qwen3-0.6B"
    enforce_eager: bool = False
    enable_prefix_caching: bool = True
    kv_cache_dtype: str = "bf16"
    block_size: int = 16
    max_model_len: int | None = None
    max_num_batched_tokens: int = 16384
    long_prefill_token_threshold: int = 0
    enable_chunked_prefill: bool = True
    scheduler_delay_factor: float = 0.0
    max_num_seqs: int = 512
    gpu_memory_utilization: float = 0.9
    cudagraph_capture_sizes: str = "[1,2,4,8,16,32,48,64,128,256]"
    cudagraph_prefill_sizes: str = "[]"
    cudagraph_prefill_slots: int = 2
    load_dummy: str | None = None
    torch_profiler_dir: str | None = None
    mark_trace: bool = False
    deferred_output: bool = True
    level: int = 3
    cudagraph_mode: str = "FULL"
    hf_overrides: dict | None = None
    num_kvcache_blocks: int = -1
    dtype: str = "bf16"
    seed: int = 0

    @staticmethod
    def add_cli_args(parser: argparse.ArgumentParser) -> argparse.ArgumentParser:
        parser.add_argument("--model", type=str, default="Qwen/Qwen3-0.6B", help="Model folder (config.json + safetensors).")
        parser.add_argument("--enforce-eager", action="store_true", help="Never replay captured HIP graphs.")
        parser.add_argument("--enable-prefix-caching", action=argparse.BooleanOptionalAction, default=True,
                            help="Reuse cache pages that already hold the beginning of a new prompt.")
        parser.add_argument("--kv-cache-dtype", choices=["bf16"], default="bf16", help="KV cache type (the model's own).")
        parser.add_argument("--block-size", type=int, default=16, help="Tokens per KV cache block.")
        parser.add_argument("--max-model-len", type=int, default=None, help="Longest sequence (prompt + output).")
        parser.add_argument("--max-num-batched-tokens", type=int, default=16384, help="Token budget of one step.")
        parser.add_argument("--long-prefill-token-threshold", type=int, default=0,
                            help="Cap on a prompt portion per step (0: none).")
        parser.add_argument("--enable-chunked-prefill", action=argparse.BooleanOptionalAction, default=True,
                            help="Cut prompts into portions under the token budget.")
        parser.add_argument("--scheduler-delay-factor", type=float, default=0.0,
                            help="Hold new prompts this many prompt-latencies while others decode.")
        parser.add_argument("--max-num-seqs", type=int, default=512, help="Most requests running at a time.")
        parser.add_argument("--gpu-memory-utilization", type=float, default=0.9, help="Share of GPU memory to use.")
        parser.add_argument("--cudagraph-capture-sizes", type=str, default="[1,2,4,8,16,32,48,64,128,256]",
                            help="Decode batch sizes captured as HIP graphs.")
        parser.add_argument("--cudagraph-prefill-sizes", type=str, default="[]",
                            help="Ours: prompt-token capacities of graphs for steps with prompt portions beside decode "
                                 "tokens, e.g. [512]; empty (the default): such steps are launched one by one, ahead of time.")
        parser.add_argument("--cudagraph-prefill-slots", type=int, default=2,
                            help="Ours: prompt portions one such graph holds at most.")
        parser.add_argument("--load-dummy", type=str, nargs="?", const="random", default=None,
                            help="Skip the checkpoint: seeded random weights.")
        parser.add_argument("--torch-profiler-dir", type=str, default=None, help="Write a torch.profiler trace here.")
        parser.add_argument("--mark-trace", action="store_true",
                            help="Name every operation's kernels in profiler traces (record_function spans).")
        parser.add_argument("--deferred-output", action=argparse.BooleanOptionalAction, default=True,
                            help="Launch the next decode step before the host has read the last one's tokens.")
        # the reference's two switches of its tracing compiler and graph modes (atom/model_engine/arg_utils.py
        # :195-208): there is no compiler here, so the level changes nothing; NONE means --enforce-eager, every
        # other mode the one kind of graph this engine has (a whole decode step)
        parser.add_argument("--level", type=int, default=3, help="Accepted for the reference's command lines; no effect.")
        parser.add_argument("--cudagraph-mode", type=str, default="FULL",
                            choices=["NONE", "PIECEWISE", "FULL", "FULL_AND_PIECEWISE", "AF_PIECEWISE"],
                            help="NONE: never replay graphs (as --enforce-eager); any other: whole decode steps.")
        parser.add_argument("--hf-overrides", type=json.loads, default=None, help="JSON dict of config.json overrides.")
        parser.add_argument("--num-kvcache-blocks", type=int, default=-1, help="Cache pages (-1: from free memory).")
        parser.add_argument("--dtype", choices=["bf16", "bfloat16", "fp32", "float32"], default="bf16",
                            help="bf16: the serving kernels; fp32: everything in true 32-bit.")
        parser.add_argument("--seed", type=int, default=0, help="Seed of sampling and of random weights.")
        return parser

    @classmethod
    def from_cli_args(cls, args: argparse.Namespace) -> "EngineArgs":
        names = [f.name for f in fields(cls)]
        return cls(**{n: getattr(args, n) for n in names if hasattr(args, n)})

    def _get_engine_kwargs(self) -> dict:
        kwargs = {f.name: getattr(self, f.name) for f in fields(self) if f.name != "model"}
        kwargs["kv_cache_block_size"] = kwargs.pop("block_size")
        kwargs["cudagraph_capture_sizes"] = parse_size_list(kwargs["cudagraph_capture_sizes"])
        kwargs["cudagraph_prefill_sizes"] = parse_size_list(kwargs["cudagraph_prefill_sizes"])
        kwargs.pop("level")
        if kwargs.pop("cudagraph_mode") == "NONE":
            kwargs["enforce_eager"] = True
        return kwargs

    def create_engine(self, tokenizer=None):
        from .llm_engine import LLMEngine

        return LLMEngine(self.model, tokenizer=tokenizer, **self._get_engine_kwargs())
