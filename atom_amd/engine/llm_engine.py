"""The Python entry point, in ATOM's manner (atom/model_engine/llm_engine.py:36-260):

    llm = LLMEngine(model_dir, **config_kwargs)
    outputs = llm.generate(prompts, sampling_params)   # prompts: strings or token-id lists

Each output is a dict with the reference's keys (llm_engine.py:752-762): ``text``,
``token_ids``, ``logprobs``, ``latency``, ``finish_reason``, ``num_tokens_input``,
``num_tokens_output``, ``ttft``, ``tpot``.  Everything runs in this process: one step is
schedule -> step function -> sampler -> postprocess.
"""

from __future__ import annotations

import logging
import os
import time

import torch

from ..config.engine_config import Config
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .core import TORCH_DTYPES, build_core, load_model
from .scheduler import Scheduler
from .sequence import Sequence, SequenceStatus

logger = logging.getLogger("atom_amd")


def _load_tokenizer(path: str):
    """A tokenizer if the folder has one (atom/model_engine/llm_engine.py:23-33); prompts
    given as token ids need none."""
    if not any(os.path.isfile(os.path.join(path, f)) for f in ("tokenizer.json", "tokenizer.model", "vocab.json")):
        return None
    from transformers import AutoTokenizer

    return AutoTokenizer.from_pretrained(path)


class _Stage:
    """Host memory (pinned where there is a GPU) that a step's sampled tokens and their log-probabilities
    are copied into."""

    def __init__(self, rows: int, pinned: bool):
        self.pinned = pinned
        self.grow(max(1, rows))

    def grow(self, rows: int) -> None:
        self.tokens = torch.zeros(rows, dtype=torch.int32, pin_memory=self.pinned)
        self.logprobs = torch.zeros(rows, dtype=torch.float32, pin_memory=self.pinned)


class _InFlight:
    """A step that has been queued on the device and not yet read."""

    def __init__(self, batch, finals, start: float):
        self.batch = batch
        self.finals = finals
        self.start = start
        self.tokens: torch.Tensor | None = None
        self.logprobs: torch.Tensor | None = None
        self.ready = torch.cuda.Event() if torch.cuda.is_available() else _NoEvent()


class _NoEvent:
    def record(self):
        pass

    def synchronize(self):
        pass


class LLMEngine:
    def __init__(self, model: str, tokenizer=None, ops=None, weight_source=None, **kwargs):
        unknown = sorted(k for k in kwargs if k not in Config.__dataclass_fields__)
        if unknown:
            raise TypeError(f"LLMEngine: unknown option(s) {unknown}; known: {sorted(Config.__dataclass_fields__)}")
        self.config = cfg = Config(model, **kwargs)
        self.tokenizer = tokenizer if tokenizer is not None else (
            _load_tokenizer(model) if isinstance(model, str) and os.path.isdir(model) else None)
        self.dtype = TORCH_DTYPES[cfg.dtype]
        if ops is None:
            from ..kernels.hip import HipKernels

            ops = HipKernels(cfg.device)
        if cfg.mark_trace and hasattr(ops, "mark_trace"):
            ops.mark_trace()
        self.ops = ops
        source = weight_source
        if source is None and cfg.load_dummy:
            from ..config.registry import build_model
            from ..weights.random_init import RandomSource

            source = RandomSource(build_model(cfg.model_config), cfg.seed, device=cfg.device)
        self.model, _ = load_model(cfg.model, dtype=self.dtype, device=cfg.device, model_config=cfg.model_config,
                                   source=source)
        self.core = build_core(
            self.model, ops, dtype=self.dtype, device=cfg.device, page_size=cfg.kv_cache_block_size,
            num_pages=cfg.num_kvcache_blocks if cfg.num_kvcache_blocks > 0 else None,
            budget_bytes=self._cache_budget() if cfg.num_kvcache_blocks <= 0 else None,
            max_num_seqs=cfg.max_num_seqs, max_model_len=cfg.max_model_len,
            max_num_batched_tokens=cfg.max_num_batched_tokens,
            graph_sizes=None if cfg.enforce_eager else cfg.cudagraph_capture_sizes,
            graph_prefill_sizes=cfg.cudagraph_prefill_sizes, graph_prefill_slots=cfg.cudagraph_prefill_slots,
            prefix_caching=cfg.enable_prefix_caching)
        self._log_capacity()
        if self.core.graphs is not None:   # as the reference's engine does before it serves (engine_core.py:131-138)
            captured = self.core.graphs.capture_all()
            logger.info("captured %d decode graphs for batch sizes %s", captured, self.core.graphs.sizes)
        self.scheduler = Scheduler(cfg, self.core)
        self.sampler = Sampler(ops, cfg.device, cfg.max_num_seqs)
        self.seqs: dict[int, Sequence] = {}
        self._profiler = None
        self.deferred_output = bool(cfg.deferred_output)
        self._in_flight: _InFlight | None = None
        self.steps_launched = 0          # steps queued on the device so far ...
        self.steps_launched_ahead = 0    # ... and how many of them before the step before them had been read
        # two pinned buffers take turns: a step's tokens are read while the next step's are on their way
        self._stages = [_Stage(cfg.max_num_seqs, pinned=torch.device(cfg.device).type == "cuda") for _ in range(2)]
        self._next_stage = 0

    def _cache_budget(self) -> int:
        """Bytes for the cache: the share of device memory ``gpu_memory_utilization`` allows minus what is
        in use, minus what the decode graphs will take and a 2 % margin
        (atom/model_engine/model_runner.py:1591-1611, 1737-1749)."""
        dev = torch.device(self.config.device)
        if dev.type != "cuda":
            return 64 << 20
        free, total = torch.cuda.mem_get_info(dev)
        used = total - free
        graphs = 0 if self.config.enforce_eager else self._graph_estimate()
        safety = int(total * 0.02)
        budget = max(0, min(int(total * self.config.gpu_memory_utilization) - used - graphs - safety, free))
        logger.info("Memory budget: total_gpu=%.2fGB, free=%.2fGB, utilization=%s, in_use=%.2fGB, "
                    "cudagraph_est=%.2fGB, safety=%.2fGB, available_for_kv=%.2fGB", total / 2**30, free / 2**30,
                    self.config.gpu_memory_utilization, used / 2**30, graphs / 2**30, safety / 2**30, budget / 2**30)
        return budget

    def _graph_estimate(self) -> int:
        """Bytes the decode graphs' shared pool will hold: every bucket keeps its float32 logits, and the
        buckets share the memory of one step's activations (what a layer frees during capture the next
        layer takes again), which the largest bucket sizes; product slices and slack on top."""
        cfg, spec = self.config, self.model.spec
        sizes = [s for s in cfg.cudagraph_capture_sizes if s <= cfg.max_num_seqs]
        if not sizes:
            return 0
        widest = max((int(p.shape[0]) for block in self.model.blocks for part in block.walk()
                      for p in part.params.values() if p.dim() == 2), default=spec.hidden_size)
        rows, logits_rows = max(sizes), sum(sizes)
        if cfg.cudagraph_prefill_sizes:
            # a graph per (portion tokens P, single tokens N >= 8): logits at the portion slots and the single
            # tokens, activations for P + N rows
            mixed = [s for s in sizes if s >= 8] or sizes[-1:]
            logits_rows += len(cfg.cudagraph_prefill_sizes) * sum(cfg.cudagraph_prefill_slots + n for n in mixed)
            rows = max(rows, max(cfg.cudagraph_prefill_sizes) + max(mixed))
        live = rows * (4 * spec.hidden_size + 8 * widest) * 4
        return logits_rows * spec.vocab_size * 4 + 2 * live + (128 << 20)

    def _log_capacity(self) -> None:
        """How many requests the pages hold at once, by context length
        (the reference's table, atom/model_engine/model_runner.py:1751-1781)."""
        cfg = self.config
        full = [g for g in self.core.plan.groups if g.window is None]
        if not full:
            return
        pages, page = min(g.num_pages for g in full), full[0].page_size
        lines = []
        for pct in (10, 30, 50, 70, 90, 100):
            ctx = max(1, cfg.max_model_len * pct // 100)
            per_req = -(-ctx // page)
            by_pages = pages // per_req
            most = min(cfg.max_num_seqs, by_pages)
            bound = "slots" if most == cfg.max_num_seqs < by_pages else "blocks"
            lines.append(f"  {pct:>3}% ({ctx:>7} tok): {per_req:>6} blk/req -> max_concurrent={most:<5} (bound by {bound})")
        logger.info("Concurrent capacity vs context length (max_model_len=%d, block_size=%d, max_slots=%d, "
                    "pool_blocks=%d, cache %.2fGB):\n%s", cfg.max_model_len, page, cfg.max_num_seqs, pages,
                    self.core.plan.total_bytes(cfg.max_num_seqs) / 2**30, "\n".join(lines))

    # ------------------------------------------------------------------ requests

    def add_request(self, prompt, sampling_params: SamplingParams | None = None) -> list[Sequence]:
        sp = sampling_params or SamplingParams()
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; this model folder has none (pass token ids)")
            token_ids = self.tokenizer.encode(prompt)
        else:
            token_ids = [int(t) for t in prompt]
        if not token_ids:
            raise ValueError("an empty prompt cannot be run")
        stop_seqs = []
        if sp.stop_strings:   # atom/model_engine/llm_engine.py:661-671
            if self.tokenizer is None:
                raise ValueError("stop_strings need a tokenizer")
            stop_seqs = [self.tokenizer.encode(s, add_special_tokens=False) for s in sp.stop_strings]
        out = []
        for k in range(sp.n):
            base = sp.seed if sp.seed is not None else self.config.seed
            seq = Sequence(token_ids, sp, stop_seqs)
            seq.seed = (base * 1_000_003 + seq.id * 7919 + k) if sp.seed is None else (base + k)
            self.seqs[seq.id] = seq
            self.scheduler.add(seq)
            out.append(seq)
        return out

    def abort(self, request_id: int) -> bool:
        """Ends a waiting or running request early (``request_id``: the ``id`` of a sequence that
        ``add_request`` returned).  It leaves at the next step with ``finish_reason`` "aborted" and what it
        has generated so far; its pages and slot go back to the pools.  Returns whether it was found."""
        return self.scheduler.abort(request_id)

    def is_finished(self) -> bool:
        return self.scheduler.is_finished() and self._in_flight is None

    # ------------------------------------------------------------------ one step

    def step(self) -> list[Sequence]:
        """Runs one scheduled batch; returns the sequences that left in it.

        With ``deferred_output`` (the default, and the reference's way, atom/model_engine/model_runner.py
        :358-392) the batch that follows a decode step is launched before the host reads that step's
        tokens, whenever the scheduler can tell what it will hold (``Scheduler.schedule_ahead``): the
        new step takes its tokens from the sampler's output on the device.  A request that turns out to
        have finished is run once too often and that result dropped."""
        done = []
        if self._in_flight is None:
            batch = self.scheduler.schedule()
            done += self.scheduler.take_rejected()
            if batch is None:
                return done
            self._in_flight = self._launch(batch, None)
        running = self._in_flight
        ahead = None
        if self.deferred_output:
            batch = self.scheduler.schedule_ahead(running.batch)
            done += self.scheduler.take_rejected()   # requests that the schedule turned away or found aborted
            if batch is not None:
                ahead = self._launch(batch, {it.seq.id: k for k, it in enumerate(running.finals)})
                self.steps_launched_ahead += 1
        done += self._finish(running)
        self._in_flight = ahead
        return done

    def _launch(self, batch, sampled_rows: dict[int, int] | None) -> "_InFlight":
        """Queues the batch's step and its sampling on the device; waits for nothing."""
        start = time.time()
        self.steps_launched += 1
        with torch.profiler.record_function(self._run_label(batch)):
            logits = self.core.step(batch.entries(sampled_rows))
        finals = [it for it in batch.items if it.is_final]
        flight = _InFlight(batch, finals, start)
        if finals:
            # the tokens stay on the device for a step scheduled ahead and go to pinned memory for the host
            tokens = self.sampler(logits, [it.seq.sampling_params for it in finals],
                                  [it.seq.seed for it in finals],
                                  [it.seq.num_completion_tokens for it in finals],
                                  out=self.core.sampled[:len(finals)])
            stage = self._stages[self._next_stage]
            self._next_stage = (self._next_stage + 1) % len(self._stages)
            if len(finals) > stage.tokens.numel():
                stage.grow(len(finals))
            flight.tokens = stage.tokens[:len(finals)]
            flight.tokens.copy_(tokens, non_blocking=True)
            if any(it.seq.sampling_params.logprobs for it in finals):
                flight.logprobs = stage.logprobs[:len(finals)]
                flight.logprobs.copy_(self.sampler.logprobs(logits, tokens), non_blocking=True)
            flight.ready.record()
        return flight

    def _finish(self, flight: "_InFlight") -> list[Sequence]:
        """Waits for the step's tokens and hands them to the scheduler."""
        sampled = {}
        if flight.finals:
            flight.ready.synchronize()
            host = flight.tokens.tolist()
            lps = flight.logprobs.tolist() if flight.logprobs is not None else None
            for k, it in enumerate(flight.finals):
                sampled[it.seq.id] = host[k]
                if (lps is not None and it.seq.sampling_params.logprobs
                        and it.seq.status == SequenceStatus.RUNNING):
                    it.seq.logprobs.append(lps[k])
        return self.scheduler.postprocess(flight.batch, sampled, time.time() - flight.start)

    def drain(self) -> list[Sequence]:
        """Finishes a step that is still running without starting another."""
        if self._in_flight is None:
            return []
        flight, self._in_flight = self._in_flight, None
        return self._finish(flight)

    @staticmethod
    def _run_label(batch) -> str:
        """The span name of a step in a profiler trace, in the reference's form
        (atom/model_engine/run_labels.py:1-37): ``prefill[bs=2 tok=96 ctx=160]``, ``decode[bs=8 ctx=..]``."""
        prefill = [it for it in batch.items if not it.is_decode]
        decode = [it for it in batch.items if it.is_decode]
        parts = []
        if prefill:
            parts.append(f"prefill[bs={len(prefill)} tok={sum(it.num_tokens for it in prefill)} "
                         f"ctx={sum(it.start + it.num_tokens for it in prefill)}]")
        if decode:
            parts.append(f"decode[bs={len(decode)} ctx={sum(it.start + 1 for it in decode)}]")
        return "+".join(parts)

    # ------------------------------------------------------------------ generate

    def _output(self, seq: Sequence) -> dict:
        ids = seq.completion_token_ids
        text = self.tokenizer.decode(ids) if self.tokenizer is not None else ""
        n = seq.num_completion_tokens
        ttft = seq.first_token_time - seq.arrive_time if seq.first_token_time else 0.0
        tpot = (seq.leave_time - seq.first_token_time) / (n - 1) if n > 1 else 0.0
        logger.info("Request %s finished with reason %s. Input tokens: %d, output tokens: %d, latency: %.2fs, "
                    "TTFT: %.3fs, TPOT: %.3fs", seq.id, seq.leave_reason, seq.num_prompt_tokens, n,
                    seq.leave_time - seq.arrive_time, ttft, tpot)
        return {"text": text, "token_ids": ids, "logprobs": seq.logprobs or None,
                "latency": seq.leave_time - seq.arrive_time, "finish_reason": seq.leave_reason,
                "num_tokens_input": seq.num_prompt_tokens, "num_tokens_output": n, "ttft": ttft, "tpot": tpot}

    def generate(self, prompts, sampling_params: SamplingParams | list[SamplingParams] | None = None) -> list[dict]:
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params or SamplingParams()] * len(prompts)
        if len(sampling_params) != len(prompts):
            raise ValueError("one SamplingParams per prompt, or one for all")
        pending = {}
        for prompt, sp in zip(prompts, sampling_params):
            for seq in self.add_request(prompt, sp):
                pending[seq.id] = seq
        outputs = {}
        while pending:
            for seq in self.step():
                if seq.id in pending:
                    outputs[seq.id] = self._output(seq)
                    del pending[seq.id]
                    self.seqs.pop(seq.id, None)
            if self.is_finished() and pending:
                raise RuntimeError(f"the scheduler is idle but {len(pending)} request(s) never finished")
        self.drain()   # a step launched ahead for requests that have all finished
        return [outputs[i] for i in sorted(outputs)]

    # ------------------------------------------------------------------ profiling

    def start_profile(self):
        """torch.profiler trace into ``torch_profiler_dir`` (atom/model_engine/model_runner.py:1025-1129)."""
        if not self.config.torch_profiler_dir or self._profiler is not None:
            return
        from torch.profiler import ProfilerActivity, profile

        self._profiler = profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA])
        self._profiler.__enter__()

    def stop_profile(self):
        if self._profiler is None:
            return
        self._profiler.__exit__(None, None, None)
        os.makedirs(self.config.torch_profiler_dir, exist_ok=True)
        self._profiler.export_chrome_trace(os.path.join(self.config.torch_profiler_dir, "trace.json"))
        self._profiler = None
