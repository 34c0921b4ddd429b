"""Turns logits rows into token ids with the sampling kernel.

Semantics are the reference's (atom/model_ops/sampler.py:43-171, prepare_sample at
atom/model_engine/model_runner.py:2661-2707): temperatures at or below 1e-10 mean argmax;
otherwise an exponential race over ``softmax(logits / T)``; top-k / top-p arrays are
passed only when some request sets them, and filter on the temperature-scaled
distribution.  The noise of a row comes from (the request's seed, how many tokens it has
sampled), not from a generator shared by the batch.
"""

from __future__ import annotations

import torch

from .params import SamplingParams

SAMPLER_EPS = 1e-10  # atom/model_ops/sampler.py:31


class _Staging:
    """Pinned host memory for one step's per-row sampling parameters and the event that says its copy
    to the device has run: the copy is asynchronous, so the host never waits for the step before it."""

    def __init__(self, rows: int, pinned: bool):
        self.rows = rows
        self.host = torch.zeros(rows * Sampler.ROW_BYTES, dtype=torch.uint8, pin_memory=pinned)
        self.copied = torch.cuda.Event() if pinned else None
        self.pending = False


class Sampler:
    ROW_BYTES = 32   # seed i64, counter i64, temperature f32, top_p f32, top_k i32, 4 spare

    def __init__(self, ops, device, max_rows: int = 64):
        self.ops = ops
        self.device = torch.device(device)
        self._rows = 0
        self._stages: list[_Staging] = []
        self._turn = 0
        self._dev = None
        self._reserve(max_rows)

    def _reserve(self, rows: int) -> None:
        pinned = self.device.type == "cuda"
        self._rows = rows
        self._stages = [_Staging(rows, pinned) for _ in range(4)]
        self._dev = torch.zeros(rows * self.ROW_BYTES, dtype=torch.uint8, device=self.device)

    @staticmethod
    def _fields(buf: torch.Tensor, cap: int, rows: int):
        """Views of a buffer's five arrays (seeds, counters, temperatures, top_ps, top_ks), ``rows`` long."""
        seeds = buf[:8 * cap].view(torch.int64)[:rows]
        counters = buf[8 * cap:16 * cap].view(torch.int64)[:rows]
        temps = buf[16 * cap:20 * cap].view(torch.float32)[:rows]
        top_ps = buf[20 * cap:24 * cap].view(torch.float32)[:rows]
        top_ks = buf[24 * cap:28 * cap].view(torch.int32)[:rows]
        return seeds, counters, temps, top_ps, top_ks

    def __call__(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
                 counters: list[int], out: torch.Tensor | None = None) -> torch.Tensor:
        """``logits`` float32 [rows, vocab]; returns int32 [rows] on the device (``out`` if given)."""
        rows = logits.shape[0]
        assert rows == len(params) == len(seeds) == len(counters)
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        temps = [p.temperature if p.temperature > SAMPLER_EPS else 0.0 for p in params]
        if not any(temps):  # all greedy
            self.ops.sample(logits, None, out)
            return out
        need_k = any(p.top_k != -1 for p in params)
        need_p = any(p.top_p < 1.0 for p in params)
        if rows > self._rows:
            self._reserve(max(rows, 2 * self._rows))
        # one pinned buffer, one asynchronous copy
        stage = self._stages[self._turn]
        self._turn = (self._turn + 1) % len(self._stages)
        if stage.pending:
            stage.copied.synchronize()   # its last copy has run (four steps ago: it has)
            stage.pending = False
        h_seeds, h_counters, h_temps, h_ps, h_ks = self._fields(stage.host, self._rows, rows)
        h_seeds.copy_(torch.tensor([s & 0x7FFFFFFFFFFFFFFF for s in seeds], dtype=torch.int64))
        h_counters.copy_(torch.tensor(counters, dtype=torch.int64))
        h_temps.copy_(torch.tensor(temps, dtype=torch.float32))
        if need_p:
            h_ps.copy_(torch.tensor([p.top_p for p in params], dtype=torch.float32))
        if need_k:
            h_ks.copy_(torch.tensor([p.top_k for p in params], dtype=torch.int32))
        self._dev.copy_(stage.host, non_blocking=True)
        if stage.copied is not None:
            stage.copied.record()
            stage.pending = True
        sd, ct, t, ps, ks = self._fields(self._dev, self._rows, rows)
        self.ops.sample(logits, t, out, top_ks=ks if need_k else None, top_ps=ps if need_p else None,
                        seeds=sd, counters=ct, eps=SAMPLER_EPS)
        return out

    @staticmethod
    def logprobs(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
        """log-probability of each sampled token (atom/model_engine/model_runner.py:3233-3240)."""
        return torch.log_softmax(logits.float(), dim=-1).gather(1, tokens.long().unsqueeze(1)).squeeze(1)
