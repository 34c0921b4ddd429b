"""Turns logits rows into token ids with the sampling kernel.

Semantics are the reference's (atom/model_ops/sampler.py:43-171, prepare_sample at
atom/model_engine/model_runner.py:2661-2707): temperatures at or below 1e-10 mean argmax;
otherwise an exponential race over ``softmax(logits / T)``; top-k / top-p arrays are
passed only when some request sets them, and filter on the temperature-scaled
distribution.  The noise of a row comes from (the request's seed, how many tokens it has
sampled), not from a generator shared by the batch.
"""

from __future__ import annotations

import numpy as np
import torch

from .params import SamplingParams

SAMPLER_EPS = 1e-10  # atom/model_ops/sampler.py:31


class Sampler:
    def __init__(self, ops, device):
        self.ops = ops
        self.device = torch.device(device)

    def __call__(self, logits: torch.Tensor, params: list[SamplingParams], seeds: list[int],
                 counters: list[int], out: torch.Tensor | None = None) -> torch.Tensor:
        """``logits`` float32 [rows, vocab]; returns int32 [rows] on the device (``out`` if given)."""
        rows = logits.shape[0]
        assert rows == len(params) == len(seeds) == len(counters)
        if out is None:
            out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        temps = np.array([p.temperature if p.temperature > SAMPLER_EPS else 0.0 for p in params], dtype=np.float32)
        if not temps.any():  # all greedy
            self.ops.sample(logits, None, out)
            return out
        need_k = any(p.top_k != -1 for p in params)
        need_p = any(p.top_p < 1.0 for p in params)
        dev = logits.device
        t = torch.from_numpy(temps).to(dev)
        ks = torch.tensor([p.top_k for p in params], dtype=torch.int32, device=dev) if need_k else None
        ps = torch.tensor([p.top_p for p in params], dtype=torch.float32, device=dev) if need_p else None
        sd = torch.tensor([s & 0x7FFFFFFFFFFFFFFF for s in seeds], dtype=torch.int64, device=dev)
        ct = torch.tensor(counters, dtype=torch.int64, device=dev)
        self.ops.sample(logits, t, out, top_ks=ks, top_ps=ps, seeds=sd, counters=ct, eps=SAMPLER_EPS)
        return out

    @staticmethod
    def logprobs(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
        """log-probability of each sampled token (atom/model_engine/model_runner.py:3233-3240)."""
        return torch.log_softmax(logits.float(), dim=-1).gather(1, tokens.long().unsqueeze(1)).squeeze(1)
