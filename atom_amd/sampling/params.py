"""Sampling parameters with ATOM's names, defaults and checks
(atom/sampling_params.py:8-30), plus ``seed``: the reference has no seed anywhere
(atom/model_engine/model_runner.py:125-127 is dead code); here each request draws from
its own seeded stream, so its tokens do not depend on its batch-mates."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Union


@dataclass
class SamplingParams:
    temperature: float = 1.0
    top_k: int = -1          # -1: keep all tokens
    top_p: float = 1.0       # 1.0: keep all tokens
    max_tokens: int = 64
    ignore_eos: bool = False
    stop_strings: Optional[list[str]] = None
    n: int = 1
    logprobs: Optional[Union[bool, int]] = None
    seed: Optional[int] = None

    def __post_init__(self):
        if self.top_k != -1 and self.top_k < 1:
            raise ValueError("top_k must be -1 (disabled) or >= 1")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in range (0.0, 1.0]")
        if self.n < 1:
            raise ValueError("n must be >= 1")
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be >= 1")
