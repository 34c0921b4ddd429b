"""A request's state as the scheduler sees it (atom/model_engine/sequence.py:15-260)."""

from __future__ import annotations

import itertools
import time
from enum import Enum, auto

from ..sampling.params import SamplingParams


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()
    ABORTED = auto()


class Sequence:
    counter = itertools.count()

    def __init__(self, token_ids: list[int], sampling_params: SamplingParams | None = None,
                 stop_token_sequences: list[list[int]] | None = None, seed: int | None = None):
        sp = sampling_params or SamplingParams()
        self.id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        self.num_cached_tokens = 0          # tokens whose keys and values are in the cache
        self.is_partial_prefill = False
        self.awaits_token = False           # the last token is a placeholder for one still on the device
        self.sampling_params = sp
        self.temperature = sp.temperature
        self.max_tokens = sp.max_tokens
        self.ignore_eos = sp.ignore_eos
        self.stop_token_sequences = stop_token_sequences or []
        self.seed = seed if seed is not None else (sp.seed if sp.seed is not None else self.id)
        self.leave_reason = ""
        self.logprobs: list[float] = []
        self.num_preemptions = 0
        self.num_prefix_hit_tokens = 0      # tokens of the last admission that came from the prefix cache
        self.arrive_time = time.time()
        self.first_token_time = 0.0
        self.leave_time = 0.0

    def __len__(self) -> int:
        return len(self.token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def completion_token_ids(self) -> list[int]:
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def is_finished(self) -> bool:
        return self.status == SequenceStatus.FINISHED

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(int(token_id))

    # A step may be scheduled before the host has read the token that the step before it sampled (the
    # reference appends a placeholder and overwrites it, atom/model_engine/scheduler.py:2127-2133,
    # 2196-2247): the sequence then ends in a placeholder until ``resolve_placeholder``.
    PLACEHOLDER = 0

    def append_placeholder(self) -> None:
        if self.awaits_token:
            raise AssertionError(f"sequence {self.id} already ends in a token that is not known yet")
        self.token_ids.append(self.PLACEHOLDER)
        self.awaits_token = True

    def resolve_placeholder(self, token_id: int) -> None:
        if not self.awaits_token:
            raise AssertionError(f"sequence {self.id} awaits no token")
        self.token_ids[-1] = int(token_id)
        self.awaits_token = False
