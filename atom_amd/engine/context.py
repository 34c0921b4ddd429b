"""What one step hands to the parts: the kernel library, the flat token axis and,
per group of layers that share block tables, where keys are written and read."""

from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..kernels.hip import AttentionMeta


@dataclass
class KVBinding:
    """The pages of one run of a layer.  ``writes`` is False for a run that reads the
    keys and values another run wrote."""

    group: int
    k_cache: torch.Tensor  # [num_pages, Hkv, page_size, D]
    v_cache: torch.Tensor  # [num_pages, Hkv, D, page_size]
    writes: bool = True


@dataclass
class StateBinding:
    """The per-request state of one run of a layer: ``state[slot]`` belongs to the request
    that holds ``slot``; it is zero when the request's first tokens arrive."""

    state: torch.Tensor  # [num_slots, *shape]


@dataclass
class StepContext:
    ops: object
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_seqs: int
    positions: torch.Tensor                      # int32 [T]
    attention: dict[int, AttentionMeta] = field(default_factory=dict)
    slot_mappings: dict[int, torch.Tensor] = field(default_factory=dict)  # int32 [T] per group
    # host-side copies, for mixers that walk requests themselves
    seq_starts: list[int] = field(default_factory=list)   # first row of each request in the token axis
    seq_lens: list[int] = field(default_factory=list)     # rows of each request in this step
    seq_cached: list[int] = field(default_factory=list)   # tokens of each request before this step
    state_slots: list[int] = field(default_factory=list)  # state slot of each request
