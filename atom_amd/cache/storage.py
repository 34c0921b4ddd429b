"""Device memory of the cache: the pages of every run of a layer that keeps keys and
values, and the state tensors of every run that keeps a per-request state.

Sizing follows the reference's rule of reserving fixed per-request needs first and
giving the rest to the pages that grow with context
(atom/model_ops/attentions/sub_pool_spec.py:203-246): window groups and state are sized
by ``max_num_seqs``; groups that keep every key get the remaining bytes.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..engine.context import KVBinding, StateBinding
from ..parts.base import KVCacheNeed, StateNeed
from .manager import GroupSpec


@dataclass
class CachePlan:
    groups: list[GroupSpec]
    run_group: list[int | None]   # per run of the order: its group, or None if it keeps no pages
    bytes_per_page: list[int]     # per group, summed over the runs that own pages in it

    def total_bytes(self) -> int:
        return sum(g.num_pages * b for g, b in zip(self.groups, self.bytes_per_page))


def _elem_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


def group_runs(model) -> tuple[list[int | None], list[int | None]]:
    """(window of each group, group of each run).  Runs whose mixers keep keys with the same
    window share a group, that is, block tables."""
    windows: list[int | None] = []
    run_group: list[int | None] = []
    for run in model.order:
        need = model.blocks[run.layer].mixer.cache_need()
        if isinstance(need, KVCacheNeed):
            if need.window not in windows:
                windows.append(need.window)
            run_group.append(windows.index(need.window))
        else:
            run_group.append(None)
    return windows, run_group


def plan_cache(model, page_size: int, dtype: torch.dtype, *, num_pages: int | None = None,
               budget_bytes: int | None = None, max_num_seqs: int = 1, max_model_len: int = 0,
               max_num_batched_tokens: int = 0) -> CachePlan:
    """Either ``num_pages`` for every group, or a byte budget to divide."""
    windows, run_group = group_runs(model)
    per_page = [0] * len(windows)
    for run, group in zip(model.order, run_group):
        if group is None or run.reads_run is not None:
            continue
        need = model.blocks[run.layer].mixer.cache_need()
        per_page[group] += 2 * need.num_kv_heads * need.head_dim * page_size * _elem_size(dtype)
    if num_pages is not None:
        counts = [num_pages] * len(windows)
    else:
        if budget_bytes is None:
            raise ValueError("plan_cache needs num_pages or budget_bytes")
        full_pages = -(-max_model_len // page_size)
        counts = [0] * len(windows)
        left = budget_bytes
        for gi, w in enumerate(windows):
            if w is None:
                continue
            per_req = min(full_pages, -(-(w + max_num_batched_tokens) // page_size) + 1)
            counts[gi] = per_req * max_num_seqs
            left -= counts[gi] * per_page[gi]
        full = [gi for gi, w in enumerate(windows) if w is None]
        if full:
            pages = max(0, left) // max(1, sum(per_page[gi] for gi in full))
            for gi in full:
                counts[gi] = pages
    groups = [GroupSpec(page_size, c, w) for c, w in zip(counts, windows)]
    return CachePlan(groups, run_group, per_page)


class CacheStorage:
    """Allocates what the plan says and hands each run its binding."""

    def __init__(self, model, plan: CachePlan, num_state_slots: int, device, dtype: torch.dtype):
        self.plan = plan
        self.bindings: list = []
        self.state_tensors: list[torch.Tensor] = []
        for i, (run, group) in enumerate(zip(model.order, plan.run_group)):
            need = model.blocks[run.layer].mixer.cache_need()
            if isinstance(need, KVCacheNeed):
                if run.reads_run is not None:
                    src = self.bindings[run.reads_run]
                    self.bindings.append(KVBinding(src.group, src.k_cache, src.v_cache, writes=False))
                    continue
                g = plan.groups[group]
                k = torch.zeros((g.num_pages, need.num_kv_heads, g.page_size, need.head_dim), dtype=dtype, device=device)
                v = torch.zeros((g.num_pages, need.num_kv_heads, need.head_dim, g.page_size), dtype=dtype, device=device)
                self.bindings.append(KVBinding(group, k, v, writes=True))
            elif isinstance(need, StateNeed):
                if run.reads_run is not None:
                    raise ValueError(f"run {i}: a state cannot be read from another run")
                state = torch.zeros((num_state_slots, *need.shape), dtype=need.dtype, device=device)
                self.state_tensors.append(state)
                self.bindings.append(StateBinding(state))
            else:
                self.bindings.append(None)

    def reset_state(self, slots: list[int]) -> None:
        """Zeroes the state of slots whose requests start in this step."""
        if not slots or not self.state_tensors:
            return
        idx = torch.tensor(slots, dtype=torch.long, device=self.state_tensors[0].device)
        for state in self.state_tensors:
            state.index_fill_(0, idx, 0)
