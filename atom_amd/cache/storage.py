"""Device memory of the cache: what every run of a layer keeps between steps, allocated
as its cache kind says (``cache.kinds``): pages of keys and values, per-request state,
or whatever another registered kind holds.

Sizing follows the reference's rule of reserving fixed per-request needs first and
giving the rest to the pages that grow with context
(atom/model_ops/attentions/sub_pool_spec.py:203-246): window groups and per-slot memory
are sized by ``max_num_seqs``; groups that keep every key get the remaining bytes.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .kinds import CacheKind, kind_of
from .manager import GroupSpec


@dataclass
class CachePlan:
    groups: list[GroupSpec]
    run_group: list[int | None]   # per run of the order: its group, or None if it keeps no pages
    bytes_per_page: list[int]     # per group, summed over the runs that own pages in it
    bytes_per_slot: int = 0       # memory of fixed size per request, summed over the runs that own some

    def total_bytes(self, num_slots: int = 0) -> int:
        return sum(g.num_pages * b for g, b in zip(self.groups, self.bytes_per_page)) + num_slots * self.bytes_per_slot


def group_runs(model) -> tuple[list[int | None], list[int | None]]:
    """(window of each group, group of each run).  Runs whose mixers keep pages with the same
    window share a group, that is, block tables."""
    windows: list[int | None] = []
    run_group: list[int | None] = []
    for run in model.order:
        need = model.blocks[run.layer].mixer.cache_need()
        kind = kind_of(need)
        if kind is not None and kind.paged:
            window = kind.window(need)
            if window not in windows:
                windows.append(window)
            run_group.append(windows.index(window))
        else:
            run_group.append(None)
    return windows, run_group


def plan_cache(model, page_size: int, dtype: torch.dtype, *, num_pages: int | None = None,
               budget_bytes: int | None = None, max_num_seqs: int = 1, max_model_len: int = 0,
               max_num_batched_tokens: int = 0) -> CachePlan:
    """Either ``num_pages`` for every group, or a byte budget to divide."""
    windows, run_group = group_runs(model)
    per_page = [0] * len(windows)
    per_slot = 0
    for run, group in zip(model.order, run_group):
        if run.reads_run is not None:
            continue
        mixer = model.blocks[run.layer].mixer
        need = mixer.cache_need()
        kind = kind_of(need)
        if kind is None:
            continue
        if group is not None:
            problem = mixer.page_size_problem(page_size)
            if problem:
                raise ValueError(f"cache pages of {page_size} tokens do not suit layer {run.layer} "
                                 f"({type(mixer).__name__}): {problem}")
        per_slot += kind.request_bytes(need, dtype)
        if group is not None:
            per_page[group] += kind.page_bytes(need, page_size, dtype)
    if num_pages is not None:
        counts = [num_pages] * len(windows)
    else:
        if budget_bytes is None:
            raise ValueError("plan_cache needs num_pages or budget_bytes")
        full_pages = -(-max_model_len // page_size)
        counts = [0] * len(windows)
        left = budget_bytes - per_slot * max_num_seqs
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
    return CachePlan(groups, run_group, per_page, per_slot)


class CacheStorage:
    """Allocates what the plan says and hands each run its binding."""

    def __init__(self, model, plan: CachePlan, num_state_slots: int, device, dtype: torch.dtype):
        self.plan = plan
        self.device = torch.device(device)
        self.bindings: list = []
        self._owned: list[tuple] = []    # (kind, binding) of every run that owns memory
        for i, (run, group) in enumerate(zip(model.order, plan.run_group)):
            need = model.blocks[run.layer].mixer.cache_need()
            kind = kind_of(need)
            if kind is None:
                self.bindings.append(None)
                continue
            if run.reads_run is not None:
                try:
                    self.bindings.append(kind.share(self.bindings[run.reads_run]))
                except ValueError as e:
                    raise ValueError(f"run {i}: {e}") from None
                continue
            g = plan.groups[group] if group is not None else None
            binding = kind.allocate(need, group=group, num_pages=g.num_pages if g else 0,
                                    page_size=g.page_size if g else 0, num_slots=num_state_slots, device=device,
                                    dtype=dtype)
            self.bindings.append(binding)
            self._owned.append((kind, binding))
        # kinds that clear something when a request starts (the others inherit the base's empty method)
        self._resettable = [(k, b) for k, b in self._owned if type(k).reset is not CacheKind.reset]

    @property
    def state_tensors(self) -> list[torch.Tensor]:
        """The per-request state tensors, in running order."""
        return [b.state for _, b in self._owned if hasattr(b, "state")]

    def reset_state(self, slots: list[int]) -> None:
        """Clears the per-request memory of slots whose requests start in this step."""
        if not slots or not self._resettable:
            return
        idx = torch.tensor(slots, dtype=torch.long, device=self.device)
        for kind, binding in self._resettable:
            kind.reset(binding, idx)
