"""The kinds of memory a mixer may keep between steps, and what the engine binds to a run
of a layer for each.

A mixer names its need with an object (``KVCacheNeed``, ``StateNeed``, or one of a type
registered here); the type of that object selects a ``CacheKind``, which says how such
memory is sized, allocated, shared between runs and cleared for a new request.  Planning
and allocation (``cache.storage``) and the engine go through this registry only, so another
kind of memory (a latent cache, a ring of recent tokens) is registered, not patched in.

The reference plans its pools from per-class specs in the same spirit
(atom/model_ops/attentions/sub_pool_spec.py:49-246: STATE classes sized by
``max_num_seqs``, one PAGE class taking the rest).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import KVCacheNeed, StateNeed


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


def _elem_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


class CacheKind:
    """How one kind of memory is planned and bound.  ``paged`` kinds live in pages that the cache
    manager hands out per request (runs with the same ``window`` share block tables); the others hold
    a fixed amount per state slot."""

    paged = False

    def window(self, need) -> int | None:
        """Paged kinds: how many of the latest tokens a later query can still see (None: all)."""
        return None

    def keeps_every_token(self, need) -> bool:
        """True if everything a request's earlier tokens left is still there later, in pages: only then
        can a new request take over pages that already hold its beginning (the prefix cache)."""
        return False

    def page_bytes(self, need, page_size: int, dtype: torch.dtype) -> int:
        return 0

    def request_bytes(self, need, dtype: torch.dtype) -> int:
        """Bytes held per state slot, whatever the context length."""
        return 0

    def allocate(self, need, *, group: int | None, num_pages: int, page_size: int, num_slots: int, device,
                 dtype: torch.dtype):
        raise NotImplementedError

    def share(self, binding):
        """What a run gets that reads the memory of the run that owns ``binding``."""
        raise ValueError(f"{type(self).__name__}: this kind of memory cannot be read from another run")

    def reset(self, binding, slots: torch.Tensor) -> None:
        """Clears the per-request part of ``binding`` for the state slots in ``slots`` (int64, on the device),
        whose requests start in the coming step."""


class PagedKeysValues(CacheKind):
    paged = True

    def window(self, need):
        return need.window

    def keeps_every_token(self, need):
        return need.window is None

    def page_bytes(self, need, page_size, dtype):
        return 2 * need.num_kv_heads * need.head_dim * page_size * _elem_size(dtype)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        k = torch.zeros((num_pages, need.num_kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
        v = torch.zeros((num_pages, need.num_kv_heads, need.head_dim, page_size), dtype=dtype, device=device)
        return KVBinding(group, k, v, writes=True)

    def share(self, binding):
        return KVBinding(binding.group, binding.k_cache, binding.v_cache, writes=False)


class SlotState(CacheKind):
    def request_bytes(self, need, dtype):
        n = 1
        for s in need.shape:
            n *= int(s)
        return n * _elem_size(need.dtype)

    def allocate(self, need, *, group, num_pages, page_size, num_slots, device, dtype):
        return StateBinding(torch.zeros((num_slots, *need.shape), dtype=need.dtype, device=device))

    def reset(self, binding, slots):
        binding.state.index_fill_(0, slots, 0)


_KINDS: dict[type, CacheKind] = {}


def register_cache_kind(need_type: type, kind: CacheKind, *, replace: bool = False) -> None:
    if need_type in _KINDS and not replace:
        raise KeyError(f"a cache kind for {need_type.__name__} is already registered")
    _KINDS[need_type] = kind


def unregister_cache_kind(need_type: type) -> None:
    _KINDS.pop(need_type, None)


def kind_of(need) -> CacheKind | None:
    """The kind that handles ``need`` (None for a mixer that keeps nothing)."""
    if need is None:
        return None
    for cls in type(need).__mro__:
        if cls in _KINDS:
            return _KINDS[cls]
    raise KeyError(f"no cache kind is registered for {type(need).__name__}; known: "
                   f"{sorted(t.__name__ for t in _KINDS)}")


register_cache_kind(KVCacheNeed, PagedKeysValues())
register_cache_kind(StateNeed, SlotState())
