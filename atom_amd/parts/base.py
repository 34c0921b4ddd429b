"""What a model is put together from.

A *part* owns parameters and computes; it is given every size and constant it needs
and never learns which model it sits in.  Five kinds are chosen layer by layer from a
configuration, each through a registry of its own (two more, the embedding and the head, once a model):

    mixer              mixes information across positions (attention, or anything with
                       a cache or a per-request state of its own)
    feed-forward       acts on each token alone (dense gated MLP, experts)
    norm               normalises a row, optionally adding the residual stream first
    position encoding  what a mixer applies to queries and keys (rotary tables)
    block              arranges norm, mixer and feed-forward around the residual stream

A part declares its parameters as ``ParamSpec``s; the loader fills them from checkpoint
tensors by name (several checkpoint tensors may be stacked into one parameter).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable

import torch


# ----------------------------------------------------------------------------- parameters


@dataclass(frozen=True)
class Source:
    """One checkpoint tensor that lands in rows [offset, offset + rows) of a parameter."""

    name: str      # relative to the part's prefix, e.g. "q_proj.weight"
    offset: int
    rows: int


@dataclass(frozen=True)
class ParamSpec:
    """A parameter of a part.

    kind: 'matrix' (kept in the serving type: bfloat16, or float32 on the 32-bit path; a
          checkpoint tensor stored in 32-bit stays 32-bit), 'vector' (norm weights and biases,
          always float32), 'table' (integers, int32).
    init: how the random-weights mode draws each source tensor: 'normal' N(0, std),
          'one_plus_normal' 1 + N(0, norm_std), 'zeros'.
    """

    shape: tuple[int, ...]
    kind: str
    sources: tuple[Source, ...]
    init: str = "normal"

    @staticmethod
    def single(name: str, shape: tuple[int, ...], kind: str = "matrix", init: str = "normal") -> "ParamSpec":
        return ParamSpec(tuple(shape), kind, (Source(name, 0, shape[0]),), init)

    @staticmethod
    def stacked(names_rows: list[tuple[str, int]], trailing: tuple[int, ...], kind: str = "matrix",
                init: str = "normal") -> "ParamSpec":
        sources, offset = [], 0
        for name, rows in names_rows:
            sources.append(Source(name, offset, rows))
            offset += rows
        return ParamSpec((offset, *trailing), kind, tuple(sources), init)


class Part:
    """Base of every part: a name prefix, declared parameters, children."""

    def __init__(self, prefix: str = ""):
        self.prefix = prefix
        self.params: dict[str, torch.Tensor] = {}

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def children(self) -> list["Part"]:
        return []

    def walk(self):
        yield self
        for child in self.children():
            yield from child.walk()

    def full_name(self, local: str) -> str:
        return f"{self.prefix}.{local}" if self.prefix else local

    def finalize(self, device, dtype) -> None:
        """Called once after the parameters are bound; builds derived tables."""

    def p(self, name: str) -> torch.Tensor | None:
        return self.params.get(name)


# ----------------------------------------------------------------------------- cache needs


@dataclass(frozen=True)
class KVCacheNeed:
    """A mixer that keeps keys and values of past tokens in pages.  ``window`` None = all keys."""

    num_kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class StateNeed:
    """A mixer that keeps a state of fixed size per request (zeroed when a request starts)."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


# ----------------------------------------------------------------------------- the four computing kinds


class Norm(Part):
    #: True when the norm hands ``x`` to ``ctx.ops.rmsnorm`` as it is: a mixer or feed-forward may return
    #: a product that is still a sum of slices (``ops.linear(..., defer=True)``), which that kernel adds
    #: while it reads.  Other norms get a tensor (the block calls ``ops.materialize`` first).
    accepts_deferred = False

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_residual(self, ctx, x: torch.Tensor, residual: torch.Tensor | None):
        """Adds ``x`` to the residual stream (starting it when None) and returns
        (norm of the sum, the residual stream)."""
        raise NotImplementedError

    def forward_rows(self, ctx, x, residual, rows: torch.Tensor) -> torch.Tensor:
        """Norm of ``x + residual`` at the given rows only; nothing else is written."""
        raise NotImplementedError


class PositionEncoding(Part):
    """Provides what the mixer's kernels need to encode positions."""


class Embedding(Part):
    """Token ids to the model's first hidden rows.  Built with ``vocab_size``, ``hidden_size`` and whatever
    else its choice names (a multiplier, say)."""

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    """Normed hidden rows to float32 logits over the vocabulary.  Built with ``vocab_size``, ``hidden_size``,
    ``tied_to`` (the model's embedding when the head shares its table, else None) and whatever else its choice
    names (a cap on the logits, a bias)."""

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Mixer(Part):
    #: True when ``forward`` hands its input to ``ctx.ops.linear`` / ``linear_silu`` as it is and reads nothing of
    #: it but ``shape``, ``dtype`` and ``device``: the norm before the mixer may then be left to that product
    #: (the input is a ``PendingNorm``).  Other mixers always get a tensor.
    accepts_deferred = False
    #: True when ``forward`` launches the same kernels whatever the batch holds and reads the batch
    #: only through device arrays of ``ctx``: a decode step of such mixers may be replayed as a HIP graph
    graph_safe = False

    def cache_need(self):
        """What this mixer keeps between steps: a ``KVCacheNeed``, a ``StateNeed``, an object of any other
        registered cache kind (``cache.kinds.register_cache_kind``), or None."""
        return None

    def page_size_problem(self, page_size: int) -> str | None:
        """Why this mixer's kernels cannot work with cache pages of ``page_size`` tokens, or None if they can.
        Asked when the cache is planned, so that a page size is refused before anything is allocated."""
        return None

    def step_key(self):
        """Mixers that return equal keys (hashable, not None) share one ``prepare_step`` a step; None:
        this mixer prepares nothing."""
        return None

    def prepare_step(self, batch) -> dict:
        """Integer arrays (numpy int32, any shape) that this mixer's kernels want on the device for this
        step, by name, derived on the host from ``batch`` (an ``engine.context.BatchView``).  The engine
        copies them with the step's other arrays in its one transfer and hands them back as device
        tensors: ``ctx.prepared[self.step_key()][name]``.  For a batch with ``batch.replayed`` set the
        arrays' shapes may depend on ``batch.q_lens`` only: they live in a captured graph's fixed buffer."""
        return {}

    def forward(self, ctx, x: torch.Tensor, cache) -> torch.Tensor:
        """``cache`` is what the engine bound to this run of the layer: a ``KVBinding`` for a
        ``KVCacheNeed``, a ``StateBinding`` for a ``StateNeed``, else None."""
        raise NotImplementedError


class FeedForward(Part):
    #: as ``Mixer.accepts_deferred``
    accepts_deferred = False

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    def forward(self, ctx, hidden: torch.Tensor, residual: torch.Tensor | None, cache):
        """Returns (hidden, residual) for the next block."""
        raise NotImplementedError

    @property
    def mixer(self) -> Mixer:
        raise NotImplementedError


# ----------------------------------------------------------------------------- registries


class Registry:
    """Name -> factory.  Registering a taken name is an error unless ``replace`` is set."""

    def __init__(self, kind: str):
        self.kind = kind
        self._items: dict[str, Callable] = {}

    def register(self, name: str, factory: Callable | None = None, *, replace: bool = False):
        def put(f):
            if name in self._items and not replace:
                raise KeyError(f"{self.kind} '{name}' is already registered")
            self._items[name] = f
            return f

        return put(factory) if factory is not None else put

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> Callable:
        if name not in self._items:
            raise KeyError(f"unknown {self.kind} '{name}'; known: {sorted(self._items)}")
        return self._items[name]

    def build(self, name: str, **kwargs):
        return self.get(name)(**kwargs)

    def names(self) -> list[str]:
        return sorted(self._items)


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block")
EMBEDDINGS = Registry("embedding")
HEADS = Registry("head")


@dataclass(frozen=True)
class PartChoice:
    """A part chosen by name with its parameters, as a configuration writes it down."""

    kind: str
    args: dict = field(default_factory=dict)

    def build(self, registry: Registry, **extra):
        return registry.build(self.kind, **{**self.args, **extra})
