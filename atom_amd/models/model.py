"""A causal language model as data: an embedding, blocks chosen layer by layer, the
order in which they run, a final norm and a head.  Nothing here is specific to an
architecture; an architecture is a function from its configuration to a ``ModelSpec``.
"""

from __future__ import annotations

import re
from dataclasses import dataclass, field

import torch

from ..parts.base import BLOCKS, EMBEDDINGS, HEADS, NORMS, Part, PartChoice


@dataclass(frozen=True)
class LayerRun:
    """One entry of the running order.  ``layer`` may appear in several runs (shared
    weights, each run with a cache of its own); ``reads_run`` names an earlier run
    (by its place in the order) whose cache this run reads instead of writing one."""

    layer: int
    reads_run: int | None = None


@dataclass
class ModelSpec:
    vocab_size: int
    hidden_size: int
    blocks: list[PartChoice]                 # one per layer; kind from the BLOCKS registry
    final_norm: PartChoice
    tie_word_embeddings: bool = False
    # the embedding and the head, chosen from their registries like every other part; they are built with
    # vocab_size and hidden_size (the head also with tied_to) beside what the choice names
    embedding: PartChoice = field(default_factory=lambda: PartChoice("token_embedding"))
    head: PartChoice = field(default_factory=lambda: PartChoice("lm_head"))
    order: list[LayerRun] | None = None      # default: every layer once, in turn
    max_positions: int = 0
    embedding_prefix: str = "model.embed_tokens"
    layer_prefix: str = "model.layers.{}"
    final_norm_prefix: str = "model.norm"
    head_prefix: str = "lm_head"
    ignorable: tuple[str, ...] = ()          # checkpoint tensors that may be present and are not used
    # checkpoint tensors dropped by the form of their name (atom/model_loader/weight_names.py:160-188): cache
    # scales, rotation tables that a checkpoint still carries, whatever starts with a prefix the model names
    drop_suffixes: tuple[str, ...] = ("kv_scale",)
    drop_substrings: tuple[str, ...] = ("inv_freq",)
    drop_prefixes: tuple[str, ...] = ()

    def running_order(self) -> list[LayerRun]:
        return list(self.order) if self.order is not None else [LayerRun(i) for i in range(len(self.blocks))]


class CausalLM(Part):
    def __init__(self, spec: ModelSpec):
        super().__init__("")
        self.spec = spec
        self.embedding = spec.embedding.build(EMBEDDINGS, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size,
                                              prefix=spec.embedding_prefix)
        self.blocks = [choice.build(BLOCKS, prefix=spec.layer_prefix.format(i)) for i, choice in enumerate(spec.blocks)]
        self.final_norm = spec.final_norm.build(NORMS, prefix=spec.final_norm_prefix)
        self.head = spec.head.build(HEADS, vocab_size=spec.vocab_size, hidden_size=spec.hidden_size,
                                    tied_to=self.embedding if spec.tie_word_embeddings else None,
                                    prefix=spec.head_prefix)
        self.order = spec.running_order()
        for i, run in enumerate(self.order):
            if not (0 <= run.layer < len(self.blocks)):
                raise ValueError(f"run {i} names layer {run.layer}, the model has {len(self.blocks)}")
            if run.reads_run is not None:
                if not (0 <= run.reads_run < i):
                    raise ValueError(f"run {i} reads the cache of run {run.reads_run}, which does not come before it")
                if self.order[run.reads_run].reads_run is not None:
                    raise ValueError(f"run {i} reads run {run.reads_run}, which has no cache of its own")
                a = self.blocks[run.layer].mixer.cache_need()
                b = self.blocks[self.order[run.reads_run].layer].mixer.cache_need()
                if a != b:
                    raise ValueError(f"run {i} cannot read the cache of run {run.reads_run}: {a} differs from {b}")
        self.ignorable = set(spec.ignorable)
        if spec.tie_word_embeddings:
            self.ignorable.add(f"{spec.head_prefix}.weight")
        head, _, tail = spec.layer_prefix.partition("{}")
        self._layer_name = re.compile(re.escape(head) + r"(\d+)" + (re.escape(tail) if tail else "") + r"\.")
        self.dtype: torch.dtype | None = None
        self.device: torch.device | None = None

    def children(self):
        return [self.embedding, *self.blocks, self.final_norm, self.head]

    def drops(self, name: str) -> str | None:
        """Why a checkpoint tensor that no parameter names is left aside without an error, or None if it
        is not: the exact names of ``ignorable``, the name forms of the reference's checkpoint rewriter
        (atom/model_loader/weight_names.py:160-188: ``*kv_scale``, ``*inv_freq*``, model-declared
        prefixes) and the tensors of layers beyond the model's last (``_is_past_last_layer``, :197-201:
        a checkpoint run with fewer layers than it holds)."""
        spec = self.spec
        if name in self.ignorable:
            return "not used by this model"
        if any(name.endswith(s) for s in spec.drop_suffixes):
            return "a cache scale"
        if any(s in name for s in spec.drop_substrings):
            return "a table the engine computes itself"
        if any(name.startswith(p) for p in spec.drop_prefixes):
            return "under a prefix the model leaves out"
        match = self._layer_name.search(name)
        if match is not None and int(match.group(1)) >= len(self.blocks):
            return f"of a layer beyond the model's {len(self.blocks)}"
        return None

    @property
    def vocab_size(self) -> int:
        return self.spec.vocab_size

    def forward(self, ctx, token_ids: torch.Tensor, caches: list, want_rows: torch.Tensor | None):
        """Runs the step's tokens through every run of the order; returns float32 logits
        at ``want_rows`` (None: nothing is wanted, the cache is only filled)."""
        hidden = self.embedding.forward(ctx, token_ids)
        residual = None
        for run, cache in zip(self.order, caches):
            hidden, residual = self.blocks[run.layer].forward(ctx, hidden, residual, cache)
        if want_rows is None or want_rows.numel() == 0:
            return None
        if not self.final_norm.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        normed = self.final_norm.forward_rows(ctx, hidden, residual, want_rows)
        return self.head.forward(ctx, normed)
