"""The step function and what it stands on: the model, the cache manager, the cache's
device memory.

``EngineCore.step`` takes a batch of (request, its next tokens, the places whose logits
are wanted): portions of prompts beside single decoded tokens, cut anywhere.  It runs
exactly those tokens as one flat batch against the cache that earlier steps left and
returns float32 logits at the wanted places, in the order of the entries.

The reference's step (atom/model_engine/model_runner.py:3325-3415) takes either prompt
portions or decode tokens; its batch record already lays prompt portions before decode
tokens on one token axis (model_runner.py:441-449, scheduler.py:353-358), which is the
layout used here for both at once.  The derived arrays are the reference's
(atom/model_ops/attentions/backends.py:374-497): positions ``cached .. cached+n-1``,
``slot = block_table[pos // bs] * bs + pos % bs``, ``cu_seqlens_q``, ``context_lens``,
zero-padded block tables.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.kinds import kind_of
from ..cache.manager import CacheManager
from ..cache.storage import CachePlan, CacheStorage
from .context import BatchView, StepContext, pack_int32


@dataclass
class StepEntry:
    req_id: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)   # places among ``tokens`` whose logits are wanted
    reserve: int | None = None                      # pages are held up to this length (admission)
    # The entry's one token is row ``feed`` of ``EngineCore.sampled`` (what the last step's sampler wrote
    # there) and is read on the device; ``tokens`` then holds a placeholder.  The reference feeds decode
    # steps the same way (atom/model_ops/decode_input_ids.py:1-32, model_runner.py:553-560).
    feed: int | None = None


class EngineCore:
    def __init__(self, model, ops, plan: CachePlan, max_num_seqs: int, device, dtype: torch.dtype,
                 graph_sizes: list[int] | None = None, max_model_len: int = 0, prefix_caching: bool = False,
                 graph_prefill_sizes: list[int] | None = None, graph_prefill_slots: int | None = None):
        self.model = model
        self.ops = ops
        self.device = torch.device(device)
        self.dtype = dtype
        self.plan = plan
        # the prefix cache needs every mixer's memory to be pages that keep all that earlier tokens left
        needs = [model.blocks[run.layer].mixer.cache_need() for run in model.order]
        self.prefix_caching = bool(prefix_caching and plan.groups and all(
            kind_of(n).keeps_every_token(n) for n in needs if n is not None))
        self.manager = CacheManager(plan.groups, max_num_seqs, prefix_caching=self.prefix_caching)
        self.storage = CacheStorage(model, plan, max_num_seqs, self.device, dtype)
        self.lengths: dict[object, int] = {}   # tokens of each live request that are in the cache
        self.max_positions = model.spec.max_positions
        self.steps_run = 0
        self._fresh_slots: list[int] = []      # slots claimed since the last step: zeroed before it runs
        # where a sampler leaves its tokens when the next step is to read them on the device (StepEntry.feed)
        self.sampled = torch.zeros(max(1, max_num_seqs), dtype=torch.int32, device=self.device)
        # mixers that want arrays of their own on the device every step, one per distinct step key
        self.preparers: dict = {}
        for run in model.order:
            mixer = model.blocks[run.layer].mixer
            key = mixer.step_key()
            if key is not None and key not in self.preparers:
                self.preparers[key] = mixer
        self._staging = _Staging(self.device)
        # decode-only steps replay a captured HIP graph per batch-size bucket (None: always eager)
        self.graphs = None
        if graph_sizes:
            from .graphs import DecodeGraphs

            graphs = DecodeGraphs(self, graph_sizes, max_model_len or self.max_positions, graph_prefill_sizes,
                                  **({} if graph_prefill_slots is None else {"prefill_slots": graph_prefill_slots}))
            self.graphs = graphs if graphs.usable else None

    # ------------------------------------------------------------------ requests

    def is_live(self, req_id) -> bool:
        return req_id in self.lengths

    def num_cached(self, req_id) -> int:
        return self.lengths.get(req_id, 0)

    def open(self, req_id) -> None:
        """Registers a request: it holds a state slot from now to ``close``.  A step opens
        unknown requests itself; a scheduler opens them when it admits them, to take pages."""
        if req_id in self.lengths:
            return
        self.manager.open(req_id)
        self.lengths[req_id] = 0
        self._fresh_slots.append(self.manager.state_slot(req_id))

    def match_prefix(self, req_id, token_ids) -> int:
        """For a request just opened: takes cached pages that already hold the beginning of ``token_ids``
        and returns how many tokens need not be run (0 without a prefix cache)."""
        if not self.prefix_caching or self.lengths.get(req_id, 0) != 0:
            return 0
        covered = self.manager.match_prefix(req_id, token_ids)
        self.lengths[req_id] = covered
        return covered

    def close(self, req_id) -> None:
        """Ends a request: its pages and state slot go back."""
        if req_id in self.lengths:
            del self.lengths[req_id]
            self.manager.close(req_id)

    def can_step(self, entries: list[StepEntry]) -> bool:
        """Whether the pools hold enough free pages (and slots) for all entries at once."""
        need = [0] * len(self.plan.groups)
        new_requests = 0
        for e in entries:
            cached = self.num_cached(e.req_id)
            if e.req_id not in self.lengths:
                new_requests += 1
            for gi, n in enumerate(self.manager.pages_missing(e.req_id, cached, cached + len(e.tokens), e.reserve)):
                need[gi] += n
        return (new_requests <= self.manager.slots.num_free
                and all(n <= pool.num_free for n, pool in zip(need, self.manager.pools)))

    # ------------------------------------------------------------------ the step

    def step(self, entries: list[StepEntry]) -> torch.Tensor | None:
        if not entries:
            return None
        ids = [e.req_id for e in entries]
        if len(set(ids)) != len(ids):
            raise ValueError("a request appears twice in one step")
        vocab = self.model.vocab_size
        for e in entries:
            if not e.tokens:
                raise ValueError(f"request {e.req_id!r}: a step entry needs at least one token")
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:
                raise ValueError(f"request {e.req_id!r}: token id outside [0, {vocab})")
            if e.feed is not None and (len(e.tokens) != 1 or not 0 <= e.feed < self.sampled.numel()):
                raise ValueError(f"request {e.req_id!r}: a token read on the device must be the entry's only one "
                                 f"and name one of the {self.sampled.numel()} sampled rows")
            if any(w < 0 or w >= len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.req_id!r}: a wanted place is outside its {len(e.tokens)} tokens")
            end = self.num_cached(e.req_id) + len(e.tokens)
            if self.max_positions and end > self.max_positions:
                raise ValueError(f"request {e.req_id!r}: {end} tokens exceed the model's {self.max_positions} positions")
        if not self.can_step(entries):
            from ..cache.manager import OutOfPages
            raise OutOfPages("the cache cannot hold this step's tokens")

        # prompt portions first, single tokens after them (stable)
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) == 1)
        for e in entries:
            self.open(e.req_id)
            cached = self.lengths[e.req_id]
            self.manager.cover(e.req_id, cached, cached + len(e.tokens), e.reserve)
        self.storage.reset_state(self._fresh_slots)
        self._fresh_slots = []

        cached_now = [self.lengths[e.req_id] for e in entries]
        if self.graphs is not None and self.graphs.accepts(entries, cached_now):
            logits = self.graphs.run(entries, cached_now)
        else:
            ctx, token_ids, want_rows = self._build(entries, order)
            logits = self.model.forward(ctx, token_ids, self.storage.bindings, want_rows)

        for e in entries:
            self.lengths[e.req_id] += len(e.tokens)
            self.manager.commit(e.req_id, self.lengths[e.req_id], e.tokens if self.prefix_caching else None,
                                last_unknown=e.feed is not None)
        self.steps_run += 1
        return logits

    def resolve(self, req_id, position: int, token: int) -> None:
        """Tells the cache's bookkeeping the value of a token that a step read on the device
        (``StepEntry.feed``); a request that has ended meanwhile, or whose token no step has read, is skipped."""
        if req_id in self.lengths and self.manager.awaited_position(req_id) == position:
            self.manager.amend(req_id, position, token)

    def batch_view(self, q_lens: list[int], cached: list[int], replayed: bool = False, prefill_capacity: int = 0,
                   prefill_slots: int = 0, num_prefill: int | None = None) -> BatchView:
        return BatchView(ops=self.ops, dtype=self.dtype, q_lens=q_lens, cached=cached,
                         num_prefill=sum(1 for n in q_lens if n > 1) if num_prefill is None else num_prefill,
                         page_sizes=[g.page_size for g in self.manager.groups], replayed=replayed,
                         prefill_capacity=prefill_capacity, prefill_slots=prefill_slots)

    def _build(self, entries: list[StepEntry], order: list[int]):
        """Every array of the step in one int32 host buffer (pinned), one copy to the device, and the
        context whose tensors are views of the device buffer."""
        mgr = self.manager
        num_seqs = len(entries)
        q_lens = [len(entries[i].tokens) for i in order]
        cached = [self.lengths[entries[i].req_id] for i in order]
        total = sum(q_lens)
        starts = np.zeros(num_seqs + 1, dtype=np.int32)
        np.cumsum(q_lens, out=starts[1:])

        tokens = np.empty(total, dtype=np.int32)
        positions = np.empty(total, dtype=np.int32)
        token_seq = np.empty(total, dtype=np.int32)
        row_of_entry = {}
        for b, i in enumerate(order):
            e = entries[i]
            s, n = int(starts[b]), q_lens[b]
            tokens[s:s + n] = e.tokens
            positions[s:s + n] = np.arange(cached[b], cached[b] + n, dtype=np.int32)
            token_seq[s:s + n] = b
            row_of_entry[i] = s
        cached_lens = np.asarray(cached, dtype=np.int32)
        context_lens = cached_lens + np.asarray(q_lens, dtype=np.int32)
        state_slots = [mgr.state_slot(entries[i].req_id) for i in order]
        want = [row_of_entry[i] + w for i, e in enumerate(entries) for w in e.want]
        want_rows = np.asarray(want, dtype=np.int32)

        feeds = any(e.feed is not None for e in entries)
        feed = np.full(total if feeds else 0, -1, dtype=np.int32)
        if feeds:
            for i, e in enumerate(entries):
                if e.feed is not None:
                    feed[row_of_entry[i]] = e.feed
        pieces = [tokens, positions, token_seq, starts, context_lens, cached_lens,
                  np.asarray(state_slots, dtype=np.int32), want_rows, feed]
        fixed = len(pieces)
        widths = []
        for gi, g in enumerate(mgr.groups):
            tables = [mgr.block_table(entries[i].req_id, gi) for i in order]
            width = max(1, max(len(t) for t in tables))
            bt = np.zeros((num_seqs, width), dtype=np.int32)
            for b, t in enumerate(tables):
                row = np.asarray(t, dtype=np.int32)
                bt[b, :len(t)] = np.where(row < 0, 0, row)
            slots = np.concatenate([mgr.slot_mapping(entries[i].req_id, gi, cached[b], q_lens[b])
                                    for b, i in enumerate(order)]) if total else np.empty(0, np.int32)
            pieces += [bt.reshape(-1), slots]
            widths.append(width)
        # what the mixers ask for
        view = self.batch_view(q_lens, cached)
        asked = []   # (step key, name, shape, index among the pieces)
        for key, mixer in self.preparers.items():
            for name, array in mixer.prepare_step(view).items():
                array = np.ascontiguousarray(array, dtype=np.int32)
                asked.append((key, name, array.shape, len(pieces)))
                pieces.append(array.reshape(-1))

        offsets, length = pack_int32(pieces)
        dev = self._staging.send(pieces, offsets, length)

        def at(k):
            return dev[offsets[k]:offsets[k] + pieces[k].size]

        (d_tokens, d_positions, d_token_seq, d_starts, d_ctx, d_cached, d_slots, d_want, d_feed) = (
            at(k) for k in range(fixed))
        if feeds:
            self.ops.feed_tokens(d_tokens, d_feed, self.sampled)
        ctx = StepContext(ops=self.ops, dtype=self.dtype, device=self.device, num_tokens=total, num_seqs=num_seqs,
                          positions=d_positions, token_seq=d_token_seq, cu_seqlens_q=d_starts, context_lens=d_ctx,
                          cached_lens=d_cached, slot_of_seq=d_slots, num_prefill=view.num_prefill,
                          max_q_len=max(q_lens), max_context_len=int(context_lens.max()),
                          seq_starts=[int(s) for s in starts[:-1]], seq_lens=q_lens, seq_cached=cached,
                          state_slots=state_slots)
        for gi, g in enumerate(mgr.groups):
            ctx.block_tables[gi] = at(fixed + 2 * gi).view(num_seqs, widths[gi])
            ctx.slot_mappings[gi] = at(fixed + 1 + 2 * gi)
            ctx.page_sizes[gi] = g.page_size
        for key, name, shape, k in asked:
            ctx.prepared.setdefault(key, {})[name] = at(k).view(shape)
        return ctx, d_tokens, (d_want if want_rows.size else None)


class _Staging:
    """Pinned host buffers that a step's integer arrays are gathered in before their one copy to the
    device.  The copy does not block the host; a buffer is written again only after the copy out of it
    has finished (an event per buffer), the reference's pinned twin with its event
    (atom/utils/__init__.py:566-617, atom/model_engine/model_runner.py:1356-1401).  Off the GPU: plain memory."""

    def __init__(self, device: torch.device, buffers: int = 3):
        self.device = device
        self.pinned = device.type == "cuda"
        self.hosts: list[torch.Tensor | None] = [None] * buffers
        self.events = [torch.cuda.Event() if self.pinned else None for _ in range(buffers)]
        self.pending = [False] * buffers
        self.turn = 0

    def send(self, pieces: list[np.ndarray], offsets: list[int], length: int) -> torch.Tensor:
        k = self.turn
        self.turn = (k + 1) % len(self.hosts)
        if self.pending[k]:
            self.events[k].synchronize()
            self.pending[k] = False
        host = self.hosts[k]
        if host is None or host.numel() < length:
            host = torch.zeros(max(length, 4096) * 2, dtype=torch.int32, pin_memory=self.pinned)
            self.hosts[k] = host
        flat = host.numpy()
        for off, p in zip(offsets, pieces):
            flat[off:off + p.size] = p
        if not self.pinned:
            return host[:length].clone().to(self.device)
        dev = torch.empty(length, dtype=torch.int32, device=self.device)
        dev.copy_(host[:length], non_blocking=True)
        self.events[k].record()
        self.pending[k] = True
        return dev


TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16, "fp32": torch.float32}


def load_model(model_dir: str | None, *, dtype: torch.dtype, device, model_config=None, source=None, progress=None):
    """Builds the model that ``config.json`` names through the registry and fills its
    weights from the folder's safetensors (or from ``source``, e.g. random weights)."""
    from ..config.model_config import read_config_json
    from ..config.registry import build_model, model_config_from_dict
    from ..weights.loader import SafetensorsFolder, load_weights

    if model_config is None:
        model_config = model_config_from_dict(read_config_json(model_dir))
    model = build_model(model_config)
    if source is None:
        source = SafetensorsFolder(model_dir)
    load_weights(model, source, device, dtype, progress)
    return model, model_config


def build_core(model, ops, *, dtype: torch.dtype, device, page_size: int = 16, num_pages: int | None = None,
               budget_bytes: int | None = None, max_num_seqs: int = 4, max_model_len: int = 0,
               max_num_batched_tokens: int = 0, graph_sizes: list[int] | None = None,
               prefix_caching: bool = False, graph_prefill_sizes: list[int] | None = None,
               graph_prefill_slots: int | None = None) -> EngineCore:
    from ..cache.storage import plan_cache

    plan = plan_cache(model, page_size, dtype, num_pages=num_pages, budget_bytes=budget_bytes,
                      max_num_seqs=max_num_seqs, max_model_len=max_model_len,
                      max_num_batched_tokens=max_num_batched_tokens)
    return EngineCore(model, ops, plan, max_num_seqs, device, dtype, graph_sizes=graph_sizes,
                      max_model_len=max_model_len, prefix_caching=prefix_caching,
                      graph_prefill_sizes=graph_prefill_sizes, graph_prefill_slots=graph_prefill_slots)
