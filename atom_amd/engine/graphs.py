"""HIP graphs for steps whose shape repeats.

A step in which every request brings one token has the same kernels whatever the
requests are; only the contents of the step's integer arrays differ.  Such a step is
captured once per batch-size bucket (the reference captures decode graphs for a list of
sizes, largest first, atom/model_engine/model_runner.py:3949-4298, sizes from
atom/model_engine/arg_utils.py:59) and replayed: the arrays live in one static device
buffer that is overwritten before each replay.  A batch smaller than its bucket is
padded the reference's way (model_runner.py:2577-2590): padding rows have token 0,
context length 0 (attention sees no key), cache slot -1 (nothing is written) and
request index -1.

The same holds for the steps of continuous batching under a small token budget: up to
``prefill_slots`` prompt portions of at most P tokens together, beside single tokens of up
to N running requests.  Such a step is captured per (P, N) bucket with this layout:

    token rows   [ the portions' tokens, packed | padding up to P | N single tokens ]
    requests     [ prefill_slots portions (unused: no tokens) | one request that owns the
                   padding rows and has no context | N single-token requests ]

so the single tokens always sit at rows P .. P + N - 1 and every kernel's grid depends on
the bucket alone.  What a mixer lists for the portions (attention: tiles of query rows)
has a fixed capacity and is padded with entries that name request -1.  Logits are
formed at one row per portion (its last) and per single token.

Buckets are captured on first use, or all at once with ``capture_all`` (the engine does that
when it is built).  Every graph shares one memory pool.
"""

from __future__ import annotations

import gc

import numpy as np
import torch

from .context import StepContext


PREFILL_SLOTS = 2    # prompt portions a replayed step holds at most, unless the engine's configuration says otherwise


class _Captured:
    def __init__(self, shape: tuple[int, int, int]):
        self.shape = shape                      # (P prompt-token rows, R portion slots, N single-token rows)
        p, r, n = shape
        self.num_tokens = p + n
        self.first_single = r + 1 if p else 0   # request row of the first single-token request
        self.num_seqs = self.first_single + n
        self.num_logits = r + n
        self.graph: torch.cuda.CUDAGraph | None = None
        self.host: torch.Tensor | None = None      # pinned int32
        self.dev: torch.Tensor | None = None       # int32, same layout
        self.logits: torch.Tensor | None = None    # float32 [num_logits, vocab]
        self.offsets: dict = {}
        self.copied = torch.cuda.Event()
        self.copy_pending = False
        # what the pinned buffer holds per request row and group: (the request's serial, pages written), so
        # that a request that keeps its row only has its new pages written
        self.row_state: list[list[tuple | None]] = []


class DecodeGraphs:
    def __init__(self, core, sizes: list[int], max_model_len: int, prefill_sizes: list[int] | None = None,
                 prefill_slots: int = PREFILL_SLOTS):
        self.core = core
        limit = core.manager.slots.num_slots
        self.sizes = sorted({int(s) for s in sizes if 0 < int(s) <= limit})
        self.prefill_sizes = sorted({int(s) for s in (prefill_sizes or []) if int(s) >= 2})
        self.prefill_slots = int(prefill_slots)
        # steps with prompt portions come in fewer sizes of their single-token part: a graph per (P, N) pair
        self.mixed_sizes = [s for s in self.sizes if s >= 8] or self.sizes[-1:]
        self.max_model_len = int(max_model_len)
        self.widths = [max(1, -(-self.max_model_len // g.page_size)) for g in core.manager.groups]
        self.captured: dict[tuple, _Captured] = {}
        self.pool = None
        self.replays = 0
        self.mixed_replays = 0
        self.usable = bool(self.sizes) and core.device.type == "cuda" and all(
            getattr(block.mixer, "graph_safe", False) for block in core.model.blocks)

    def bucket(self, num_seqs: int) -> int | None:
        for s in self.sizes:
            if s >= num_seqs:
                return s
        return None

    def shape_for(self, entries) -> tuple[int, int, int] | None:
        """The bucket that holds these entries, or None."""
        portions = [e for e in entries if len(e.tokens) > 1]
        singles = len(entries) - len(portions)
        if not portions:
            n = self.bucket(max(1, singles))
            return None if n is None else (0, 0, n)
        n = next((s for s in self.mixed_sizes if s >= singles), None)
        if n is None:
            return None
        total = sum(len(e.tokens) for e in portions)
        if not self.prefill_sizes or len(portions) > self.prefill_slots or total > self.prefill_sizes[-1]:
            return None
        # a graph forms logits at a portion's last row only
        if any(e.want not in ([], [len(e.tokens) - 1]) or e.feed is not None for e in portions):
            return None
        return (next(p for p in self.prefill_sizes if p >= total), self.prefill_slots, n)

    def accepts(self, entries, cached: list[int]) -> bool:
        if not self.usable or not entries:
            return False
        if self.shape_for(entries) is None:
            return False
        return max(c + len(e.tokens) for c, e in zip(cached, entries)) <= self.max_model_len

    # ------------------------------------------------------------------ layout

    def _view_of(self, cap: _Captured, q_lens: list[int], cached: list[int]):
        p, r, _ = cap.shape
        return self.core.batch_view(q_lens, cached, replayed=True, prefill_capacity=p, prefill_slots=r,
                                    num_prefill=cap.first_single)

    def _layout(self, cap: _Captured) -> int:
        t, s = cap.num_tokens, cap.num_seqs
        pieces = [("tokens", t), ("feed", t), ("positions", t), ("token_seq", t), ("starts", s + 1),
                  ("context_lens", s), ("cached_lens", s), ("slot_of_seq", s), ("want", cap.num_logits)]
        for gi, width in enumerate(self.widths):
            pieces += [(f"bt{gi}", s * width), (f"slots{gi}", t)]
        # what the mixers ask for: in a replayed step the shapes depend on the bucket only
        view = self._view_of(cap, self._padded_q_lens(cap, []), [0] * s)
        for key, mixer in self.core.preparers.items():
            for name, array in mixer.prepare_step(view).items():
                pieces.append((("prepared", key, name, tuple(np.shape(array))), int(np.size(array))))
        cursor = 0
        for name, n in pieces:
            cap.offsets[name] = (cursor, n)
            cursor += (n + 3) // 4 * 4
        return cursor

    @staticmethod
    def _padded_q_lens(cap: _Captured, portion_lens: list[int]) -> list[int]:
        """Tokens of every request row of the bucket: the portions, then the request that owns the padding rows,
        then the single tokens."""
        p, r, n = cap.shape
        if not p:
            return [1] * n
        lens = list(portion_lens) + [0] * (r - len(portion_lens))
        return lens + [p - sum(lens)] + [1] * n

    def _fill(self, cap: _Captured, entries, cached: list[int]) -> list[int]:
        """Writes the step's arrays into the pinned buffer (padding beyond the entries); returns, for every
        entry, the row of the graph's logits that is its own."""
        if cap.copy_pending:
            cap.copied.synchronize()   # the last copy out of this buffer has finished
            cap.copy_pending = False
        host = cap.host.numpy()
        p, r, n = cap.shape
        mgr = self.core.manager

        def view(name):
            off, count = cap.offsets[name]
            return host[off:off + count]

        tokens, positions, token_seq, feed = view("tokens"), view("positions"), view("token_seq"), view("feed")
        tokens[:] = 0
        feed[:] = -1
        positions[:] = 0
        token_seq[:] = -1
        ctx_lens, cached_lens, slot_of_seq = view("context_lens"), view("cached_lens"), view("slot_of_seq")
        ctx_lens[:] = 0
        cached_lens[:] = 0
        slot_of_seq[:] = -1
        starts, want = view("starts"), view("want")
        want[:] = 0
        if not cap.row_state:
            cap.row_state = [[None] * cap.num_seqs for _ in self.widths]
        slot_arrays = [view(f"slots{gi}") for gi in range(len(self.widths))]
        for slots in slot_arrays:
            slots[:] = -1
        tables = [view(f"bt{gi}").reshape(cap.num_seqs, width) for gi, width in enumerate(self.widths)]

        # which request row and token rows every entry gets
        logits_row, placed = [], []          # placed: (entry, its cached tokens, request row, first token row)
        at, portions, singles = 0, 0, 0
        for e, c in zip(entries, cached):
            if len(e.tokens) > 1:
                placed.append((e, c, portions, at))
                logits_row.append(portions)
                at += len(e.tokens)
                portions += 1
            else:
                placed.append((e, c, cap.first_single + singles, p + singles))
                logits_row.append(r + singles)
                singles += 1
        q_lens = self._padded_q_lens(cap, [len(e.tokens) for e in entries if len(e.tokens) > 1])
        starts[0] = 0
        np.cumsum(q_lens, out=starts[1:])
        full_cached = [0] * cap.num_seqs
        for i, (e, c, row, first) in enumerate(placed):
            k = len(e.tokens)
            tokens[first:first + k] = e.tokens
            if e.feed is not None:
                feed[first] = e.feed
            positions[first:first + k] = np.arange(c, c + k, dtype=np.int32)
            token_seq[first:first + k] = row
            ctx_lens[row] = c + k
            cached_lens[row] = c
            full_cached[row] = c
            slot_of_seq[row] = mgr.state_slot(e.req_id)
            want[logits_row[i]] = first + k - 1
            for gi, width in enumerate(self.widths):
                table = mgr.block_table(e.req_id, gi)
                page_size = mgr.groups[gi].page_size
                slot_arrays[gi][first:first + k] = mgr.slot_mapping(e.req_id, gi, c, k)
                bt, state = tables[gi], cap.row_state[gi]
                held, serial = state[row], mgr.serial(e.req_id)
                windowed = mgr.groups[gi].window is not None
                if table[(c + k - 1) // page_size] < 0:
                    raise AssertionError(f"request {e.req_id!r}: position {c + k - 1} has no page")
                if not windowed and held is not None and held[0] == serial and held[1] <= len(table):
                    if held[1] < len(table):     # pages appended since the row was last written
                        bt[row, held[1]:len(table)] = table[held[1]:]
                else:
                    line = np.asarray(table, dtype=np.int32)
                    bt[row, :len(table)] = np.where(line < 0, 0, line)
                    bt[row, len(table):] = 0
                state[row] = (serial, len(table))
            # request rows without an entry keep what they had: their context length is 0, nothing reads them
        if self.core.preparers:
            batch = self._view_of(cap, q_lens, full_cached)
            for key, mixer in self.core.preparers.items():
                for name, array in mixer.prepare_step(batch).items():
                    array = np.ascontiguousarray(array, dtype=np.int32)
                    piece = ("prepared", key, name, tuple(array.shape))
                    if piece not in cap.offsets:
                        raise AssertionError(f"{type(mixer).__name__}.prepare_step: '{name}' has shape {array.shape} "
                                             f"in this step, not the shape the graph {cap.shape} was captured with")
                    view(piece)[:] = array.reshape(-1)
        return logits_row

    def _context(self, cap: _Captured):
        core = self.core
        p, r, n = cap.shape

        def view(name):
            off, count = cap.offsets[name]
            return cap.dev[off:off + count]

        # every mixer reads the batch from the device; there are no host-side lists in a replayed step
        ctx = StepContext(ops=core.ops, dtype=core.dtype, device=core.device, num_tokens=cap.num_tokens,
                          num_seqs=cap.num_seqs, positions=view("positions"), token_seq=view("token_seq"),
                          cu_seqlens_q=view("starts"), context_lens=view("context_lens"),
                          cached_lens=view("cached_lens"), slot_of_seq=view("slot_of_seq"),
                          num_prefill=cap.first_single, max_q_len=max(p, 1),
                          # a bound, not the batch's own: no request of a replayed step is longer (accepts())
                          max_context_len=self.max_model_len, replayed=True)
        for gi, (g, width) in enumerate(zip(core.manager.groups, self.widths)):
            ctx.block_tables[gi] = view(f"bt{gi}").view(cap.num_seqs, width)
            ctx.slot_mappings[gi] = view(f"slots{gi}")
            ctx.page_sizes[gi] = g.page_size
        for piece in cap.offsets:
            if isinstance(piece, tuple) and piece[0] == "prepared":
                _, key, name, shape = piece
                ctx.prepared.setdefault(key, {})[name] = view(piece).view(shape)
        return ctx, view("tokens"), view("want"), view("feed")

    # ------------------------------------------------------------------ capture and replay

    def _capture(self, shape: tuple[int, int, int]) -> _Captured:
        core = self.core
        cap = _Captured(shape)
        total = self._layout(cap)
        cap.host = torch.zeros(max(total, 4), dtype=torch.int32, pin_memory=True)
        cap.dev = torch.zeros(max(total, 4), dtype=torch.int32, device=core.device)
        self._fill(cap, [], [])                       # all padding: the warm-up touches no cache slot
        cap.dev.copy_(cap.host)
        ctx, tokens, want, feed = self._context(cap)
        stream = torch.cuda.Stream(device=core.device)
        stream.wait_stream(torch.cuda.current_stream(core.device))
        with torch.cuda.stream(stream):
            core.ops.feed_tokens(tokens, feed, core.sampled)
            core.model.forward(ctx, tokens, core.storage.bindings, want)   # first-use allocations happen here
        stream.synchronize()
        if self.pool is None:
            self.pool = torch.cuda.graph_pool_handle()
        cap.graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: a collected tensor, event or older graph
        # frees device objects, which is not allowed during capture and aborts the process (the reference
        # pauses it for the same reason, atom/model_engine/model_runner.py:4046-4055).
        gc.collect()
        gc_was_enabled = gc.isenabled()
        gc.disable()
        try:
            ctx, tokens, want, feed = self._context(cap)    # a fresh context: nothing remembered from the warm-up
            with torch.cuda.graph(cap.graph, pool=self.pool, stream=stream):
                # rows whose token the last step's sampler left on the device take it from there
                core.ops.feed_tokens(tokens, feed, core.sampled)
                cap.logits = core.model.forward(ctx, tokens, core.storage.bindings, want)
        finally:
            if gc_was_enabled:
                gc.enable()
        self.captured[shape] = cap
        return cap

    def capture_all(self) -> int:
        """Captures every decode bucket now, largest first (atom/model_engine/model_runner.py:3973), so that no
        decode step of a running engine pays for a capture.  Returns how many graphs there are."""
        if self.usable:
            for size in sorted(self.sizes, reverse=True):
                if (0, 0, size) not in self.captured:
                    self._capture((0, 0, size))
            for p in sorted(self.prefill_sizes, reverse=True):
                for size in sorted(self.mixed_sizes, reverse=True):
                    if (p, self.prefill_slots, size) not in self.captured:
                        self._capture((p, self.prefill_slots, size))
        return len(self.captured)

    def run(self, entries, cached: list[int]) -> torch.Tensor | None:
        """Float32 logits at the entries' wanted places (a portion's last row, a single token), in the
        order of the entries; None if nothing is wanted.  The tensor is the graph's own output or a
        selection of it, valid until the graph's next replay."""
        shape = self.shape_for(entries)
        cap = self.captured.get(shape) or self._capture(shape)
        logits_row = self._fill(cap, entries, cached)
        cap.dev.copy_(cap.host, non_blocking=True)
        cap.copied.record()
        cap.copy_pending = True
        cap.graph.replay()
        self.replays += 1
        if shape[0]:
            self.mixed_replays += 1
        picked = [row for row, e in zip(logits_row, entries) if e.want]
        if not picked:
            return None
        if picked == list(range(len(picked))):
            return cap.logits[:len(picked)]
        index = torch.tensor(picked, dtype=torch.long, device=self.core.device)
        return cap.logits.index_select(0, index)
