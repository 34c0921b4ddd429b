"""HIP graphs for decode-only steps.

A step in which every request brings one token has the same kernels whatever the
requests are; only the contents of the step's integer arrays differ.  Such a step is
captured once per batch-size bucket (the reference captures decode graphs for a list of
sizes, largest first, atom/model_engine/model_runner.py:3949-4298, sizes from
atom/model_engine/arg_utils.py:59) and replayed: the arrays live in one static device
buffer that is overwritten before each replay.  A batch smaller than its bucket is
padded the reference's way (model_runner.py:2577-2590): padding rows have token 0,
context length 0 (attention sees no key), cache slot -1 (nothing is written) and
request index -1.

Buckets are captured on first use, or all at once with ``capture_all`` (the engine does that when it
is built).  Every captured graph shares one memory pool.
"""

from __future__ import annotations

import gc

import numpy as np
import torch

from .context import StepContext


class _Captured:
    def __init__(self, size: int):
        self.size = size
        self.graph: torch.cuda.CUDAGraph | None = None
        self.host: torch.Tensor | None = None      # pinned int32
        self.dev: torch.Tensor | None = None       # int32, same layout
        self.logits: torch.Tensor | None = None    # float32 [size, vocab]
        self.offsets: dict[str, tuple[int, int]] = {}
        self.copied = torch.cuda.Event()
        self.copy_pending = False
        # what the pinned buffer holds per row and group: (the request's serial, pages written), so that a
        # request that keeps its row only has its new pages written
        self.row_state: list[list[tuple | None]] = []


class DecodeGraphs:
    def __init__(self, core, sizes: list[int], max_model_len: int):
        self.core = core
        limit = core.manager.slots.num_slots
        self.sizes = sorted({int(s) for s in sizes if 0 < int(s) <= limit})
        self.max_model_len = int(max_model_len)
        self.widths = [max(1, -(-self.max_model_len // g.page_size)) for g in core.manager.groups]
        self.captured: dict[int, _Captured] = {}
        self.pool = None
        self.replays = 0
        self.usable = bool(self.sizes) and core.device.type == "cuda" and all(
            getattr(block.mixer, "graph_safe", False) for block in core.model.blocks)

    def bucket(self, num_seqs: int) -> int | None:
        for s in self.sizes:
            if s >= num_seqs:
                return s
        return None

    def accepts(self, entries, cached: list[int]) -> bool:
        if not self.usable or not entries or any(len(e.tokens) != 1 for e in entries):
            return False
        if self.bucket(len(entries)) is None:
            return False
        return max(cached) + 1 <= self.max_model_len

    # ------------------------------------------------------------------ layout

    def _layout(self, size: int) -> tuple[dict[str, tuple[int, int]], int]:
        pieces = [("tokens", size), ("feed", size), ("positions", size), ("token_seq", size), ("starts", size + 1),
                  ("context_lens", size), ("cached_lens", size), ("slot_of_seq", size), ("want", size)]
        for gi, width in enumerate(self.widths):
            pieces += [(f"bt{gi}", size * width), (f"slots{gi}", size)]
        # what the mixers ask for: in a replayed step the shapes depend on the bucket only
        view = self.core.batch_view([1] * size, [0] * size, replayed=True)
        for key, mixer in self.core.preparers.items():
            for name, array in mixer.prepare_step(view).items():
                pieces.append((("prepared", key, name, tuple(np.shape(array))), int(np.size(array))))
        offsets, cursor = {}, 0
        for name, n in pieces:
            offsets[name] = (cursor, n)
            cursor += (n + 3) // 4 * 4
        return offsets, cursor

    def _fill(self, cap: _Captured, entries, cached: list[int]) -> None:
        """Writes the step's arrays into the pinned buffer (padding beyond the entries)."""
        if cap.copy_pending:
            cap.copied.synchronize()   # the last copy out of this buffer has finished
            cap.copy_pending = False
        host = cap.host.numpy()
        size, n = cap.size, len(entries)
        mgr = self.core.manager

        def view(name):
            off, count = cap.offsets[name]
            return host[off:off + count]

        tokens, positions, token_seq = view("tokens"), view("positions"), view("token_seq")
        tokens[:] = 0
        feed = view("feed")
        feed[:] = -1
        positions[:] = 0
        token_seq[:] = -1
        ctx_lens = view("context_lens")
        ctx_lens[:] = 0
        cached_lens, slot_of_seq = view("cached_lens"), view("slot_of_seq")
        cached_lens[:] = 0
        slot_of_seq[:] = -1
        view("starts")[:] = np.arange(size + 1, dtype=np.int32)
        view("want")[:] = np.arange(size, dtype=np.int32)
        for b, e in enumerate(entries):
            tokens[b] = e.tokens[0]
            if e.feed is not None:
                feed[b] = e.feed
            positions[b] = cached[b]
            token_seq[b] = b
            ctx_lens[b] = cached[b] + 1
            cached_lens[b] = cached[b]
            slot_of_seq[b] = mgr.state_slot(e.req_id)
        if not cap.row_state:
            cap.row_state = [[None] * size for _ in self.widths]
        for gi, width in enumerate(self.widths):
            bt = view(f"bt{gi}").reshape(size, width)
            slots = view(f"slots{gi}")
            slots[:] = -1
            page_size = mgr.groups[gi].page_size
            windowed = mgr.groups[gi].window is not None
            state = cap.row_state[gi]
            for b, e in enumerate(entries):
                table = mgr.block_table(e.req_id, gi)
                page = table[cached[b] // page_size]
                if page < 0:
                    raise AssertionError(f"request {e.req_id!r}: position {cached[b]} has no page")
                slots[b] = page * page_size + cached[b] % page_size
                held = state[b]
                serial = mgr.serial(e.req_id)
                if not windowed and held is not None and held[0] == serial and held[1] <= len(table):
                    if held[1] < len(table):     # pages appended since the row was last written
                        bt[b, held[1]:len(table)] = table[held[1]:]
                else:
                    row = np.asarray(table, dtype=np.int32)
                    bt[b, :len(table)] = np.where(row < 0, 0, row)
                    bt[b, len(table):] = 0
                state[b] = (serial, len(table))
            # rows beyond the entries keep what they had: their context length is 0, nothing reads them
        if self.core.preparers:
            batch = self.core.batch_view([1] * size, list(cached) + [0] * (size - n), replayed=True)
            for key, mixer in self.core.preparers.items():
                for name, array in mixer.prepare_step(batch).items():
                    array = np.ascontiguousarray(array, dtype=np.int32)
                    piece = ("prepared", key, name, tuple(array.shape))
                    if piece not in cap.offsets:
                        raise AssertionError(f"{type(mixer).__name__}.prepare_step: '{name}' has shape {array.shape} "
                                             f"in this step, not the shape the graph of {size} rows was captured with")
                    view(piece)[:] = array.reshape(-1)

    def _context(self, cap: _Captured):
        core, size = self.core, cap.size

        def view(name):
            off, count = cap.offsets[name]
            return cap.dev[off:off + count]

        # every mixer reads the batch from the device; there are no host-side lists in a replayed step
        ctx = StepContext(ops=core.ops, dtype=core.dtype, device=core.device, num_tokens=size, num_seqs=size,
                          positions=view("positions"), token_seq=view("token_seq"), cu_seqlens_q=view("starts"),
                          context_lens=view("context_lens"), cached_lens=view("cached_lens"),
                          slot_of_seq=view("slot_of_seq"), num_prefill=0, max_q_len=1,
                          max_context_len=max(w * g.page_size for w, g in zip(self.widths, core.manager.groups))
                          if self.widths else self.max_model_len, replayed=True)
        for gi, (g, width) in enumerate(zip(core.manager.groups, self.widths)):
            ctx.block_tables[gi] = view(f"bt{gi}").view(size, width)
            ctx.slot_mappings[gi] = view(f"slots{gi}")
            ctx.page_sizes[gi] = g.page_size
        for piece in cap.offsets:
            if isinstance(piece, tuple) and piece[0] == "prepared":
                _, key, name, shape = piece
                ctx.prepared.setdefault(key, {})[name] = view(piece).view(shape)
        return ctx, view("tokens"), view("want"), view("feed")

    # ------------------------------------------------------------------ capture and replay

    def _capture(self, size: int) -> _Captured:
        core = self.core
        cap = _Captured(size)
        cap.offsets, total = self._layout(size)
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
            with torch.cuda.graph(cap.graph, pool=self.pool, stream=stream):
                # rows whose token the last step's sampler left on the device take it from there
                core.ops.feed_tokens(tokens, feed, core.sampled)
                cap.logits = core.model.forward(ctx, tokens, core.storage.bindings, want)
        finally:
            if gc_was_enabled:
                gc.enable()
        self.captured[size] = cap
        return cap

    def capture_all(self) -> int:
        """Captures every bucket now, largest first (atom/model_engine/model_runner.py:3973), so that no
        step of a running engine pays for a capture.  Returns how many graphs there are."""
        if self.usable:
            for size in sorted(self.sizes, reverse=True):
                if size not in self.captured:
                    self._capture(size)
        return len(self.captured)

    def run(self, entries, cached: list[int]) -> torch.Tensor:
        """Float32 logits [len(entries), vocab] of the entries' single tokens."""
        size = self.bucket(len(entries))
        cap = self.captured.get(size) or self._capture(size)
        self._fill(cap, entries, cached)
        cap.dev.copy_(cap.host, non_blocking=True)
        cap.copied.record()
        cap.copy_pending = True
        cap.graph.replay()
        self.replays += 1
        return cap.logits[:len(entries)]
