"""Continuous batching above the step function.

Rules kept from the reference's scheduler (atom/model_engine/scheduler.py): FIFO
admission with head-of-line blocking (:1187-1347), ``max_num_seqs`` and a per-step token
budget ``max_num_batched_tokens`` (:1180-1186), prompts cut into portions under the
budget with a truncated portion floored to a multiple of ``max(block_size, 64)`` and a
sliver not scheduled unless the batch is empty (:1733-1753), permanent rejection of
requests that can never run (:989-1050), preemption of the last running request when
pages run out, the preempted request going back to the head of the waiting queue and
later prefilling prompt plus generated tokens (:1917-1952, :1277-1283), the finishing
rules in their order (:2296-2329), and with the prefix cache on a new request starting after the
pages that already hold its beginning (``num_new = num_tokens - hits * block``, :1187-1347).

What differs: the reference schedules prompt portions *or* decode tokens per step
(:1370-1429); here one step holds both.  Running requests that decode are scheduled
first (one token each), then unfinished prompts, then new admissions, all under the one
token budget.  Pages are taken when a request is scheduled: a group that keeps every key
reserves the whole prompt at admission (as ``BlockManager.allocate`` does, block_manager.py
:447-470), a window group only what the step needs.
"""

from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

from .core import StepEntry
from .sequence import Sequence, SequenceStatus


@dataclass
class ScheduledItem:
    seq: Sequence
    num_tokens: int          # tokens of this step
    start: int               # = seq.num_cached_tokens when scheduled
    is_decode: bool
    is_final: bool           # after this step the sequence has all its tokens in the cache


@dataclass
class ScheduledBatch:
    items: list[ScheduledItem] = field(default_factory=list)

    @property
    def total_tokens(self) -> int:
        return sum(i.num_tokens for i in self.items)

    @property
    def num_decode(self) -> int:
        return sum(1 for i in self.items if i.is_decode)

    @property
    def num_prefill(self) -> int:
        return sum(1 for i in self.items if not i.is_decode)

    def entries(self, sampled_rows: dict[int, int] | None = None) -> list[StepEntry]:
        """``sampled_rows``: for a batch scheduled ahead, sequence id -> the row in which the step before
        this one samples that sequence's token; its entry names that row instead of the token."""
        out = []
        for it in self.items:
            tokens = it.seq.token_ids[it.start:it.start + it.num_tokens]
            want = [it.num_tokens - 1] if it.is_final else []
            reserve = it.seq.num_tokens if not it.is_decode else None
            feed = None
            if it.seq.awaits_token and it.start + it.num_tokens == it.seq.num_tokens:
                feed = sampled_rows[it.seq.id]
            out.append(StepEntry(it.seq.id, tokens, want, reserve, feed))
        return out


class Scheduler:
    def __init__(self, config, core, clock=time.time):
        """``core`` is the ``EngineCore`` whose cache manager this scheduler takes pages from; ``clock``
        tells the time (tests pass their own)."""
        self.core = core
        self.clock = clock
        self.manager = core.manager
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.max_model_len = config.max_model_len
        self.block_size = config.kv_cache_block_size
        self.enable_chunked_prefill = config.enable_chunked_prefill
        self.long_prefill_token_threshold = config.long_prefill_token_threshold
        self.delay_factor = config.scheduler_delay_factor
        self.eos_token_id = config.eos_token_id
        self.stop_token_ids = set(config.stop_token_ids or [])
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()
        self._rejected: list[Sequence] = []
        self.total_preemptions = 0
        self._last_prompt_time = 0.0
        self._last_prompt_latency = 0.0
        # requests that reach their token count in the step that is still running: a step scheduled ahead leaves them out
        self._sit_out: set[int] = set()

    # ------------------------------------------------------------------ queues

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def extend(self, seqs) -> None:
        for s in seqs:
            self.add(s)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running and not self._rejected

    def take_rejected(self) -> list[Sequence]:
        out, self._rejected = self._rejected, []
        return out

    # ------------------------------------------------------------------ helpers

    def _unschedulable_reason(self, seq: Sequence) -> str | None:
        """Why a request can never run, or None (atom/model_engine/scheduler.py:989-1050)."""
        n = seq.num_tokens
        if n > self.max_model_len:
            return f"{n} tokens exceed max_model_len {self.max_model_len}"
        if not self.enable_chunked_prefill and n > self.max_num_batched_tokens:
            return f"{n} tokens exceed max_num_batched_tokens {self.max_num_batched_tokens} with chunked prefill off"
        for gi, g in enumerate(self.manager.groups):
            if g.window is None:
                need = -(-n // g.page_size)
                if need > g.num_pages:
                    return f"needs {need} cache pages, the pool has {g.num_pages}"
        return None

    def _chunked_prefill_size(self, num_new: int, budget_left: int, batched: int) -> int:
        """How many of a prompt's ``num_new`` outstanding tokens run in this step; 0 means wait.  The rule is
        the reference's (atom/model_engine/scheduler.py:1733-1753): everything if the budget allows; else
        the budget rounded down to whole units of ``max(block_size, 64)`` tokens; a remainder smaller than
        one unit runs only when the step would otherwise be empty."""
        if num_new <= budget_left:
            return num_new
        unit = max(self.block_size, 64)
        whole_units = (budget_left // unit) * unit
        if whole_units:
            return whole_units
        return budget_left if batched == 0 else 0

    def _prefill_chunk_for_budget(self, num_new: int, budget_left: int, batched: int) -> int | None:
        """The same for a new request, or None when it has to wait.  Without chunked prefill a prompt runs
        whole or not at all; it may exceed the budget only in a step of its own
        (atom/model_engine/scheduler.py:1755-1767)."""
        if not self.enable_chunked_prefill:
            fits = num_new <= budget_left or batched == 0
            return num_new if fits else None
        size = self._chunked_prefill_size(num_new, budget_left, batched)
        return size if size > 0 else None

    def _passed_delay(self, now: float) -> bool:
        """atom/model_engine/scheduler.py:2761-2777: hold new prompts until the oldest waiting
        request has waited ``delay_factor`` times the last prompt step's latency."""
        if self.delay_factor <= 0 or not self.waiting or not self.running:
            return True
        earliest = min(s.arrive_time for s in self.waiting)
        return (now - earliest) > self.delay_factor * self._last_prompt_latency

    def preempt(self, seq: Sequence) -> None:
        """atom/model_engine/scheduler.py:1928-1952: back to the head of the waiting queue, pages
        and slot given back; on re-admission prompt plus generated tokens are prefilled."""
        self.total_preemptions += 1
        seq.num_preemptions += 1
        seq.status = SequenceStatus.WAITING
        seq.is_partial_prefill = False
        seq.num_cached_tokens = 0
        self.core.close(seq.id)
        self.waiting.appendleft(seq)

    def _preempt_one_running(self, protect: set[int]) -> bool:
        """Preempts the last running request that is not scheduled in this step."""
        for index in range(len(self.running) - 1, -1, -1):
            cand = self.running[index]
            if cand.id in protect:
                continue
            del self.running[index]
            self.preempt(cand)
            return True
        return False

    # ------------------------------------------------------------------ schedule

    def abort(self, seq_id: int) -> bool:
        """Marks a waiting or running request as aborted (atom/model_engine/engine_utility.py:219-229): it
        leaves at the next ``schedule`` with the reason "aborted", its pages and slot given back, whether it
        had started or not (atom/model_engine/scheduler.py:1195-1197, 2284-2285).  What a step that is
        still running computes for it is dropped.  Returns whether the request was found."""
        for seq in list(self.running) + list(self.waiting):
            if seq.id == seq_id and seq.status in (SequenceStatus.WAITING, SequenceStatus.RUNNING):
                seq.status = SequenceStatus.ABORTED
                return True
        return False

    def _leave_aborted(self, seq: Sequence) -> None:
        seq.leave_reason = "aborted"
        seq.leave_time = self.clock()
        seq.awaits_token = False
        self.core.close(seq.id)
        self._rejected.append(seq)

    def _sweep_aborted(self) -> None:
        for seq in [s for s in self.running if s.status == SequenceStatus.ABORTED]:
            self.running.remove(seq)
            if seq.awaits_token:          # the placeholder of a step whose result is dropped
                seq.token_ids.pop()
            self._leave_aborted(seq)

    def get_next_batch_info(self) -> tuple[bool, int, int]:
        """What the next step will mostly be, without scheduling it: (it holds prompt tokens, its tokens,
        its requests).  The reference's estimate (atom/model_engine/scheduler.py:2724-2759), for steps that
        hold decode tokens and prompt portions together: running requests decode one token each, the rest
        of the budget goes to unfinished and then to waiting prompts."""
        decoding = [s for s in self.running if s.status == SequenceStatus.RUNNING and not s.is_partial_prefill]
        tokens = reqs = min(len(decoding), self.max_num_seqs, self.max_num_batched_tokens)
        prompt_tokens = 0
        pending = [s for s in self.running if s.status == SequenceStatus.RUNNING and s.is_partial_prefill]
        pending += [s for s in self.waiting if s.status == SequenceStatus.WAITING]
        for seq in pending:
            left = self.max_num_batched_tokens - tokens
            if reqs >= self.max_num_seqs or left <= 0:
                break
            want = seq.num_tokens - seq.num_cached_tokens
            if 0 < self.long_prefill_token_threshold < want:
                want = self.long_prefill_token_threshold
            take = self._prefill_chunk_for_budget(want, left, tokens)
            if not take:
                break
            tokens += take
            prompt_tokens += take
            reqs += 1
        return prompt_tokens > 0, tokens, reqs

    def schedule(self) -> ScheduledBatch | None:
        self._sweep_aborted()
        if not self.running and not self.waiting:
            return None
        batch = ScheduledBatch()
        scheduled: set[int] = set()
        batched = 0
        mgr = self.manager

        # ---- running requests that decode: one token each
        for seq in list(self.running):
            # a request preempted earlier in this loop is WAITING by now
            if (seq.status != SequenceStatus.RUNNING or seq.is_partial_prefill or seq.id in scheduled
                    or seq.id in self._sit_out):
                continue
            if len(batch.items) >= self.max_num_seqs or batched + 1 > self.max_num_batched_tokens:
                break
            cached = seq.num_cached_tokens
            preempted_self = False
            while not mgr.can_cover(seq.id, cached, cached + 1):
                if self._preempt_one_running(scheduled | {seq.id}):
                    continue
                self.running.remove(seq)
                self.preempt(seq)
                preempted_self = True
                break
            if preempted_self:
                continue
            mgr.cover(seq.id, cached, cached + 1)
            batch.items.append(ScheduledItem(seq, 1, cached, True, True))
            scheduled.add(seq.id)
            batched += 1

        # ---- unfinished prompts among the running requests
        for seq in list(self.running):
            if not seq.is_partial_prefill or seq.id in scheduled or seq.status != SequenceStatus.RUNNING:
                continue
            if len(batch.items) >= self.max_num_seqs:
                break
            remaining = seq.num_tokens - seq.num_cached_tokens
            if 0 < self.long_prefill_token_threshold < remaining:
                remaining = self.long_prefill_token_threshold
            chunk = self._chunked_prefill_size(remaining, self.max_num_batched_tokens - batched, batched)
            if chunk <= 0:
                break
            cached = seq.num_cached_tokens
            if not mgr.can_cover(seq.id, cached, cached + chunk, seq.num_tokens):
                # only a window group can be short here; wait for pages rather than evict
                break
            mgr.cover(seq.id, cached, cached + chunk, seq.num_tokens)
            batch.items.append(ScheduledItem(seq, chunk, cached, False, cached + chunk >= seq.num_tokens))
            scheduled.add(seq.id)
            batched += chunk

        # ---- new requests, in arrival order
        now = self.clock()
        while (self.waiting and len(batch.items) < self.max_num_seqs and batched < self.max_num_batched_tokens
               and self._passed_delay(now)):
            seq = self.waiting.popleft()
            if seq.status == SequenceStatus.ABORTED:
                self._leave_aborted(seq)
                continue
            reason = self._unschedulable_reason(seq)
            if reason is not None:
                seq.status = SequenceStatus.FINISHED
                seq.leave_reason = f"unschedulable: {reason}"
                seq.leave_time = self.clock()
                self._rejected.append(seq)
                continue
            if len(self.running) >= self.max_num_seqs or not mgr.can_open():
                self.waiting.appendleft(seq)
                break
            # the request is opened first: pages that already hold the beginning of its tokens (prefix
            # cache) are taken before the rest is counted
            self.core.open(seq.id)
            hit = self.core.match_prefix(seq.id, seq.token_ids)
            num_new = seq.num_tokens - hit
            if self.enable_chunked_prefill and 0 < self.long_prefill_token_threshold < num_new:
                num_new = self.long_prefill_token_threshold
            chunk = self._prefill_chunk_for_budget(num_new, self.max_num_batched_tokens - batched, batched)
            if chunk is None or not mgr.can_cover(seq.id, hit, hit + chunk, seq.num_tokens):
                self.core.close(seq.id)
                self.waiting.appendleft(seq)
                break
            mgr.cover(seq.id, hit, hit + chunk, seq.num_tokens)
            seq.status = SequenceStatus.RUNNING
            seq.num_cached_tokens = hit
            seq.num_prefix_hit_tokens = hit
            self.running.append(seq)
            batch.items.append(ScheduledItem(seq, chunk, hit, False, hit + chunk >= seq.num_tokens))
            scheduled.add(seq.id)
            batched += chunk

        if not batch.items:
            return None
        if batch.num_prefill:
            self._last_prompt_time = now
        return batch

    # ------------------------------------------------------------------ the step after a running one

    def schedule_ahead(self, running_batch: ScheduledBatch) -> ScheduledBatch | None:
        """The batch that follows ``running_batch``, made before that batch's tokens are known, so that
        the device never waits for the host between two steps (the reference's deferred output,
        atom/model_engine/model_runner.py:358-392, scheduler.py:2127-2133).

        What ``running_batch`` does to its requests apart from the tokens' values is applied at once: their
        cached lengths move on, and every request that gets a token from it ends in a placeholder until the
        token arrives.  Then the ordinary ``schedule`` makes the next batch: decode tokens (read on the device
        from the sampler's output), further prompt portions, admissions.  This is done only when nothing in it
        can depend on the tokens' values: no request reaches its token count in ``running_batch`` while others
        wait for its place (with nobody waiting such a request simply takes no further part), and the pools hold
        the pages of one more token for every decoding request, so that nobody has to be preempted.  A request
        that turns out to have ended on its token (eos, a stop sequence) has then run once too often, and that
        result is dropped.  In every other case this returns None and changes nothing: the caller waits for
        the running batch and schedules as usual.

        One more way to None: all the checks pass, the running batch's effects are applied (cached lengths,
        placeholders) and the ordinary ``schedule`` then finds nothing to run, because every request that is left
        reaches its token count in ``running_batch`` and nobody waits.  The requests then already end in
        placeholders; ``postprocess(running_batch, tokens)`` overwrites them as it does after a step launched
        ahead, so the caller still only has to wait for the running batch and go on."""
        items = running_batch.items
        if self._rejected or not items:
            return None
        if any(it.seq.status != SequenceStatus.RUNNING or it.seq.awaits_token for it in items):
            return None
        if any(s.status != SequenceStatus.RUNNING or s.awaits_token for s in self.running):
            return None
        mgr = self.manager
        need = [0] * len(mgr.groups)
        done_by_count = set()
        for it in items:
            if not it.is_final:
                continue
            seq = it.seq
            # with the token that the running batch gives it
            if seq.num_completion_tokens + 1 >= seq.max_tokens or seq.num_tokens + 1 >= self.max_model_len:
                if self.waiting:
                    return None   # its place goes to a waiting request in the very next step
                done_by_count.add(seq.id)
                continue
            after = it.start + it.num_tokens
            for gi, n in enumerate(mgr.pages_missing(seq.id, after, after + 1)):
                need[gi] += n
        in_batch = {it.seq.id for it in items}
        for seq in self.running:   # decoding requests that sat this batch out
            if seq.id not in in_batch and not seq.is_partial_prefill:
                for gi, n in enumerate(mgr.pages_missing(seq.id, seq.num_cached_tokens, seq.num_cached_tokens + 1)):
                    need[gi] += n
        if any(n > mgr.num_free_pages(gi) for gi, n in enumerate(need)):
            return None
        for it in items:
            it.seq.num_cached_tokens = it.start + it.num_tokens
            it.seq.is_partial_prefill = not it.is_final
            if it.is_final:
                it.seq.append_placeholder()
        self._sit_out = done_by_count
        try:
            return self.schedule()
        finally:
            self._sit_out = set()

    # ------------------------------------------------------------------ after the step

    def _finish_reason(self, seq: Sequence, token: int) -> str | None:
        """atom/model_engine/scheduler.py:2296-2329: stop sequences first; only if none matched,
        eos, then stop token ids, then max_tokens."""
        for stop_seq in seq.stop_token_sequences:
            n = len(stop_seq)
            if n and seq.num_completion_tokens >= 1 and seq.token_ids[-n:] == list(stop_seq):
                return "stop_sequence"
        if not seq.ignore_eos and token == self.eos_token_id:
            return "eos"
        if not seq.ignore_eos and token in self.stop_token_ids:
            return f"stop_{token}"
        if seq.num_completion_tokens >= seq.max_tokens:
            return "max_tokens"
        if seq.num_tokens >= self.max_model_len:
            return "max_model_len"
        return None

    def postprocess(self, batch: ScheduledBatch, sampled: dict[int, int], step_seconds: float = 0.0) -> list[Sequence]:
        """``sampled`` maps sequence id -> sampled token for every final item.  Returns the
        sequences that finished."""
        finished = []
        now = self.clock()
        if batch.num_prefill:
            self._last_prompt_latency = step_seconds
        for it in batch.items:
            seq = it.seq
            if seq.status != SequenceStatus.RUNNING:
                continue   # it finished while this batch, scheduled ahead, was running: the result is dropped
            if not seq.awaits_token:
                seq.num_cached_tokens = it.start + it.num_tokens
            if not it.is_final:
                seq.is_partial_prefill = True
                continue
            seq.is_partial_prefill = False
            token = sampled[seq.id]
            if seq.awaits_token:   # scheduled ahead meanwhile: the placeholder becomes the token
                seq.resolve_placeholder(token)
                self.core.resolve(seq.id, seq.num_tokens - 1, token)
            else:
                seq.append_token(token)
            if seq.first_token_time == 0.0:
                seq.first_token_time = now
            reason = self._finish_reason(seq, token)
            if reason is not None:
                seq.status = SequenceStatus.FINISHED
                seq.leave_reason = reason
                seq.leave_time = now
                self.core.close(seq.id)
                self.running.remove(seq)
                finished.append(seq)
        return finished
