"""What one step hands to the parts: the kernel library, the flat token axis and the batch's
arrays on the device; per group of layers that share block tables, where keys are written and
read; and whatever each mixer asked for in its ``prepare_step``.

Everything a kernel needs to know about the batch is a device array here, in eager steps and in
steps replayed from a captured graph alike.  The host-side lists exist only in eager steps."""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.kinds import KVBinding, StateBinding  # noqa: F401  (their home used to be this module)


@dataclass
class BatchView:
    """A step's batch as a mixer's ``prepare_step`` sees it, on the host.  Requests that bring more
    than one token (prompt portions) come first on the token axis, the single tokens after them."""

    ops: object
    dtype: torch.dtype             # the type of the step's activations
    q_lens: list[int]              # tokens of each request in this step
    cached: list[int]              # tokens of each request before this step
    num_prefill: int               # how many requests bring more than one token
    page_sizes: list[int]          # of each group of layers
    # The step is (or will be) replayed from a captured graph: the arrays' shapes may depend only on the
    # number of requests and on the two capacities below.  Request rows without a live request are padding:
    # single-token rows with no context, and, where prompt portions are held, one row behind the
    # ``prefill_slots`` portion rows that owns the unused token rows (it counts in ``num_prefill``; a portion
    # row that is not in use has no tokens).
    replayed: bool = False
    prefill_capacity: int = 0      # replayed: token rows set aside for prompt portions
    prefill_slots: int = 0         # replayed: request rows set aside for prompt portions

    def portions(self) -> list[int]:
        """The request rows that bring a prompt portion in this step."""
        rows = range(self.prefill_slots) if self.replayed else range(self.num_prefill)
        return [b for b in rows if self.q_lens[b] > 1]

    def tile_capacity(self, rows: int) -> int:
        """How many tiles of ``rows`` query rows the portions of a replayed step can need at most."""
        return -(-self.prefill_capacity // rows) + self.prefill_slots

    @property
    def num_seqs(self) -> int:
        return len(self.q_lens)

    @property
    def max_q_len(self) -> int:
        """The most tokens a request brings (in a replayed step: can bring)."""
        if self.replayed:
            return max(self.prefill_capacity, 1)
        return max(self.q_lens) if self.q_lens else 0


@dataclass
class StepContext:
    ops: object
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_seqs: int
    positions: torch.Tensor                      # int32 [T] absolute position of each token in its request
    token_seq: torch.Tensor | None = None        # int32 [T] row of its request (-1: padding)
    cu_seqlens_q: torch.Tensor | None = None     # int32 [S + 1] first token of each request
    context_lens: torch.Tensor | None = None     # int32 [S] tokens of each request once this step has run
    cached_lens: torch.Tensor | None = None      # int32 [S] tokens of each request before this step
    slot_of_seq: torch.Tensor | None = None      # int32 [S] state slot of each request (-1: padding)
    block_tables: dict[int, torch.Tensor] = field(default_factory=dict)   # per group: int32 [S, width]
    slot_mappings: dict[int, torch.Tensor] = field(default_factory=dict)  # per group: int32 [T] (-1: no write)
    page_sizes: dict[int, int] = field(default_factory=dict)
    # host numbers that pick kernels and grids (upper bounds in a replayed step)
    num_prefill: int = 0
    max_q_len: int = 1
    max_context_len: int = 0
    replayed: bool = False
    # what each mixer's ``prepare_step`` returned, on the device: step key -> name -> int32 tensor
    prepared: dict = field(default_factory=dict)
    # a scratch dictionary for parts: what one layer derived from the above and the next can use again
    memo: dict = field(default_factory=dict)
    # host-side copies, for mixers that walk requests themselves; None in a replayed step
    seq_starts: list[int] | None = None   # first row of each request in the token axis
    seq_lens: list[int] | None = None     # rows of each request in this step
    seq_cached: list[int] | None = None   # tokens of each request before this step
    state_slots: list[int] | None = None  # state slot of each request


def pack_int32(pieces: list[np.ndarray]) -> tuple[list[int], int]:
    """Offsets of the pieces in one int32 buffer (each padded to 4 ints) and the buffer's length."""
    offsets, cursor = [], 0
    for p in pieces:
        offsets.append(cursor)
        cursor += (int(p.size) + 3) // 4 * 4
    return offsets, max(cursor, 4)
