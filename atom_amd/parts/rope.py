"""Rotary position encoding: float32 cos/sin tables [max_positions, rotary_dim / 2].

atom/model_ops/rotary_embedding.py:58-80: ``inv_freq_j = base ** (-2j / rotary_dim)``,
``angle = position * inv_freq`` and its cos and sin, all float32.  The reference then
casts the tables to the model's type (:48-50); here they stay float32 and the rotation
is done in float32 by the kernel that also norms q/k and writes the cache.
"""

from __future__ import annotations

import torch

from .base import POSITION_ENCODINGS, PositionEncoding

_TABLES: dict = {}


class RotaryEncoding(PositionEncoding):
    """NeoX-style rotation of the first ``rotary_dim`` elements of each head."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None,
                 prefix: str = ""):
        super().__init__(prefix)
        self.head_dim = head_dim
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError(f"rotary_dim must be even and in (0, head_dim], got {self.rotary_dim}")
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def finalize(self, device, dtype):
        key = (self.rotary_dim, self.theta, self.max_positions, str(device))
        if key not in _TABLES:
            inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim))
            t = torch.arange(self.max_positions, dtype=torch.float32)
            freqs = torch.einsum("i,j->ij", t, inv_freq)
            _TABLES[key] = (freqs.cos().contiguous().to(device), freqs.sin().contiguous().to(device))
        self.cos, self.sin = _TABLES[key]


POSITION_ENCODINGS.register("rotary", RotaryEncoding)
