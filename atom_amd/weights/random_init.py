"""The random-weights mode: from a configuration and a seed, every tensor a checkpoint
of that model would hold, either in memory or written as a model folder
(``config.json`` + ``model.safetensors``) that the name-based loader then reads like
any other.  The reference's ``--load_dummy`` (atom/model_loader/loader.py:178-227) is
unseeded and fills the live parameters; this one is seeded per tensor name, so a
tensor's values depend on the seed and its name only.

Matrices and embeddings are N(0, std); norm weights are 1 + N(0, norm_std), so that a
norm weight that is dropped or put in the wrong place changes the result; biases are
N(0, std).
"""

from __future__ import annotations

import os
import zlib

import torch

from ..config.model_config import ModelConfig
from ..config.registry import build_model
from .loader import TensorSource, expected_tensors


def random_tensor(name: str, shape, init: str, seed: int, std: float, norm_std: float,
                  dtype: torch.dtype, device: str = "cpu") -> torch.Tensor:
    """Drawn on ``device``; the values depend on (seed, name, device kind) only."""
    g = torch.Generator(device=device)
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    if init == "zeros":
        t = torch.zeros(shape, device=device)
    elif init == "one_plus_normal":
        t = 1.0 + norm_std * torch.randn(shape, generator=g, device=device)
    elif init == "normal":
        t = torch.randn(shape, generator=g, device=device, dtype=torch.float32 if device == "cpu" else dtype) * std
    else:
        raise ValueError(f"unknown init {init!r}")
    return t.to(dtype)


class RandomSource(TensorSource):
    """Draws each tensor when it is asked for (nothing is held: an 8B model streams through)."""

    def __init__(self, model, seed: int, std: float = 0.02, norm_std: float = 0.1,
                 dtype: torch.dtype = torch.bfloat16, device: str = "cpu"):
        self.expected = expected_tensors(model)
        self.seed, self.std, self.norm_std, self._dtype = seed, std, norm_std, dtype
        self.device = device
        self.where = f"<random weights, seed {seed}>"

    def names(self):
        return list(self.expected)

    def shape(self, name):
        return tuple(self.expected[name][0])

    def dtype(self, name):
        return self._dtype

    def get(self, name):
        shape, spec = self.expected[name]
        init = "normal" if spec.init == "normal" else spec.init
        return random_tensor(name, shape, init, self.seed, self.std, self.norm_std, self._dtype, self.device)


def random_state_dict(config: ModelConfig, seed: int, std: float = 0.02, norm_std: float = 0.1,
                      dtype: torch.dtype = torch.bfloat16) -> dict[str, torch.Tensor]:
    src = RandomSource(build_model(config), seed, std, norm_std, dtype)
    return {name: src.get(name) for name in sorted(src.names())}


def write_random_model(folder: str, config: ModelConfig, seed: int, std: float = 0.02, norm_std: float = 0.1,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes ``config.json`` and ``model.safetensors``; returns the folder."""
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    tensors = random_state_dict(config, seed, std, norm_std, dtype)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"),
              metadata={"format": "pt"})
    return folder
