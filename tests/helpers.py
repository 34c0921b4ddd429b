"""Shared test helpers: tiny model folders, the engine on them, the oracle's logits."""

from __future__ import annotations

import functools
import os
import tempfile

import torch

import plain_model
from tiny import CONFIGS, PAGE, write_tiny

_TMP = tempfile.TemporaryDirectory(prefix="atom_amd_tests_")


@functools.lru_cache(maxsize=None)
def tiny_folder(which: str, stored: str = "bfloat16") -> str:
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored]
    return write_tiny(os.path.join(_TMP.name, stored), which, dtype)


@functools.lru_cache(maxsize=None)
def oracle_weights(which: str, stored: str = "bfloat16"):
    return plain_model.load_folder(tiny_folder(which, stored))


def oracle_logits(which: str, ids, order=None, stored: str = "bfloat16") -> torch.Tensor:
    cfg, tensors = oracle_weights(which, stored)
    return plain_model.qwen3_logits(cfg, tensors, ids, order=order)


def random_ids(which: str, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[which]["vocab_size"], (n,), generator=g).tolist()


_OPS = {}


def gpu_ops():
    from atom_amd.kernels.hip import HipKernels

    if "hip" not in _OPS:
        _OPS["hip"] = HipKernels("cuda:0")
    return _OPS["hip"]


def make_core(which: str, dtype: str, ops, device: str, num_pages: int = 64, max_num_seqs: int = 8,
              page_size: int | None = None, stored: str = "bfloat16", order=None, graph_sizes=None):
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model

    tdtype = TORCH_DTYPES[dtype]
    model, _ = load_model(tiny_folder(which, stored), dtype=tdtype, device=device)
    if order is not None:
        from atom_amd.models.model import LayerRun

        model.order = [LayerRun(layer, src) for layer, src in order]
    return build_core(model, ops, dtype=tdtype, device=device, page_size=page_size or PAGE[which],
                      num_pages=num_pages, max_num_seqs=max_num_seqs, graph_sizes=graph_sizes)
