"""Weights by tensor name from safetensors.

Every parameter a model's parts declare names the checkpoint tensors it is made of
(atom/model_loader/weight_dispatch.py:101-145 and the packed placement of
atom/model_ops/linear.py:1830-1863 are the reference's form of this).  The loader
reads each named tensor, checks its shape and copies it into its rows.  Matrices are
kept in bfloat16 for serving (a matrix the checkpoint stores in 32-bit stays 32-bit),
or widened to float32 on the 32-bit path; norm weights and biases are float32; integer
tensors become int32.  Unlike the reference, which only warns
(atom/model_loader/loading_core.py:389-468), anything missing, unexpected or
mis-shaped is one error that lists all of it.  What the reference's checkpoint rewriter
drops by the form of a name (atom/model_loader/weight_names.py:160-201: cache scales,
``inv_freq`` tables, layers beyond ``num_hidden_layers``) is dropped here too, through
the model's ``drops(name)``, with a debug line in the log.
"""

from __future__ import annotations

import json
import logging
import os
from typing import Callable

import torch

from ..parts.base import ParamSpec, Part


logger = logging.getLogger("atom_amd")


class WeightError(RuntimeError):
    def __init__(self, missing, unexpected, mismatched, where: str):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.mismatched = sorted(mismatched)
        lines = [f"the weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.mismatched:
            lines.append(f"  wrong shape ({len(self.mismatched)}): " + "; ".join(
                f"{n}: checkpoint {tuple(got)} vs model {tuple(want)}" for n, got, want in self.mismatched))
        super().__init__("\n".join(lines))


def param_dtype(spec: ParamSpec, stored: torch.dtype | None, serving: torch.dtype) -> torch.dtype:
    if spec.kind == "vector":
        return torch.float32
    if spec.kind == "table":
        return torch.int32
    if serving == torch.float32:
        return torch.float32
    # serving in bfloat16: 16-bit stays 16-bit (as bfloat16); a matrix stored in 32-bit stays so
    if stored is not None and stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


class TensorSource:
    """Named tensors: ``names()``, ``shape(name)``, ``dtype(name)``, ``get(name)``."""

    where = "<memory>"

    def names(self) -> list[str]:
        raise NotImplementedError

    def shape(self, name: str) -> tuple[int, ...]:
        raise NotImplementedError

    def dtype(self, name: str) -> torch.dtype:
        raise NotImplementedError

    def get(self, name: str) -> torch.Tensor:
        raise NotImplementedError


class SafetensorsFolder(TensorSource):
    """All ``*.safetensors`` files of a folder (atom/model_loader/weight_iterator.py:240-249,
    322-327); with an index file every shard it names must exist
    (atom/model_loader/loading_core.py:53-88)."""

    def __init__(self, folder: str):
        from safetensors import safe_open

        self.where = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        files = sorted(f for f in os.listdir(folder) if f.endswith(".safetensors"))
        if os.path.isfile(index):
            with open(index) as f:
                named = sorted(set(json.load(f)["weight_map"].values()))
            absent = [n for n in named if not os.path.isfile(os.path.join(folder, n))]
            if absent:
                shown = ", ".join(absent[:20]) + (" ..." if len(absent) > 20 else "")
                raise FileNotFoundError(f"{folder}: the index names {len(absent)} shard(s) that are not there: {shown}")
            files = named
        if not files:
            raise FileNotFoundError(f"no .safetensors file in {folder!r}")
        self._handles = []
        self._where: dict[str, object] = {}
        for name in files:
            handle = safe_open(os.path.join(folder, name), framework="pt", device="cpu")
            self._handles.append(handle)
            for key in handle.keys():
                self._where.setdefault(key, handle)

    def names(self):
        return list(self._where)

    def shape(self, name):
        return tuple(self._where[name].get_slice(name).get_shape())

    def dtype(self, name):
        return _ST_DTYPES[self._where[name].get_slice(name).get_dtype()]

    def get(self, name):
        return self._where[name].get_tensor(name)


_ST_DTYPES = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
              "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
              "BOOL": torch.bool}


class DictSource(TensorSource):
    def __init__(self, tensors: dict[str, torch.Tensor], where: str = "<memory>"):
        self.tensors = tensors
        self.where = where

    def names(self):
        return list(self.tensors)

    def shape(self, name):
        return tuple(self.tensors[name].shape)

    def dtype(self, name):
        return self.tensors[name].dtype

    def get(self, name):
        return self.tensors[name]


def expected_tensors(model: Part) -> dict[str, tuple[tuple[int, ...], ParamSpec]]:
    """Checkpoint tensor name -> (shape, the parameter spec it belongs to)."""
    out = {}
    for part in model.walk():
        for spec in part.param_specs().values():
            for src in spec.sources:
                out[part.full_name(src.name)] = ((src.rows, *spec.shape[1:]), spec)
    return out


def load_weights(model: Part, source: TensorSource, device, dtype: torch.dtype,
                 progress: Callable[[str], None] | None = None) -> None:
    """Fills every declared parameter of ``model`` from ``source`` or raises ``WeightError``."""
    expected = expected_tensors(model)
    present = set(source.names())
    drops = getattr(model, "drops", None)
    missing = [n for n in expected if n not in present]
    unexpected = []
    for n in sorted(present):
        if n in expected:
            continue
        why = drops(n) if drops is not None else None
        if why is None:
            unexpected.append(n)
        else:
            logger.debug("checkpoint tensor %s dropped: %s", n, why)
    mismatched = [(n, source.shape(n), shape) for n, (shape, _) in expected.items()
                  if n in present and tuple(source.shape(n)) != tuple(shape)]
    if missing or unexpected or mismatched:
        raise WeightError(missing, unexpected, mismatched, source.where)

    done = 0
    for part in model.walk():
        for local, spec in part.param_specs().items():
            stored = {source.dtype(part.full_name(s.name)) for s in spec.sources}
            widest = torch.float32 if (torch.float32 in stored or torch.float64 in stored) else next(iter(stored))
            target = param_dtype(spec, widest, dtype)
            param = torch.empty(spec.shape, dtype=target, device=device)
            for s in spec.sources:
                tensor = source.get(part.full_name(s.name))
                param[s.offset:s.offset + s.rows].copy_(tensor.to(device=device, dtype=target), non_blocking=False)
            part.params[local] = param
            done += 1
            if progress and done % 64 == 0:
                progress(f"loaded {done} parameters")
    for part in model.walk():
        part.finalize(torch.device(device), dtype)
    model.dtype = dtype
    model.device = torch.device(device)


def load_model_folder(model: Part, folder: str, device, dtype: torch.dtype, progress=None) -> None:
    load_weights(model, SafetensorsFolder(folder), device, dtype, progress)
