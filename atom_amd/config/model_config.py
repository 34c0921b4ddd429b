"""Typed model configurations read from a checkpoint's own ``config.json`` keys.

Every size and constant a model needs comes from here; no model code holds one.
The fields and fallbacks follow what ATOM reads from the HF config for
``Qwen3ForCausalLM`` (atom/models/qwen3.py:211-239, atom/config.py:1708-1753).
"""

from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine can run."""


_MISSING = object()


def _take(raw: dict, key: str, kind, default=_MISSING):
    if key not in raw or raw[key] is None:
        if default is _MISSING:
            raise ConfigError(f"config.json lacks the required key '{key}'")
        return default
    value = raw[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if kind is int and isinstance(value, bool) or not isinstance(value, kind):
        raise ConfigError(f"config.json key '{key}' must be {kind.__name__}, got {value!r}")
    return value


@dataclass(frozen=True)
class ModelConfig:
    """What every architecture's configuration has in common."""

    architecture: str
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    torch_dtype: str
    bos_token_id: int | None
    eos_token_id: int | list[int] | None

    #: keys of config.json each subclass understands, for the round trip in to_dict()
    model_type: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: dict) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        raise NotImplementedError

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)

    def replace(self, **changes) -> "ModelConfig":
        return type(self).from_dict({**self.to_dict(), **changes})


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    """``Qwen3ForCausalLM``: grouped-query attention with per-head q/k norms, rotary
    positions, a SiLU-gated dense feed-forward and RMS norms."""

    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    hidden_act: str = "silu"
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    attention_bias: bool = False
    use_sliding_window: bool = False
    sliding_window: int | None = None
    layer_types: tuple[str, ...] | None = None

    model_type: ClassVar[str] = "qwen3"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        archs = raw.get("architectures") or [None]
        hidden = _take(raw, "hidden_size", int)
        heads = _take(raw, "num_attention_heads", int)
        # atom/models/qwen3.py:85,221: head_dim falls back to hidden_size // heads
        head_dim = _take(raw, "head_dim", int, hidden // heads)
        # atom/config.py:1708-1722: rope_theta may live under rope_parameters
        rope = raw.get("rope_parameters") or {}
        theta = rope.get("rope_theta", raw.get("rope_theta"))
        if theta is None:
            raise ConfigError("config.json lacks 'rope_theta' (or rope_parameters.rope_theta)")
        scaling = raw.get("rope_scaling")
        rope_type = (scaling or {}).get("rope_type", (scaling or {}).get("type", rope.get("rope_type", "default")))
        if rope_type not in ("default", None):
            raise ConfigError(f"rope scaling of type {rope_type!r} is not supported for {archs[0]}")
        layers = _take(raw, "num_hidden_layers", int)
        layer_types = raw.get("layer_types")
        if layer_types is not None:
            layer_types = tuple(layer_types)
        cfg = cls(
            architecture=archs[0] or "Qwen3ForCausalLM",
            vocab_size=_take(raw, "vocab_size", int),
            hidden_size=hidden,
            num_hidden_layers=layers,
            # atom/config.py:1745-1753: 8192 when the checkpoint names none
            max_position_embeddings=_take(raw, "max_position_embeddings", int, 8192),
            tie_word_embeddings=_take(raw, "tie_word_embeddings", bool, False),
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            num_attention_heads=heads,
            num_key_value_heads=_take(raw, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            intermediate_size=_take(raw, "intermediate_size", int),
            hidden_act=_take(raw, "hidden_act", str, "silu"),
            rms_norm_eps=_take(raw, "rms_norm_eps", float, 1e-6),
            rope_theta=float(theta),
            attention_bias=_take(raw, "attention_bias", bool, False),
            use_sliding_window=_take(raw, "use_sliding_window", bool, False),
            sliding_window=raw.get("sliding_window"),
            layer_types=layer_types,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        def positive(name):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")

        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            positive(name)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim must be even for rotary pairs, got {self.head_dim}")
        if self.hidden_act != "silu":  # atom/models/qwen3.py:191
            raise ConfigError(f"hidden_act must be 'silu', got {self.hidden_act!r}")
        if self.rms_norm_eps <= 0:
            raise ConfigError("rms_norm_eps must be positive")
        if self.layer_types is not None and len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(
                f"layer_types has {len(self.layer_types)} entries for {self.num_hidden_layers} layers")
        if self.use_sliding_window and self.layer_types and "sliding_attention" in self.layer_types:
            if not self.sliding_window or self.sliding_window <= 0:
                raise ConfigError("sliding layers need a positive sliding_window")

    def window_of_layer(self, layer: int) -> int | None:
        """The attention window of a layer or None for all keys: ``layer_types`` read
        as atom/models/llama.py:187-191 does, and only when ``use_sliding_window``."""
        if self.use_sliding_window and self.layer_types and self.layer_types[layer] == "sliding_attention":
            return self.sliding_window
        return None

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
        }
        for f in dataclasses.fields(self):
            if f.name == "architecture":
                continue
            value = getattr(self, f.name)
            if isinstance(value, tuple):
                value = list(value)
            out[f.name] = value
        return out


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    with open(path) as f:
        return json.load(f)
