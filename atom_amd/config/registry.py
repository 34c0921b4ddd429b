"""One registry from an architecture's name (``architectures[0]`` of config.json, as
atom/model_engine/model_runner.py:98-124,699 looks it up) to its configuration class
and the function that turns a configuration into a model."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .model_config import ConfigError, ModelConfig, Qwen3Config


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build_spec: Callable  # ModelConfig -> ModelSpec


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build_spec: Callable, *, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise KeyError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list[str]:
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture {name!r} is not supported; supported: {known_architectures()}")
    return _ARCHITECTURES[name]


def model_config_from_dict(raw: dict) -> ModelConfig:
    archs = raw.get("architectures")
    if not archs:
        raise ConfigError("config.json lacks 'architectures'")
    return get_architecture(archs[0]).config_class.from_dict(raw)


def build_model(config: ModelConfig):
    """The (unloaded) model a configuration describes."""
    from ..models.model import CausalLM

    return CausalLM(get_architecture(config.architecture).build_spec(config))


_builtin_done = False


def _ensure_builtin() -> None:
    """Registers the architectures that ship with the engine, on first use."""
    global _builtin_done
    if _builtin_done:
        return
    _builtin_done = True
    from ..models.qwen3 import qwen3_spec

    if "Qwen3ForCausalLM" not in _ARCHITECTURES:
        register_architecture("Qwen3ForCausalLM", Qwen3Config, qwen3_spec)
