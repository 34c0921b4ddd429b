from .core import EngineCore, StepEntry, build_core, load_model

__all__ = ["EngineCore", "StepEntry", "build_core", "load_model"]
