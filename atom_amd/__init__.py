"""atom_amd: a small single-GPU inference engine for AMD MI355X (gfx950)."""

from .config import Config
from .engine.llm_engine import LLMEngine
from .sampling.params import SamplingParams

__all__ = ["Config", "LLMEngine", "SamplingParams"]
