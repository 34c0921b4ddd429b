"""The engine's configuration, with ATOM's names and meanings
(atom/config.py:1424-1540) for what this engine has, plus ``dtype`` and ``seed``."""

from __future__ import annotations

from dataclasses import dataclass, field

from .model_config import ConfigError, ModelConfig, read_config_json

DTYPES = {"bf16": "bfloat16", "bfloat16": "bfloat16", "fp32": "float32", "float32": "float32"}


@dataclass
class Config:
    model: str
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int | None = None
    gpu_memory_utilization: float = 0.9
    enforce_eager: bool = False
    kv_cache_block_size: int = 16
    num_kvcache_blocks: int = -1
    kv_cache_dtype: str = "bf16"
    enable_prefix_caching: bool = True
    enable_chunked_prefill: bool = True
    long_prefill_token_threshold: int = 0
    scheduler_delay_factor: float = 0.0
    load_dummy: str | None = None
    torch_profiler_dir: str | None = None
    mark_trace: bool = False
    deferred_output: bool = True
    cudagraph_capture_sizes: list[int] = field(default_factory=lambda: [1, 2, 4, 8, 16, 32, 48, 64, 128, 256])
    # Steps that hold prompt portions beside decode tokens are replayed as graphs too when the portions
    # together have at most one of these many tokens (one graph per listed size and decode size of 8 and more).
    # Off by default: on an MI355X such steps keep the GPU busy when launched one by one, as long as they are
    # launched ahead (deferred_output), and a graph pads every step to its bucket.
    cudagraph_prefill_sizes: list[int] = field(default_factory=list)
    cudagraph_prefill_slots: int = 2      # prompt portions such a graph holds at most
    hf_overrides: dict | None = None
    dtype: str = "bf16"
    seed: int = 0
    device: str = "cuda:0"
    bos_token_id: int = -1
    eos_token_id: int = -1
    stop_token_ids: list[int] = field(default_factory=list)
    model_config: ModelConfig | None = None

    def __post_init__(self):
        from .registry import model_config_from_dict

        if self.dtype not in DTYPES:
            raise ConfigError(f"dtype must be one of {sorted(DTYPES)}, got {self.dtype!r}")
        self.dtype = DTYPES[self.dtype]
        if self.kv_cache_dtype not in ("bf16", "auto"):
            raise ConfigError("kv_cache_dtype: only 'bf16' (the model's own type) is built; quantized caches are not")
        if self.model_config is None:
            raw = read_config_json(self.model)
            if self.hf_overrides:  # atom/config.py:1699-1701
                raw = {**raw, **self.hf_overrides}
            self.model_config = model_config_from_dict(raw)
        mc = self.model_config
        # atom/config.py:1745-1753: max_model_len is clamped by the model's positions
        if self.max_model_len is None:
            self.max_model_len = mc.max_position_embeddings
        self.max_model_len = min(self.max_model_len, mc.max_position_embeddings)
        if self.kv_cache_block_size <= 0:     # what else a page size must be is the mixers' to say (plan_cache)
            raise ConfigError("kv_cache_block_size must be positive")
        # atom/config.py:1755-1767
        if self.long_prefill_token_threshold:
            if self.long_prefill_token_threshold > self.max_model_len:
                raise ConfigError("long_prefill_token_threshold must not exceed max_model_len")
            if self.long_prefill_token_threshold < self.kv_cache_block_size:
                raise ConfigError("long_prefill_token_threshold must be at least one cache block")
        if self.max_num_seqs <= 0 or self.max_num_batched_tokens <= 0:
            raise ConfigError("max_num_seqs and max_num_batched_tokens must be positive")
        if not (0.0 < self.gpu_memory_utilization <= 1.0):
            raise ConfigError("gpu_memory_utilization must be in (0, 1]")
        # atom/model_engine/llm_engine.py:48-53 and atom/config.py:1724-1729
        eos = mc.eos_token_id
        if self.eos_token_id == -1 and eos is not None:
            if isinstance(eos, (list, tuple)):
                self.eos_token_id = eos[0]
                self.stop_token_ids = sorted(set(self.stop_token_ids) | set(eos[1:]))
            else:
                self.eos_token_id = eos
        if self.bos_token_id == -1 and mc.bos_token_id is not None:
            self.bos_token_id = mc.bos_token_id
