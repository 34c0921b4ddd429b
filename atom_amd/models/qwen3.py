"""Qwen3 dense (``Qwen3ForCausalLM``) as a ``ModelSpec``: atom/models/qwen3.py:201-340.

Every layer is a pre-norm block of grouped-query attention (per-head q/k RMS norms,
rotary positions over the whole head, optional qkv bias) and a SiLU-gated MLP; all
norms share ``rms_norm_eps``.  ATOM's Qwen3 passes no sliding window (qwen3.py:125-138);
here a layer marked ``"sliding_attention"`` in ``layer_types`` gets ``sliding_window``
when ``use_sliding_window`` is set, read as atom/models/llama.py:187-191 reads it.
"""

from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..parts.base import PartChoice
from .model import ModelSpec


def qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    ffn = PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                                   "activation": cfg.hidden_act})
    rope = PartChoice("rotary", {"theta": cfg.rope_theta, "max_positions": cfg.max_position_embeddings})
    blocks = []
    for layer in range(cfg.num_hidden_layers):
        mixer = PartChoice("attention", {
            "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim, "qkv_bias": cfg.attention_bias,
            "qk_norm": True, "norm_eps": cfg.rms_norm_eps, "window": cfg.window_of_layer(layer),
            "position_encoding": rope})
        blocks.append(PartChoice("prenorm", {"mixer": mixer, "feed_forward": ffn, "norm": norm}))
    return ModelSpec(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, blocks=blocks, final_norm=norm,
                     tie_word_embeddings=cfg.tie_word_embeddings, max_positions=cfg.max_position_embeddings)
