"""The tiny configurations the tests use, as raw config.json dictionaries.  They differ
in every size and option: head counts and groups, widths that are no power of two, layer
count, vocabulary, the norms' eps, rope base, tied or untied head, bias, window."""

import os

import torch

TINY_A = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=64,
    num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128, vocab_size=256,
    rope_theta=10000.0, rms_norm_eps=1e-6, max_position_embeddings=128, tie_word_embeddings=True,
    attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")

TINY_B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=96,
    num_attention_heads=6, num_key_value_heads=3, head_dim=32, intermediate_size=160, vocab_size=311,
    rope_theta=1000000.0, rms_norm_eps=1e-5, max_position_embeddings=256, tie_word_embeddings=False,
    attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")

# ours: a head size the matrix-core kernels serve, groups of 4, qkv bias, and two layers with a window
TINY_C = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=4, hidden_size=136,
    num_attention_heads=8, num_key_value_heads=2, head_dim=64, intermediate_size=200, vocab_size=517,
    rope_theta=500000.0, rms_norm_eps=3e-6, max_position_embeddings=1024, tie_word_embeddings=False,
    attention_bias=True, use_sliding_window=True, sliding_window=40,
    layer_types=["full_attention", "sliding_attention", "sliding_attention", "full_attention"],
    hidden_act="silu", torch_dtype="bfloat16")

# ours: the head size of the full-size models (128) with groups of 4, a width and a vocabulary that are no
# power of two, a tied head: the kernel variants that serving runs, at a size the plain implementation can follow
TINY_D = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=264,
    num_attention_heads=8, num_key_value_heads=2, head_dim=128, intermediate_size=328, vocab_size=1031,
    rope_theta=1000000.0, rms_norm_eps=1e-6, max_position_embeddings=2048, tie_word_embeddings=True,
    attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")

# ours: a head size that no matrix-core attention kernel serves (48: the general kernel runs in both precisions),
# groups of 3, widths that are multiples of 8 only
TINY_E = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=104,
    num_attention_heads=6, num_key_value_heads=2, head_dim=48, intermediate_size=152, vocab_size=259,
    rope_theta=20000.0, rms_norm_eps=2e-6, max_position_embeddings=512, tie_word_embeddings=False,
    attention_bias=False, use_sliding_window=False, hidden_act="silu", torch_dtype="bfloat16")

# the weights' spread per configuration: (linear and embedding std, norm-weight std)
SPREAD = {"A": (0.02, 0.1), "B": (0.05, 0.2), "C": (0.04, 0.15), "D": (0.03, 0.1), "E": (0.05, 0.12)}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}
SEEDS = {"A": 0, "B": 1, "C": 5, "D": 8, "E": 13}
PAGE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 8}


def write_tiny(folder: str, which: str, dtype=torch.bfloat16) -> str:
    from atom_amd.config import model_config_from_dict
    from atom_amd.weights import write_random_model

    std, norm_std = SPREAD[which]
    cfg = model_config_from_dict(CONFIGS[which])
    return write_random_model(os.path.join(folder, f"tiny_{which}"), cfg, SEEDS[which], std, norm_std, dtype)
