"""A plain, slow Qwen3-dense forward pass: whole sequences, no cache, no batching.

Written from the formulas in ROCm/ATOM's sources (read, not run); every function
cites the file and lines it follows.  It shares no code with the engine: it reads
``config.json`` and ``model.safetensors`` itself, keeps everything in one floating
type (float64 by default) and recomputes the whole prefix for every call.

The functions take plain tensors so that each can be pinned on its own by a
library routine or an invariant (see ``test_plain_model.py``).
"""

from __future__ import annotations

import json
import os

import torch


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x * rsqrt(mean(x^2, last dim) + eps) * weight``.

    atom/model_ops/layernorm.py:560-564 (``RMSNormGated.forward_native``) and
    :702-708 (``GemmaRMSNorm.forward_static``, which differs only by ``1 + w``):
    the variance is a mean over the last dimension, eps is added inside the root.
    """
    variance = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight


def add_rms_norm(x, residual, weight, eps):
    """Add first, then normalise; both the normed value and the sum are returned.

    atom/model_ops/layernorm.py:66-75 (``rmsnorm2d_fwd_with_add_``: residual_out
    receives ``x + residual``, the output its norm) used at atom/models/qwen3.py:252,256,310.
    """
    summed = x + residual
    return rms_norm(summed, weight, eps), summed


def rope_angles(positions: torch.Tensor, rotary_dim: int, theta: float) -> tuple[torch.Tensor, torch.Tensor]:
    """cos and sin of ``pos * theta^(-2j/rotary_dim)``, j in [0, rotary_dim/2).

    atom/model_ops/rotary_embedding.py:58-80: ``inv_freq = 1 / base**(arange(0, d, 2)/d)``
    and ``freqs = outer(t, inv_freq)``, both in float32.  The angle is formed in
    float32 here as well (that is what fixes the table), then widened.
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    freqs = torch.einsum("i,j->ij", positions.to(torch.float32), inv_freq)
    return freqs.cos(), freqs.sin()


def rope_neox(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate pairs ``(j, j + d/2)`` of the last dimension (NeoX style).

    atom/model_ops/rotary_embedding.py:14-24 (``apply_rotary_emb``): the halves are
    ``x1, x2``; ``y1 = x1 cos - x2 sin``; ``y2 = x2 cos + x1 sin``.
    ``x`` is [tokens, heads, d]; cos/sin are [tokens, d/2].
    """
    cos = cos.unsqueeze(-2).to(x.dtype)
    sin = sin.unsqueeze(-2).to(x.dtype)
    x1, x2 = torch.chunk(x, 2, dim=-1)
    y1 = x1 * cos - x2 * sin
    y2 = x2 * cos + x1 * sin
    return torch.cat((y1, y2), dim=-1)


def causal_attention(q, k, v, scale: float, window: int | None = None, q_positions=None, k_positions=None):
    """Softmax attention of every query head over the keys it may see.

    atom/model_ops/attention_mha.py:751-765: ``causal=True``, ``softmax_scale=scale``,
    no sinks, no soft cap.  Query head h reads KV head ``h // (Hq // Hkv)``
    (grouped heads; the kernels assert ``Hq % Hkv == 0``, attention_mha.py:532).
    A query at absolute position p sees keys 0..p; with a window W only the last W
    of them, keys p-W+1..p (``window_size=(W-1, 0)``, attention_mha.py:499-501,793-795).

    q is [Tq, Hq, D]; k and v are [Tk, Hkv, D].  Positions default to 0..T-1.
    """
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    assert hq % hkv == 0
    group = hq // hkv
    if q_positions is None:
        q_positions = torch.arange(tk - tq, tk)
    if k_positions is None:
        k_positions = torch.arange(tk)
    out = torch.empty_like(q)
    for h in range(hq):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.T) * scale  # [Tq, Tk]
        dist = q_positions[:, None] - k_positions[None, :]
        hidden = dist < 0
        if window is not None:
            hidden = hidden | (dist >= window)
        scores = scores.masked_fill(hidden, float("-inf"))
        out[:, h, :] = torch.softmax(scores, dim=-1) @ vh
    return out


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """``silu(x[..., :d]) * x[..., d:]``: atom/model_ops/activation.py:78-82."""
    d = x.shape[-1] // 2
    gate = x[..., :d]
    return gate * torch.sigmoid(gate) * x[..., d:]


def gated_mlp(x, w_gate, w_up, w_down):
    """``down(silu(gate(x)) * up(x))``: atom/models/qwen3.py:194-198 with the gate
    rows first in the packed matrix (qwen3.py:321-322)."""
    gate_up = torch.cat((x @ w_gate.T, x @ w_up.T), dim=-1)
    return silu_and_mul(gate_up) @ w_down.T


def self_attention(x, positions, w, cfg, window=None, shared_kv=None):
    """One Qwen3 attention: atom/models/qwen3.py:146-162.

    qkv projection (bias only if ``attention_bias``, qwen3.py:95), per-head RMS norm
    of q and k over the head dimension *before* the rotation (qwen3.py:159-160, the
    norm sees a ``(-1, D)`` view, layernorm.py:61-63), NeoX rotation of q and k with
    ``rotary_dim == head_dim`` (qwen3.py:106-112), scaled causal attention with
    ``scale = D**-0.5`` (qwen3.py:88), output projection without bias (qwen3.py:102).

    ``shared_kv`` lets a layer read the keys and values another layer wrote
    instead of its own; it returns the (k, v) it used.
    """
    t = x.shape[0]
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = x @ w["q_proj.weight"].T
    k = x @ w["k_proj.weight"].T
    v = x @ w["v_proj.weight"].T
    if "q_proj.bias" in w:
        q = q + w["q_proj.bias"]
        k = k + w["k_proj.bias"]
        v = v + w["v_proj.bias"]
    q = q.view(t, hq, d)
    k = k.view(t, hkv, d)
    v = v.view(t, hkv, d)
    eps = cfg["rms_norm_eps"]
    q = rms_norm(q, w["q_norm.weight"], eps)
    k = rms_norm(k, w["k_norm.weight"], eps)
    cos, sin = rope_angles(positions, d, cfg["rope_theta"])
    q = rope_neox(q, cos, sin)
    k = rope_neox(k, cos, sin)
    if shared_kv is not None:
        k, v = shared_kv
    o = causal_attention(q, k, v, d ** -0.5, window, positions, positions)
    return o.reshape(t, hq * d) @ w["o_proj.weight"].T, (k, v)


def layer_window(cfg: dict, layer: int) -> int | None:
    """The window of a layer, from ``layer_types`` in the manner of
    atom/models/llama.py:187-191 (``"sliding_attention"`` -> ``config.sliding_window``).
    atom/models/qwen3.py itself passes no window (qwen3.py:125-138); the engine honours
    ``layer_types`` only when ``use_sliding_window`` is set, and so does this function."""
    if not cfg.get("use_sliding_window", False):
        return None
    types = cfg.get("layer_types")
    if types and types[layer] == "sliding_attention":
        return cfg["sliding_window"]
    return None


# --------------------------------------------------------------------------- model


def normalise_config(cfg: dict) -> dict:
    cfg = dict(cfg)
    if cfg.get("head_dim") is None:  # atom/models/qwen3.py:85
        cfg["head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
    if "rope_theta" not in cfg and "rope_parameters" in cfg:
        cfg["rope_theta"] = cfg["rope_parameters"]["rope_theta"]
    assert cfg.get("hidden_act", "silu") == "silu"  # atom/models/qwen3.py:191
    return cfg


def load_folder(folder: str, dtype=torch.float64):
    """Read ``config.json`` and ``model.safetensors`` of a model folder."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = normalise_config(json.load(f))
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return cfg, tensors


def _sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def qwen3_logits(cfg: dict, tensors: dict, ids, order=None, dtype=torch.float64, first_position: int = 0) -> torch.Tensor:
    """Logits [T, V] of one whole sequence.

    atom/models/qwen3.py:297-310: embedding; layer 0 norms the embedding and keeps
    it as the residual (:248-250), later norms add first (:251-252, :256); the MLP
    output and the residual meet in the next norm, at last in ``model.norm`` (:310).
    Logits are ``h @ lm_head.T`` (:359, embed_head.py:252), the head tied to the
    embedding when ``tie_word_embeddings`` (:339-340).

    ``order`` is the list of layer runs: ``(layer, source)`` pairs where ``source``
    is None for a run that writes keys and values of its own, or the index of an
    earlier run whose keys and values this one reads.  Default: each layer once.
    ``first_position`` numbers the tokens from there on instead of 0 (for tests of what positions mean).
    """
    cfg = normalise_config(cfg)
    ids = torch.as_tensor(ids, dtype=torch.long)
    tensors = {k: v.to(dtype) for k, v in tensors.items()}
    positions = torch.arange(ids.numel()) + first_position
    eps = cfg["rms_norm_eps"]
    if order is None:
        order = [(i, None) for i in range(cfg["num_hidden_layers"])]

    hidden = tensors["model.embed_tokens.weight"][ids]
    residual = None
    kv_of_run = []
    for layer, source in order:
        w = _sub(tensors, f"model.layers.{layer}.")
        if residual is None:
            residual = hidden
            hidden = rms_norm(hidden, w["input_layernorm.weight"], eps)
        else:
            hidden, residual = add_rms_norm(hidden, residual, w["input_layernorm.weight"], eps)
        shared = kv_of_run[source] if source is not None else None
        hidden, kv = self_attention(hidden, positions, _sub(w, "self_attn."), cfg, layer_window(cfg, layer), shared)
        kv_of_run.append(kv)
        hidden, residual = add_rms_norm(hidden, residual, w["post_attention_layernorm.weight"], eps)
        m = _sub(w, "mlp.")
        hidden = gated_mlp(hidden, m["gate_proj.weight"], m["up_proj.weight"], m["down_proj.weight"])
    hidden, _ = add_rms_norm(hidden, residual, tensors["model.norm.weight"], eps)
    head = tensors["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else tensors["lm_head.weight"]
    return hidden @ head.T


# --------------------------------------------------------------------------- sampling


def greedy(logits: torch.Tensor) -> torch.Tensor:
    """argmax per row: atom/model_ops/sampler.py:154-155."""
    return logits.argmax(dim=-1)


def exponential_race(logits: torch.Tensor, temperature: torch.Tensor, noise: torch.Tensor, eps: float = 1e-10):
    """``argmax softmax(logits / T) / (E + eps)`` with ``E ~ Exp(1)`` given.

    atom/model_ops/sampler.py:304-310 (``random_sample``, the readable twin of the
    fused op) with the logits divided by the temperature first
    (docs/model_ops_guide.md:440) and the temperature clamped to at least ``eps``
    (atom/model_engine/model_runner.py:2677).
    """
    t = torch.clamp(temperature.to(torch.float64), min=eps).unsqueeze(-1)
    probs = torch.softmax(logits.to(torch.float64) / t, dim=-1)
    return (probs / (noise.to(torch.float64) + eps)).argmax(dim=-1)


def top_k_top_p_filter(probs: torch.Tensor, top_k: int, top_p: float) -> torch.Tensor:
    """Keep the ``top_k`` likeliest tokens and, of those, the shortest prefix whose
    mass reaches ``top_p``; renormalise.  atom/model_ops/sampler.py:265-291: sorted
    descending, a token stays while the mass *before* it is <= top_p, the first
    token always stays."""
    sorted_probs, idx = torch.sort(probs, dim=-1, descending=True)
    before = torch.cumsum(sorted_probs, dim=-1) - sorted_probs
    keep = before <= top_p
    if top_k != -1:
        keep = keep & (torch.arange(probs.shape[-1]) < top_k)
    keep[..., 0] = True
    kept = sorted_probs * keep
    kept = kept / kept.sum(dim=-1, keepdim=True)
    return torch.zeros_like(probs).scatter(-1, idx, kept)
