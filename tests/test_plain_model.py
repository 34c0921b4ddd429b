"""Pins the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, and invariants, each chosen so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place, an off-by-one mask) fails."""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm
from helpers import oracle_weights, random_ids

D64 = torch.float64


def t(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D64)


# ------------------------------------------------------------------ norm


def test_rms_norm_is_the_library_routine():
    x, w = t(5, 96), 1 + 0.2 * t(96, seed=1)
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), atol=1e-12)


def test_rms_norm_scale_invariance_and_unit_rms():
    x = t(4, 64)
    ones = torch.ones(64, dtype=D64)
    y = pm.rms_norm(x, ones, 0.0)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(4, dtype=D64), atol=1e-12)
    assert torch.allclose(pm.rms_norm(3.7 * x, ones, 0.0), y, atol=1e-12)
    # eps sits inside the root and is added to the mean, not to the sum
    tiny = 1e-3 * x
    want = tiny / torch.sqrt(tiny.pow(2).mean(-1, keepdim=True) + 1e-2)
    assert torch.allclose(pm.rms_norm(tiny, ones, 1e-2), want, atol=1e-12)


def test_add_rms_norm_adds_first_and_returns_the_sum():
    x, r, w = t(3, 32), t(3, 32, seed=1), 1 + 0.1 * t(32, seed=2)
    y, s = pm.add_rms_norm(x, r, w, 1e-6)
    assert torch.equal(s, x + r)
    assert torch.allclose(y, pm.rms_norm(x + r, w, 1e-6))
    assert not torch.allclose(y, pm.rms_norm(x, w, 1e-6) + r)


# ------------------------------------------------------------------ rotation


def test_rope_is_complex_multiplication_of_split_halves():
    """Pairs are (j, j + d/2): as complex numbers x1 + i x2 they are multiplied by e^{i angle}."""
    d, theta = 32, 1e4
    x = t(6, 3, d)
    pos = torch.tensor([0, 1, 2, 7, 50, 127])
    cos, sin = pm.rope_angles(pos, d, theta)
    y = pm.rope_neox(x, cos, sin)
    z = torch.complex(x[..., :d // 2], x[..., d // 2:])
    inv = theta ** (-torch.arange(0, d, 2, dtype=D64) / d)
    rot = torch.polar(torch.ones(6, d // 2, dtype=D64), pos[:, None].to(D64) * inv)
    want = z * rot[:, None, :]
    assert torch.allclose(y[..., :d // 2], want.real, atol=1e-5)
    assert torch.allclose(y[..., d // 2:], want.imag, atol=1e-5)
    # the interleaved pairing (2j, 2j+1) is a different function
    zi = torch.view_as_complex(x.reshape(6, 3, d // 2, 2).contiguous()) * rot[:, None, :]
    assert not torch.allclose(y, torch.view_as_real(zi).reshape(6, 3, d), atol=1e-3)


def test_rope_position_zero_is_identity_and_norm_is_kept():
    x = t(4, 2, 16)
    cos, sin = pm.rope_angles(torch.zeros(4, dtype=torch.long), 16, 1e6)
    assert torch.equal(pm.rope_neox(x, cos, sin), x)
    cos, sin = pm.rope_angles(torch.tensor([3, 9, 100, 255]), 16, 1e6)
    assert torch.allclose(pm.rope_neox(x, cos, sin).norm(dim=-1), x.norm(dim=-1), atol=1e-12)


def test_rope_scores_depend_on_distance_only():
    d = 32
    q, k = t(1, 1, d), t(1, 1, d, seed=1)

    def score(m, n):
        cq, sq = pm.rope_angles(torch.tensor([m]), d, 1e4)
        ck, sk = pm.rope_angles(torch.tensor([n]), d, 1e4)
        return float((pm.rope_neox(q, cq, sq) * pm.rope_neox(k, ck, sk)).sum())

    assert abs(score(5, 2) - score(45, 42)) < 1e-4   # angles are float32
    assert abs(score(5, 2) - score(2, 5)) > 1e-3      # the sign of the distance matters


def test_rope_angles_are_formed_in_float32():
    """The table is what float32 gives: at large positions it differs from a float64 angle."""
    pos = torch.tensor([40000])
    cos, _ = pm.rope_angles(pos, 128, 1e6)
    inv32 = 1.0 / (1e6 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    assert torch.equal(cos, (pos.float()[:, None] * inv32).cos())
    assert cos.dtype == torch.float32


# ------------------------------------------------------------------ attention


def test_attention_is_sdpa_for_a_whole_prompt():
    tq, hq, hkv, d = 17, 6, 3, 32
    q, k, v = t(tq, hq, d), t(tq, hkv, d, seed=1), t(tq, hkv, d, seed=2)
    got = pm.causal_attention(q, k, v, d ** -0.5)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                          is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-10)


def test_attention_special_cases():
    d = 16
    q, k, v = t(1, 4, d), t(1, 2, d, seed=1), t(1, 2, d, seed=2)
    out = pm.causal_attention(q, k, v, 0.25)            # one key: the output is its value
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 3], v[0, 1])
    q, k, v = t(9, 4, d), t(9, 4, d, seed=1), t(9, 4, d, seed=2)   # Hkv == Hq is plain multi-head
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                          is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(pm.causal_attention(q, k, v, d ** -0.5), want, atol=1e-10)


def test_attention_grouping_is_consecutive_heads():
    """Query heads 0..G-1 read KV head 0, the next G read KV head 1 (not interleaved)."""
    q, k, v = t(5, 4, 8), t(5, 2, 8, seed=1), t(5, 2, 8, seed=2)
    out = pm.causal_attention(q, k, v, 1.0)
    alone = pm.causal_attention(q[:, 1:2], k[:, 0:1], v[:, 0:1], 1.0)
    assert torch.allclose(out[:, 1:2], alone)
    alone = pm.causal_attention(q[:, 2:3], k[:, 1:2], v[:, 1:2], 1.0)
    assert torch.allclose(out[:, 2:3], alone)


def test_attention_is_causal_and_bottom_right_aligned():
    tk, d = 12, 8
    q, k, v = t(tk, 2, d), t(tk, 1, d, seed=1), t(tk, 1, d, seed=2)
    whole = pm.causal_attention(q, k, v, 0.3)
    k2, v2 = k.clone(), v.clone()
    k2[8:], v2[8:] = 9.0, -9.0                           # later keys do not touch earlier rows
    assert torch.allclose(pm.causal_attention(q, k2, v2, 0.3)[:8], whole[:8])
    assert not torch.allclose(pm.causal_attention(q, k2, v2, 0.3)[8:], whole[8:])
    # the last 5 queries alone against all keys see what they saw in the whole prompt
    assert torch.allclose(pm.causal_attention(q[-5:], k, v, 0.3), whole[-5:])


def test_attention_window_counts_the_query_itself():
    tk, d, w = 10, 8, 3
    q, k, v = t(tk, 1, d), t(tk, 1, d, seed=1), t(tk, 1, d, seed=2)
    got = pm.causal_attention(q, k, v, 0.5, window=w)
    i = torch.arange(tk)
    mask = (i[:, None] >= i[None, :]) & (i[:, None] - i[None, :] < w)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                          attn_mask=mask, scale=0.5)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-10)
    assert torch.allclose(pm.causal_attention(q, k, v, 0.5, window=1), v.expand(-1, 1, -1))   # only itself


# ------------------------------------------------------------------ feed-forward


def test_mlp_is_silu_gate_times_up():
    x, wg, wu, wd = t(4, 24), t(40, 24, seed=1), t(40, 24, seed=2), t(24, 40, seed=3)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(pm.gated_mlp(x, wg, wu, wd), want, atol=1e-10)
    assert not torch.allclose(pm.gated_mlp(x, wu, wg, wd), want, atol=1e-3), "gate and up are not interchangeable"
    gu = t(3, 10)
    assert torch.allclose(pm.silu_and_mul(gu), F.silu(gu[:, :5]) * gu[:, 5:])


# ------------------------------------------------------------------ whole model


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_model_is_causal(which):
    cfg, tensors = oracle_weights(which)
    ids = random_ids(which, 40, 3)
    whole = pm.qwen3_logits(cfg, tensors, ids)
    assert whole.shape == (40, cfg["vocab_size"])
    assert torch.allclose(pm.qwen3_logits(cfg, tensors, ids[:25]), whole[:25], atol=1e-9)
    other = list(ids)
    other[30] = (other[30] + 1) % cfg["vocab_size"]
    changed = pm.qwen3_logits(cfg, tensors, other)
    assert torch.allclose(changed[:30], whole[:30], atol=1e-9)
    assert not torch.allclose(changed[30:], whole[30:], atol=1e-6)


def test_model_attention_block_is_its_parts_in_order():
    """q/k norm comes before the rotation and acts per head; composing the pinned parts in that
    order reproduces the block, composing them the other way round does not."""
    cfg, tensors = oracle_weights("B")
    w = {k[len("model.layers.0.self_attn."):]: v for k, v in tensors.items() if k.startswith("model.layers.0.self_attn.")}
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    x = t(7, cfg["hidden_size"])
    pos = torch.arange(7)
    got, _ = pm.self_attention(x, pos, w, cfg)
    q = F.linear(x, w["q_proj.weight"]).view(7, hq, d)
    k = F.linear(x, w["k_proj.weight"]).view(7, hkv, d)
    v = F.linear(x, w["v_proj.weight"]).view(7, hkv, d)
    cos, sin = pm.rope_angles(pos, d, cfg["rope_theta"])
    qn = pm.rope_neox(F.rms_norm(q, (d,), w["q_norm.weight"], cfg["rms_norm_eps"]), cos, sin)
    kn = pm.rope_neox(F.rms_norm(k, (d,), w["k_norm.weight"], cfg["rms_norm_eps"]), cos, sin)
    o = F.scaled_dot_product_attention(qn.transpose(0, 1)[None], kn.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                       is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    want = F.linear(o.reshape(7, hq * d), w["o_proj.weight"])
    assert torch.allclose(got, want, atol=1e-9)
    qr = F.rms_norm(pm.rope_neox(q, cos, sin), (d,), w["q_norm.weight"], cfg["rms_norm_eps"])
    assert not torch.allclose(qr, qn, atol=1e-3), "norm after rotation is a different function here"


# The assembly of the parts (what feeds what, where the residual stream starts and where norms sit) is pinned by
# three reductions to library routines and one invariant, each of which a plausible other arrangement fails.


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_model_without_attention_is_a_stack_of_library_mlps(which):
    """With every o_proj zero the mixers add nothing, and what is left is: the residual stream starts as the
    embedding itself (not its norm); each layer adds MLP(norm(stream)) with the post-attention norm's weight;
    the final norm sees the sum (atom/models/qwen3.py:248-258, 310).  Written with library routines only."""
    cfg, tensors = oracle_weights(which)
    ids = random_ids(which, 9, 21)
    silent = {k: (torch.zeros_like(v) if k.endswith("o_proj.weight") else v) for k, v in tensors.items()}
    got = pm.qwen3_logits(cfg, silent, ids)
    eps = cfg["rms_norm_eps"]
    hidden = cfg["hidden_size"]
    head = tensors["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else tensors["lm_head.weight"]

    def stack(stream, norm_of_layer):
        for layer in range(cfg["num_hidden_layers"]):
            p = f"model.layers.{layer}."
            h = F.rms_norm(stream, (hidden,), tensors[p + norm_of_layer], eps)
            act = F.silu(F.linear(h, tensors[p + "mlp.gate_proj.weight"])) * F.linear(h, tensors[p + "mlp.up_proj.weight"])
            stream = stream + F.linear(act, tensors[p + "mlp.down_proj.weight"])
        return F.linear(F.rms_norm(stream, (hidden,), tensors["model.norm.weight"], eps), head)

    embedded = tensors["model.embed_tokens.weight"][torch.tensor(ids)]
    want = stack(embedded, "post_attention_layernorm.weight")
    scale = float(want.abs().max())
    assert torch.allclose(got, want, atol=1e-9 * scale + 1e-12)
    # arrangements that this rules out: the MLP behind the input norm; a stream that starts from the normed embedding
    assert float((stack(embedded, "input_layernorm.weight") - got).abs().max()) > 1e-3 * scale
    normed = F.rms_norm(embedded, (hidden,), tensors["model.layers.0.input_layernorm.weight"], eps)
    assert float((stack(normed, "post_attention_layernorm.weight") - got).abs().max()) > 1e-3 * scale


@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_model_first_token_goes_through_values_only(which):
    """One token sees one key, so attention returns its value whatever queries and keys are: with the MLPs
    silenced (down_proj zero), each layer adds o_proj(v_proj(norm(stream))) with the input norm's weight, the
    value of KV head ``h // group`` under query head h, neither normed per head nor rotated
    (atom/models/qwen3.py:146-162)."""
    cfg, tensors = oracle_weights(which)
    token = random_ids(which, 1, 5)
    silent = {k: (torch.zeros_like(v) if k.endswith("down_proj.weight") else v) for k, v in tensors.items()}
    got = pm.qwen3_logits(cfg, silent, token)
    eps, hidden = cfg["rms_norm_eps"], cfg["hidden_size"]
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    stream = tensors["model.embed_tokens.weight"][torch.tensor(token)]
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        h = F.rms_norm(stream, (hidden,), tensors[p + "input_layernorm.weight"], eps)
        v = F.linear(h, tensors[p + "self_attn.v_proj.weight"], tensors.get(p + "self_attn.v_proj.bias"))
        per_head = v.view(1, hkv, d).repeat_interleave(hq // hkv, dim=1)      # consecutive query heads share a KV head
        stream = stream + F.linear(per_head.reshape(1, hq * d), tensors[p + "self_attn.o_proj.weight"])
    head = tensors["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else tensors["lm_head.weight"]
    want = F.linear(F.rms_norm(stream, (hidden,), tensors["model.norm.weight"], eps), head)
    assert torch.allclose(got, want, atol=1e-9 * float(want.abs().max()) + 1e-12)


@pytest.mark.parametrize("which", ["A", "B", "D"])
def test_model_sees_positions_as_distances_only(which):
    """Numbering the tokens from 37 instead of 0 changes no logit (beyond the float32 angles): the rotation is
    the last thing that happens to queries and keys.  A per-head norm *after* the rotation, with weights that
    differ over the head dimension as they do here, would break this; so would rotating the values."""
    cfg, tensors = oracle_weights(which)
    ids = random_ids(which, 30, 8)
    base = pm.qwen3_logits(cfg, tensors, ids)
    moved = pm.qwen3_logits(cfg, tensors, ids, first_position=37)
    scale = float(base.abs().max())
    assert float((base - moved).abs().max()) <= 2e-4 * scale
    # the other order is not invariant: the same check on one attention layer with the norm after the rotation
    w = {k[len("model.layers.0.self_attn."):]: v for k, v in tensors.items() if k.startswith("model.layers.0.self_attn.")}
    hq, hkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    x = t(12, cfg["hidden_size"], seed=3)

    def norm_after_rotation(first):
        pos = torch.arange(12) + first
        cos, sin = pm.rope_angles(pos, d, cfg["rope_theta"])
        q = F.rms_norm(pm.rope_neox(F.linear(x, w["q_proj.weight"]).view(12, hq, d), cos, sin), (d,), w["q_norm.weight"], 1e-6)
        k = F.rms_norm(pm.rope_neox(F.linear(x, w["k_proj.weight"]).view(12, hkv, d), cos, sin), (d,), w["k_norm.weight"], 1e-6)
        return pm.causal_attention(q, k, F.linear(x, w["v_proj.weight"]).view(12, hkv, d), d ** -0.5)

    other = norm_after_rotation(0)
    assert float((other - norm_after_rotation(37)).abs().max()) > 1e-3 * float(other.abs().max())
    pos0, pos37 = torch.arange(12), torch.arange(12) + 37
    a0, _ = pm.self_attention(x, pos0, w, cfg)
    a37, _ = pm.self_attention(x, pos37, w, cfg)
    assert float((a0 - a37).abs().max()) <= 2e-4 * float(a0.abs().max())


def test_model_head_is_tied_or_not():
    cfg, tensors = oracle_weights("A")
    assert cfg["tie_word_embeddings"] and "lm_head.weight" not in tensors
    cfg_b, tensors_b = oracle_weights("B")
    assert not cfg_b["tie_word_embeddings"] and "lm_head.weight" in tensors_b
    ids = random_ids("B", 6, 1)
    a = pm.qwen3_logits(cfg_b, tensors_b, ids)
    swapped = dict(tensors_b)
    swapped["lm_head.weight"] = tensors_b["model.embed_tokens.weight"]
    assert not torch.allclose(pm.qwen3_logits(cfg_b, swapped, ids), a, atol=1e-3)


def test_model_window_layers_differ_from_full():
    cfg, tensors = oracle_weights("C")
    ids = random_ids("C", 80, 2)
    with_window = pm.qwen3_logits(cfg, tensors, ids)
    without = pm.qwen3_logits({**cfg, "use_sliding_window": False}, tensors, ids)
    w = cfg["sliding_window"]
    assert torch.allclose(with_window[:w], without[:w], atol=1e-9), "inside the window nothing changes"
    assert not torch.allclose(with_window[w:], without[w:], atol=1e-6)


# ------------------------------------------------------------------ sampling


def test_race_tends_to_argmax_and_follows_softmax():
    g = torch.Generator().manual_seed(0)
    logits = torch.tensor([[2.0, 1.0, 0.5, -1.0, 1.5]])
    noise = torch.empty(1, 5).exponential_(generator=g)
    assert int(pm.exponential_race(logits, torch.tensor([0.0]), noise)[0]) == 0
    assert int(pm.exponential_race(logits, torch.tensor([1e-6]), noise)[0]) == 0
    draws = 20000
    noise = torch.empty(draws, 5).exponential_(generator=g)
    picks = pm.exponential_race(logits.expand(draws, -1), torch.full((draws,), 0.7), noise)
    freq = torch.bincount(picks, minlength=5).double() / draws
    want = torch.softmax(logits[0].double() / 0.7, dim=-1)
    assert float((freq - want).abs().max()) < 4 * math.sqrt(0.25 / draws)


def test_top_k_top_p_filter():
    probs = torch.tensor([0.4, 0.3, 0.15, 0.1, 0.05], dtype=D64)
    assert torch.allclose(pm.top_k_top_p_filter(probs, 2, 1.0), torch.tensor([4 / 7, 3 / 7, 0, 0, 0], dtype=D64))
    # top_p 0.7: mass before each token is 0, .4, .7, .85, .95 -> the first three stay
    kept = pm.top_k_top_p_filter(probs, -1, 0.7)
    assert torch.allclose(kept, torch.tensor([0.4, 0.3, 0.15, 0, 0], dtype=D64) / 0.85)
    assert torch.allclose(pm.top_k_top_p_filter(probs, 1, 1.0), torch.tensor([1.0, 0, 0, 0, 0], dtype=D64))
    assert torch.allclose(pm.top_k_top_p_filter(probs, -1, 1e-9), torch.tensor([1.0, 0, 0, 0, 0], dtype=D64))
    shuffled = probs[[3, 0, 4, 2, 1]]
    assert torch.allclose(pm.top_k_top_p_filter(shuffled, 2, 1.0), torch.tensor([0, 4 / 7, 0, 0, 3 / 7], dtype=D64))
