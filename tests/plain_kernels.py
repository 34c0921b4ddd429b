"""Plain PyTorch references of the engine's kernels, one per kernel, with the kernels'
signatures.  They serve two purposes: each GPU kernel is compared with its reference
alone, and on a machine without a GPU the references stand in for the kernel library so
that the engine's bookkeeping (paging, batching, the step function, the scheduler) can be
tested there.  They are test code: the engine itself has no such path.

Everything is computed in float64 and rounded once to the output's type.
"""

from __future__ import annotations

import torch

from plain_model import causal_attention, exponential_race, rms_norm, rope_neox, silu_and_mul, top_k_top_p_filter

WIDE = torch.float64


class PlainKernels:
    name = "plain"

    def embedding(self, table, ids, out):
        out.copy_(table[ids.long()].to(out.dtype))
        return out

    def feed_tokens(self, ids, source, sampled):
        take = source >= 0
        ids[take] = sampled[source[take].long()]
        return ids

    def rmsnorm(self, x, weight, eps, out, residual=None, mode="plain", rows=None):
        xs = x.to(WIDE)
        if rows is not None:
            xs = xs[rows.long()]
        if mode == "add":
            res = residual.to(WIDE)
            summed = xs + (res[rows.long()] if rows is not None else res)
        else:
            summed = xs
        if mode in ("init", "add") and rows is None:
            residual.copy_(summed.to(torch.float32))
            summed = residual.to(WIDE)  # the norm sees what the stream holds
        out.copy_(rms_norm(summed, weight.to(WIDE), eps).to(out.dtype))
        return out

    def silu_mul(self, x, out):
        out.copy_(silu_and_mul(x.to(WIDE)).to(out.dtype))
        return out

    def qk_norm_rope_kv_write(self, qkv, q_out, k_cache, v_cache, q_weight, k_weight, cos, sin, positions, slots,
                              num_heads, num_kv_heads, head_dim, rotary_dim, page_size, eps, write_kv=True):
        t = qkv.shape[0]
        q, k, v = torch.split(qkv.to(WIDE), [num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * head_dim], dim=-1)
        q = q.reshape(t, num_heads, head_dim)
        k = k.reshape(t, num_kv_heads, head_dim)
        v = v.reshape(t, num_kv_heads, head_dim)
        if q_weight is not None:
            q = rms_norm(q, q_weight.to(WIDE), eps)
        if k_weight is not None:
            k = rms_norm(k, k_weight.to(WIDE), eps)
        if rotary_dim:
            c = cos[positions.long()].to(WIDE)
            s = sin[positions.long()].to(WIDE)
            q = torch.cat((rope_neox(q[..., :rotary_dim], c, s), q[..., rotary_dim:]), dim=-1)
            k = torch.cat((rope_neox(k[..., :rotary_dim], c, s), k[..., rotary_dim:]), dim=-1)
        q_out.copy_(q.to(q_out.dtype))
        if write_kv:
            for i in range(t):
                slot = int(slots[i])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_cache[page, :, off, :] = k[i].to(k_cache.dtype)
                v_cache[page, :, :, off] = v[i].to(v_cache.dtype)
        return q_out

    def attention_tile_rows(self, dtype, head_dim, page_size, group, max_q_len):
        return 0, 0   # this attention walks tokens, it wants no tiles listed

    def paged_attention(self, q, k_cache, v_cache, out, meta, scale, window=None, parts=None):
        tokens, hq, d = q.shape
        page_size = k_cache.shape[2]
        for t in range(tokens):
            seq = int(meta.token_seq[t])
            if seq < 0:
                out[t] = 0
                continue
            pos = int(meta.positions[t])
            first = max(0, pos - window + 1) if window else 0
            keys = torch.arange(first, pos + 1)
            pages = meta.block_tables[seq].long()[keys // page_size]
            offs = keys % page_size
            k = k_cache[pages, :, offs, :].to(WIDE)        # [n, hkv, d]
            v = v_cache[pages, :, :, offs].to(WIDE)        # [n, hkv, d]
            o = causal_attention(q[t:t + 1].to(WIDE), k, v, scale, None, torch.tensor([pos]), keys)
            out[t] = o[0].to(out.dtype)
        return out

    def linear(self, x, weight, bias=None, out_dtype=None, defer=False):
        y = x.to(WIDE) @ weight.to(WIDE).T
        if bias is not None:
            y = y + bias.to(WIDE)
        return y.to(out_dtype or x.dtype)

    def linear_silu(self, x, weight, bias=None):
        return silu_and_mul(self.linear(x, weight, bias, out_dtype=WIDE)).to(x.dtype)

    def materialize(self, x):
        return x

    def exponential_noise(self, seeds, counters, vocab):
        rows = []
        for s, c in zip(seeds.tolist(), counters.tolist()):
            rows.append(exponential_noise_row(s, c, vocab))
        return torch.stack(rows)

    def sample(self, logits, temperatures, out, top_ks=None, top_ps=None, noise=None, seeds=None, counters=None,
               eps=1e-10):
        rows, vocab = logits.shape
        for r in range(rows):
            temp = float(temperatures[r]) if temperatures is not None else 0.0
            if not temp > 0:
                out[r] = int(logits[r].argmax())
                continue
            if noise is not None:
                e = noise[r if noise.shape[0] == rows and rows > 1 else 0]
            else:
                e = exponential_noise_row(int(seeds[r]), int(counters[r]), vocab)
            k = int(top_ks[r]) if top_ks is not None else -1
            p = float(top_ps[r]) if top_ps is not None else 1.0
            if (k > 0 and k < vocab) or p < 1.0:
                probs = torch.softmax(logits[r].to(WIDE) / temp, dim=-1)
                kept = top_k_top_p_filter(probs, k if 0 < k < vocab else -1, p)
                out[r] = int((kept / (e.to(WIDE) + eps)).argmax())
            else:
                out[r] = int(exponential_race(logits[r:r + 1], torch.tensor([temp]), e.unsqueeze(0), eps)[0])
        return out


_M64 = (1 << 64) - 1


def _mix64(x: int) -> int:
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _M64
    return x ^ (x >> 31)


def exponential_noise_row(seed: int, counter: int, vocab: int) -> torch.Tensor:
    """The engine's noise: Exp(1) draws from an integer mix of (seed, counter, token)."""
    import math

    base = _mix64((seed ^ ((counter * 0x9E3779B97F4A7C15) & _M64)) & _M64)
    out = []
    for v in range(vocab):
        z = _mix64((base + (v + 1) * 0xD6E8FEB86659FD93) & _M64)
        u = (float(z >> 40) + 0.5) / 16777216.0
        out.append(-math.log(u))
    return torch.tensor(out, dtype=torch.float32)
