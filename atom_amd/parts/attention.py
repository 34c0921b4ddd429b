"""Grouped-query attention over the paged cache.

The order of operations is atom/models/qwen3.py:146-162: one packed QKV product
(rows q | k | v, atom/model_ops/linear.py:1835-1848), RMS norm of every q and k
head over the head dimension (optional), rotation, the new keys and values written
to their pages, attention of the new queries over the pages, output projection.
Norm, rotation and the cache write are one kernel; the scale defaults to
``head_dim ** -0.5`` (qwen3.py:88).
"""

from __future__ import annotations

import numpy as np
import torch

from ..kernels.hip import AttentionMeta
from .base import MIXERS, POSITION_ENCODINGS, KVCacheNeed, Mixer, ParamSpec, PartChoice


class GroupedQueryAttention(Mixer):
    graph_safe = True
    accepts_deferred = True   # the input goes to the QKV product as it is

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 qkv_bias: bool = False, out_bias: bool = False, qk_norm: bool = False, norm_eps: float = 1e-6,
                 scale: float | None = None, window: int | None = None,
                 position_encoding: PartChoice | None = None, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qkv_bias = qkv_bias
        self.out_bias = out_bias
        self.qk_norm = qk_norm
        self.norm_eps = float(norm_eps)
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.window = window
        self.names = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj", "q_norm": "q_norm",
                      "k_norm": "k_norm", **(names or {})}
        self.rope = position_encoding.build(POSITION_ENCODINGS, head_dim=head_dim) if position_encoding else None

    def children(self):
        return [self.rope] if self.rope is not None else []

    def cache_need(self):
        return KVCacheNeed(self.num_kv_heads, self.head_dim, self.window)

    def param_specs(self):
        n = self.names
        q_rows, kv_rows = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        specs = {
            "qkv.weight": ParamSpec.stacked(
                [(f"{n['q']}.weight", q_rows), (f"{n['k']}.weight", kv_rows), (f"{n['v']}.weight", kv_rows)],
                (self.hidden_size,)),
            "o.weight": ParamSpec.single(f"{n['o']}.weight", (self.hidden_size, q_rows)),
        }
        if self.qkv_bias:
            specs["qkv.bias"] = ParamSpec.stacked(
                [(f"{n['q']}.bias", q_rows), (f"{n['k']}.bias", kv_rows), (f"{n['v']}.bias", kv_rows)], (),
                kind="vector")
        if self.out_bias:
            specs["o.bias"] = ParamSpec.single(f"{n['o']}.bias", (self.hidden_size,), kind="vector")
        if self.qk_norm:
            specs["q_norm.weight"] = ParamSpec.single(f"{n['q_norm']}.weight", (self.head_dim,), kind="vector",
                                                      init="one_plus_normal")
            specs["k_norm.weight"] = ParamSpec.single(f"{n['k_norm']}.weight", (self.head_dim,), kind="vector",
                                                      init="one_plus_normal")
        return specs

    # ---- what the attention kernels want to know about a step's batch

    def step_key(self):
        # the kernels' tile heights depend on the head size and on how many query heads share a KV head
        return ("attention", self.head_dim, self.num_heads // self.num_kv_heads)

    def _tile_rows(self, ops, dtype, page_size: int, max_q_len: int) -> tuple[int, int]:
        return ops.attention_tile_rows(dtype, self.head_dim, page_size, self.num_heads // self.num_kv_heads, max_q_len)

    def prepare_step(self, batch) -> dict:
        """Tiles of query rows of the prompt portions, as (request, first row) pairs, the tiles with the most
        keys first: one list for every tile height the kernels of this step use.  In a replayed step every
        list has the length the bucket can need at most; entries beyond the step's tiles name request -1."""
        if not batch.num_prefill:
            return {}
        out = {}
        portions = batch.portions()
        for page_size in set(batch.page_sizes):
            for rows in self._tile_rows(batch.ops, batch.dtype, page_size, batch.max_q_len):
                if rows and f"tiles{rows}" not in out:
                    tiles = [(b, r0) for b in portions for r0 in range(0, batch.q_lens[b], rows)]
                    tiles.sort(key=lambda t: -(batch.cached[t[0]] + t[1]))
                    if batch.replayed:
                        tiles += [(-1, 0)] * (batch.tile_capacity(rows) - len(tiles))
                    out[f"tiles{rows}"] = np.asarray(tiles, dtype=np.int32).reshape(-1, 2)
        return out

    def _meta(self, ctx, group: int) -> AttentionMeta:
        """The batch as the attention kernels take it, built once a step per group of layers."""
        key = ("attention meta", self.step_key(), group)
        meta = ctx.memo.get(key)
        if meta is None:
            page_size = ctx.page_sizes[group]
            arrays = ctx.prepared.get(self.step_key(), {})
            short, tall = self._tile_rows(ctx.ops, ctx.dtype, page_size, ctx.max_q_len) if ctx.num_prefill else (0, 0)
            meta = AttentionMeta(
                token_seq=ctx.token_seq, positions=ctx.positions, block_tables=ctx.block_tables[group],
                cu_seqlens_q=ctx.cu_seqlens_q, context_lens=ctx.context_lens, num_seqs=ctx.num_seqs,
                num_tokens=ctx.num_tokens, max_q_len=ctx.max_q_len, max_context_len=ctx.max_context_len,
                page_size=page_size, num_prefill=ctx.num_prefill,
                prefill_tiles=arrays.get(f"tiles{short}") if short else None, rows_per_tile=short or 16,
                tiles_by_rows={tall: arrays[f"tiles{tall}"]} if tall else None)
            ctx.memo[key] = meta
        return meta

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        tokens = x.shape[0]
        qkv = ops.linear(x, self.params["qkv.weight"], self.p("qkv.bias"), defer=True)
        meta = self._meta(ctx, cache.group)
        rope = self.rope
        out = torch.empty((tokens, self.num_heads, self.head_dim), dtype=x.dtype, device=x.device)
        fused = getattr(ops, "fused_decode_attention", None)
        done = None
        if fused is not None and rope is not None:
            # a decode step of few requests: one kernel from the QKV product to the attention output
            done = fused(qkv, cache.k_cache, cache.v_cache, out, meta, self.scale, self.window,
                         self.p("q_norm.weight"), self.p("k_norm.weight"), rope.cos, rope.sin,
                         ctx.slot_mappings[cache.group], self.num_heads, self.num_kv_heads, self.head_dim,
                         rope.rotary_dim, self.norm_eps, write_kv=cache.writes)
        if done is None:
            q = torch.empty((tokens, self.num_heads, self.head_dim), dtype=x.dtype, device=x.device)
            ops.qk_norm_rope_kv_write(
                qkv, q, cache.k_cache, cache.v_cache, self.p("q_norm.weight"), self.p("k_norm.weight"),
                rope.cos if rope else None, rope.sin if rope else None, ctx.positions,
                ctx.slot_mappings[cache.group], self.num_heads, self.num_kv_heads, self.head_dim,
                rope.rotary_dim if rope else 0, meta.page_size, self.norm_eps, write_kv=cache.writes)
            ops.paged_attention(q, cache.k_cache, cache.v_cache, out, meta, self.scale, self.window)
        return ops.linear(out.view(tokens, self.num_heads * self.head_dim), self.params["o.weight"], self.p("o.bias"),
                          defer=True)


MIXERS.register("attention", GroupedQueryAttention)
