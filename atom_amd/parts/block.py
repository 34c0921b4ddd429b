"""The pre-norm residual block: norm, mixer, norm, feed-forward, with the residual sum
folded into the norm that follows it (atom/models/qwen3.py:240-258): the block hands
on its feed-forward output and the residual stream, and the next norm adds them."""

from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, PartChoice


class PreNormBlock(Block):
    def __init__(self, mixer: PartChoice, feed_forward: PartChoice, norm: PartChoice, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        n = {"mixer_norm": "input_layernorm", "mixer": "self_attn", "ffn_norm": "post_attention_layernorm",
             "ffn": "mlp", **(names or {})}
        sub = lambda name: f"{prefix}.{n[name]}" if prefix else n[name]  # noqa: E731
        self.mixer_norm = norm.build(NORMS, prefix=sub("mixer_norm"))
        self._mixer = mixer.build(MIXERS, prefix=sub("mixer"))
        self.ffn_norm = norm.build(NORMS, prefix=sub("ffn_norm"))
        self.ffn = feed_forward.build(FEED_FORWARDS, prefix=sub("ffn"))

    @property
    def mixer(self):
        return self._mixer

    def children(self):
        return [self.mixer_norm, self._mixer, self.ffn_norm, self.ffn]

    def forward(self, ctx, hidden, residual, cache):
        if not self.mixer_norm.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden, residual = self.mixer_norm.forward_residual(ctx, hidden, residual)
        if not self._mixer.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden = self._mixer.forward(ctx, hidden, cache)
        if not self.ffn_norm.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden, residual = self.ffn_norm.forward_residual(ctx, hidden, residual)
        if not self.ffn.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden = self.ffn.forward(ctx, hidden)
        return hidden, residual


BLOCKS.register("prenorm", PreNormBlock)
