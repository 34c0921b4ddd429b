"""Token embedding and the language-model head (atom/model_ops/embed_head.py:138-178,
225-263).  The head may share the embedding's table (atom/models/qwen3.py:339-340);
it is applied only to the rows whose logits are asked for (embed_head.py:249-252)."""

from __future__ import annotations

import torch

from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamSpec


class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, prefix: str = ""):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size

    def param_specs(self):
        return {"weight": ParamSpec.single("weight", (self.vocab_size, self.hidden_size))}

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=ctx.dtype, device=ids.device)
        return ctx.ops.embedding(self.params["weight"], ids, out)


class LMHead(Head):
    """``logits = x @ W.T`` in float32 out.  ``tied_to`` names the embedding whose table it shares."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding | None = None, prefix: str = ""):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec.single("weight", (self.vocab_size, self.hidden_size))}

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.params["weight"] if self.tied_to is not None else self.params["weight"]

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        return ctx.ops.linear(x, self.weight, None, out_dtype=torch.float32)


EMBEDDINGS.register("token_embedding", TokenEmbedding)
HEADS.register("lm_head", LMHead)
