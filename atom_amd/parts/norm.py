"""RMS norm: ``x * rsqrt(mean(x^2) + eps) * w`` in float32, with the residual stream
(float32) added first when asked.  atom/model_ops/layernorm.py:57-75,450-460."""

from __future__ import annotations

import torch

from .base import NORMS, Norm, ParamSpec


class RMSNorm(Norm):
    accepts_deferred = True   # the kernel adds the slices of a product that is still a sum

    def __init__(self, size: int, eps: float, prefix: str = ""):
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)

    def param_specs(self):
        return {"weight": ParamSpec.single("weight", (self.size,), kind="vector", init="one_plus_normal")}

    def forward(self, ctx, x):
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        return ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out)

    def forward_residual(self, ctx, x, residual):
        pending = getattr(ctx.ops, "pending_norm", None)
        if pending is not None and residual is not None:
            # a product that has not been launched takes the residual sum as its epilogue and leaves the norm
            # to the product that follows
            lazy = pending(x, residual, self.params["weight"], self.eps)
            if lazy is not None:
                return lazy, residual
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        if residual is None:
            residual = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
            ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode="init")
        else:
            ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode="add")
        return out, residual

    def forward_rows(self, ctx, x, residual, rows):
        pending = getattr(ctx.ops, "pending_norm", None)
        if pending is not None and residual is not None:
            lazy = pending(x, residual, self.params["weight"], self.eps, rows)
            if lazy is not None:
                return lazy
        out = torch.empty((rows.numel(), self.size), dtype=x.dtype, device=x.device)
        mode = "add" if residual is not None else "plain"
        return ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode=mode, rows=rows)


NORMS.register("rmsnorm", RMSNorm)
