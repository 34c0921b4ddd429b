"""SiLU-gated dense feed-forward: ``down(silu(gate(x)) * up(x))`` with gate and up in
one packed product, gate rows first (atom/models/qwen3.py:166-198,321-322;
atom/model_ops/activation.py:78-82)."""

from __future__ import annotations

from .base import FEED_FORWARDS, FeedForward, ParamSpec


class GatedMLP(FeedForward):
    accepts_deferred = True   # the input goes to the gate/up product as it is

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", bias: bool = False,
                 prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        if activation != "silu":
            raise ValueError(f"the gated feed-forward has a SiLU kernel only, got {activation!r}")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.bias = bias
        self.names = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj", **(names or {})}

    def param_specs(self):
        n, i, h = self.names, self.intermediate_size, self.hidden_size
        specs = {
            "gate_up.weight": ParamSpec.stacked([(f"{n['gate']}.weight", i), (f"{n['up']}.weight", i)], (h,)),
            "down.weight": ParamSpec.single(f"{n['down']}.weight", (h, i)),
        }
        if self.bias:
            specs["gate_up.bias"] = ParamSpec.stacked([(f"{n['gate']}.bias", i), (f"{n['up']}.bias", i)], (),
                                                      kind="vector")
            specs["down.bias"] = ParamSpec.single(f"{n['down']}.bias", (h,), kind="vector")
        return specs

    def forward(self, ctx, x):
        ops = ctx.ops
        act = ops.linear_silu(x, self.params["gate_up.weight"], self.p("gate_up.bias"))
        # the down product may come back as slices that the next norm adds while it reads them
        return ops.linear(act, self.params["down.weight"], self.p("down.bias"), defer=True)


FEED_FORWARDS.register("gated_mlp", GatedMLP)
