"""Gated dense feed-forward: ``down(act(gate(x)) * up(x))`` with gate and up in one packed
product, gate rows first (atom/models/qwen3.py:166-198,321-322; atom/model_ops/activation.py:78-82).
SiLU runs the fused gate products; ReLU and tanh-GELU the plain product and an elementwise kernel."""

from __future__ import annotations

import torch

from .base import FEED_FORWARDS, FeedForward, ParamSpec


class GatedMLP(FeedForward):
    accepts_deferred = True   # the input goes to the gate/up product as it is

    ACTIVATIONS = ("silu", "relu", "gelu_tanh")

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", bias: bool = False,
                 prefix: str = "", names: dict[str, str] | None = None, weight_suffix: str = ".weight"):
        super().__init__(prefix)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"the gated feed-forward knows the activations {self.ACTIVATIONS}, got {activation!r}")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation
        self.bias = bias
        self.names = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj", **(names or {})}
        self.weight_suffix = weight_suffix   # what a checkpoint appends to a matrix's name ("" : nothing)

    def param_specs(self):
        n, i, h, sfx = self.names, self.intermediate_size, self.hidden_size, self.weight_suffix
        specs = {
            "gate_up.weight": ParamSpec.stacked([(f"{n['gate']}{sfx}", i), (f"{n['up']}{sfx}", i)], (h,)),
            "down.weight": ParamSpec.single(f"{n['down']}{sfx}", (h, i)),
        }
        if self.bias:
            specs["gate_up.bias"] = ParamSpec.stacked([(f"{n['gate']}.bias", i), (f"{n['up']}.bias", i)], (),
                                                      kind="vector")
            specs["down.bias"] = ParamSpec.single(f"{n['down']}.bias", (h,), kind="vector")
        return specs

    def forward(self, ctx, x):
        ops = ctx.ops
        if self.activation == "silu":
            act = ops.linear_silu(x, self.params["gate_up.weight"], self.p("gate_up.bias"))
        else:
            # the fused gate products are SiLU's; any other activation takes the product and one elementwise kernel
            both = ops.linear(x, self.params["gate_up.weight"], self.p("gate_up.bias"))
            act = torch.empty((both.shape[0], self.intermediate_size), dtype=both.dtype, device=both.device)
            ops.gated_act(both, act, self.activation)
        # the down product may come back as slices that the next norm adds while it reads them
        return ops.linear(act, self.params["down.weight"], self.p("down.bias"), defer=True)


class DenseMLP(FeedForward):
    """``down(act(up(x)))`` without a gate; ``activation`` one of silu, relu, gelu_tanh, relu_squared (the square
    of ReLU).  The activation is the up product's epilogue where its kernel offers one, else an elementwise kernel."""

    accepts_deferred = True   # the input goes to the up product as it is

    ACTIVATIONS = ("silu", "relu", "gelu_tanh", "relu_squared")

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu_squared", prefix: str = "",
                 names: dict[str, str] | None = None, weight_suffix: str = ""):
        super().__init__(prefix)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"the dense feed-forward knows the activations {self.ACTIVATIONS}, got {activation!r}")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.names = {"up": "up", "down": "down", **(names or {})}
        self.weight_suffix = weight_suffix

    def param_specs(self):
        n, i, h, sfx = self.names, self.intermediate_size, self.hidden_size, self.weight_suffix
        return {"up.weight": ParamSpec.single(f"{n['up']}{sfx}", (i, h)),
                "down.weight": ParamSpec.single(f"{n['down']}{sfx}", (h, i))}

    def forward(self, ctx, x):
        ops = ctx.ops
        act = ops.linear_act(x, self.params["up.weight"], None, self.activation)
        return ops.linear(act, self.params["down.weight"], None, defer=True)


FEED_FORWARDS.register("gated_mlp", GatedMLP)
FEED_FORWARDS.register("dense_mlp", DenseMLP)
