"""A selective state-space mixer (Dao and Gu, "Transformers are SSMs: Generalized Models and Efficient Algorithms
Through Structured State Space Duality").

One packed product gives ``z | x | B | C | dt`` (``inner = heads * vdim`` columns each for z and x, ``groups *
state`` each for B and C, ``heads`` for dt).  x, B and C together pass a short causal convolution per channel
(bias, SiLU).  With ``dt = softplus(dt + dt_bias)`` and per head h of group ``g = h // (heads / groups)``:

    S <- exp(-exp(A_log_h) dt) S + dt B_g x_h^T        (S: state x vdim)
    y_h = S^T C_g + D_h x_h

y times ``silu(z)`` is RMS-normed in ``norm_groups`` equal parts, weighted, and projected out.  A request keeps one
float32 row in its state slot: the convolution's last ``taps - 1`` inputs, then S of every head.  Step sizes,
decays, the state and the norm are float32; the packed product leaves its sums as float32.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, ParamSpec, StateNeed


class StateSpaceMixer(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state_size: int, groups: int,
                 conv_taps: int, norm_groups: int, norm_eps: float, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        if num_heads % groups:
            raise ValueError(f"{num_heads} heads are not a multiple of {groups} groups")
        if (num_heads * value_dim) % norm_groups:
            raise ValueError(f"{num_heads * value_dim} channels do not split into {norm_groups} equal parts")
        if conv_taps < 1:
            raise ValueError("the short convolution needs at least one tap")
        self.hidden_size, self.num_heads, self.value_dim = hidden_size, num_heads, value_dim
        self.state_size, self.groups, self.conv_taps, self.norm_groups = state_size, groups, conv_taps, norm_groups
        self.norm_eps = float(norm_eps)
        self.names = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log",
                      "D": "D", "norm": "norm", "o": "o", **(names or {})}

    @property
    def inner(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def channels(self) -> int:
        """Columns that pass the convolution: x | B | C."""
        return self.inner + 2 * self.groups * self.state_size

    @property
    def conv_floats(self) -> int:
        return (self.conv_taps - 1) * self.channels

    def cache_need(self):
        return StateNeed((self.conv_floats + self.num_heads * self.state_size * self.value_dim,), torch.float32)

    def param_specs(self):
        n, h = self.names, self.hidden_size
        return {
            "in.weight": ParamSpec.single(n["in"], (2 * self.inner + 2 * self.groups * self.state_size + self.num_heads, h)),
            "conv.weight": ParamSpec.single(n["conv"], (self.channels, self.conv_taps)),
            "conv.bias": ParamSpec.single(n["conv_bias"], (self.channels,), kind="vector"),
            "dt_bias": ParamSpec.single(n["dt_bias"], (self.num_heads,), kind="vector"),
            "A_log": ParamSpec.single(n["A_log"], (self.num_heads,), kind="vector"),
            "D": ParamSpec.single(n["D"], (self.num_heads,), kind="vector", init="one_plus_normal"),
            "norm.weight": ParamSpec.single(n["norm"], (self.inner,), kind="vector", init="one_plus_normal"),
            "o.weight": ParamSpec.single(n["o"], (h, self.inner)),
        }

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T = x.shape[0]
        H, V, N, G, inner, C = self.num_heads, self.value_dim, self.state_size, self.groups, self.inner, self.channels
        proj = ops.linear(x, self.params["in.weight"], None, out_dtype=torch.float32)     # z | x | B | C | dt
        xbc = torch.empty((T, C), dtype=torch.float32, device=x.device)
        ops.conv_silu_state(proj, C, self.params["conv.weight"], cache.state, ctx.cu_seqlens_q, ctx.slot_of_seq, xbc,
                            max_q_len=ctx.max_q_len, bias=self.params["conv.bias"], activation="silu", x_offset=inner)
        y = torch.empty((T, inner), dtype=torch.float32, device=x.device)
        # the raw step sizes are the product's last columns: the scan forms softplus(dt + dt_bias) and the decays
        ops.linear_scan(xbc, inner + G * N, G, xbc, inner, G, xbc, 0, proj, inner + C, cache.state, self.conv_floats,
                        ctx.cu_seqlens_q, ctx.slot_of_seq, y, H, N, V, per_channel=False, skip=self.params["D"],
                        max_q_len=ctx.max_q_len, step_bias=self.params["dt_bias"], a_log=self.params["A_log"])
        out = torch.empty((T, inner), dtype=x.dtype, device=x.device)
        ops.group_norm_gate(y, self.norm_groups, self.params["norm.weight"], self.norm_eps, out, gate=proj, gate_off=0,
                            gate_first=True)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("state_space", StateSpaceMixer)
