"""Time mixing with a decay per key channel and a bonus for the current token (Peng et al., "Eagle and Finch: RWKV
with Matrix-Valued States and Dynamic Recurrence").

With x' the previous token's input (zeros before a request's first token), each of r, k, v, g, w reads its own mix
``x + (x' - x) * mu_s``.  ``r, k, v = W_r, W_k, W_v`` of their mixes (heads x dim), ``gate = silu(W_g mix_g)``,
the decay ``w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0))`` per head and key channel, and per head

    o = (S + diag(u) k v^T)^T r;        S <- diag(w) S + k v^T

Each head's o is divided by its root mean square, the heads together are weighted (``norm``, one weight per entry)
and gated, then projected out.  A request keeps one float32 row in its state slot: the previous token's input,
then S of every head.  The decay, its inner tanh and second product, the state and the norm are float32; the four
wide products leave their sums as float32.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, ParamSpec, StateNeed


class TimeMixRecurrence(Mixer):
    graph_safe = True

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float, decay_rank: int | None = None,
                 prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        self.hidden_size, self.num_heads, self.head_dim = hidden_size, num_heads, head_dim
        self.norm_eps = float(norm_eps)
        self.decay_rank = decay_rank      # the inner size of the decay's two products; None: the checkpoint's own
        self.names = {"r": "r", "k": "k", "v": "v", "gate": "g", "decay1": "w1", "decay2": "w2", "decay_bias": "w0",
                      "bonus": "u", "norm": "norm", "o": "o", "mu": "mu", **(names or {})}

    @property
    def inner(self) -> int:
        return self.num_heads * self.head_dim

    def cache_need(self):
        return StateNeed((self.hidden_size + self.num_heads * self.head_dim * self.head_dim,), torch.float32)

    def adopt_shapes(self, shape_of):
        if self.decay_rank is None:
            shape = shape_of(self.names["decay1"])
            if shape is not None and len(shape) == 2:
                self.decay_rank = int(shape[0])

    def param_specs(self):
        n, h, c = self.names, self.hidden_size, self.inner
        if self.decay_rank is None:
            raise ValueError("decay_rank is not known: name it, or load the model from a checkpoint whose tensors say it")
        return {
            **{f"mu.{s}": ParamSpec.single(f"{n['mu']}.{s}", (h,), kind="vector") for s in self.MIXES},
            # r, k, v and the gate as the four blocks of rows of one array: each multiplies a mix of its own, side by side
            "rkvg.weight": ParamSpec.stacked([(n["r"], c), (n["k"], c), (n["v"], c), (n["gate"], c)], (h,)),
            "decay1.weight": ParamSpec.single(n["decay1"], (self.decay_rank, h)),
            "decay2.weight": ParamSpec.single(n["decay2"], (c, self.decay_rank)),
            "decay.bias": ParamSpec.single(n["decay_bias"], (c,), kind="vector"),
            "bonus": ParamSpec.single(n["bonus"], (self.num_heads, self.head_dim), kind="vector"),
            "norm.weight": ParamSpec.single(n["norm"], (c,), kind="vector", init="one_plus_normal"),
            "o.weight": ParamSpec.single(n["o"], (h, c)),
        }

    def finalize(self, device, dtype):
        # the five mixing weights as rows of one array, in the order the kernel writes the mixes
        self.mu = torch.stack([self.params[f"mu.{s}"] for s in self.MIXES]).contiguous()

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T, W = x.shape
        H, K, c, rank = self.num_heads, self.head_dim, self.inner, self.decay_rank
        mixes = torch.empty((5, T, W), dtype=x.dtype, device=x.device)
        ops.token_shift(x, self.mu, mixes, cache.state, 0, ctx.cu_seqlens_q, ctx.slot_of_seq, ctx.token_seq)
        # each of r, k, v and the gate reads a mix of its own
        r, k, v, g = ops.linear_side_by_side(mixes[:4], self.params["rkvg.weight"].view(4, c, W), out_dtype=torch.float32)
        squashed = ops.linear_act(mixes[4], self.params["decay1.weight"], None, "tanh", out_dtype=torch.float32)
        raw = torch.empty((T, c), dtype=torch.float32, device=x.device)
        ops.heads_gemm(squashed, 0, rank, 0, self.params["decay2.weight"].view(1, c, rank), raw, 0, c, 0, 1, T, c, rank,
                       exact=True)
        o = torch.empty((T, c), dtype=torch.float32, device=x.device)
        ops.linear_scan(r, 0, H, k, 0, H, v, 0, raw, 0, cache.state, W, ctx.cu_seqlens_q, ctx.slot_of_seq, o, H, K, K,
                        per_channel=True, w_bias=self.params["decay.bias"], bonus=self.params["bonus"],
                        max_q_len=ctx.max_q_len)
        out = torch.empty((T, c), dtype=x.dtype, device=x.device)
        ops.group_norm_gate(o, H, self.params["norm.weight"], self.norm_eps, out, gate=g, gate_off=0, gate_first=False)
        return ops.linear(out, self.params["o.weight"], None, defer=True)


MIXERS.register("time_mix", TimeMixRecurrence)
