"""Mixers side by side: every branch reads the same input, each keeps memory of its own, and the result is the mean
of the branches' outputs, each first RMS-normed over the model width with a weight of its own
(``<branch>.out`` under the mixer's prefix), or, with ``combine="weighted_sum"``, ``sum_b scales[b] * branch_b``
(no weights of its own; handed on as a ``ScaledSum``).

What the branches keep between steps is bound together: a ``JointNeed`` lists the branches' needs, and its cache
kind allocates, shares and clears each with the kind the need itself names.  At most one branch may keep pages; its
window and chunk decide the group of layers the mixer shares block tables with.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import MIXERS, Mixer, ParamSpec, PartChoice, ScaledSum


@dataclass(frozen=True)
class JointNeed:
    """The needs of several mixers that run side by side in one layer (None for a branch that keeps nothing)."""

    needs: tuple


class ParallelMixer(Mixer):
    def __init__(self, hidden_size: int, branches: list[tuple[str, PartChoice]], norm_eps: float, prefix: str = "",
                 out_name: str = "out", combine: str = "mean_of_norms", scales: list | None = None):
        super().__init__(prefix)
        if not 1 <= len(branches) <= 4:
            raise ValueError("one to four mixers can run side by side")
        if combine not in ("mean_of_norms", "weighted_sum"):
            raise ValueError(f"branches are joined by 'mean_of_norms' or 'weighted_sum', got {combine!r}")
        if combine == "weighted_sum" and (scales is None or len(scales) != len(branches)):
            raise ValueError("a weighted sum needs one scale per branch")
        self.combine, self.scales = combine, [float(s) for s in scales] if scales is not None else None
        self.hidden_size, self.norm_eps, self.out_name = hidden_size, float(norm_eps), out_name
        self.branch_names = [name for name, _ in branches]
        self.branches = [choice.build(MIXERS, prefix=self.full_name(name)) for name, choice in branches]
        self.graph_safe = all(b.graph_safe for b in self.branches)

    def children(self):
        return list(self.branches)

    def cache_need(self):
        return JointNeed(tuple(b.cache_need() for b in self.branches))

    def page_size_problem(self, page_size):
        for b in self.branches:
            problem = b.page_size_problem(page_size)
            if problem:
                return problem
        return None

    def step_key(self):
        keys = tuple(b.step_key() for b in self.branches)
        return ("side by side", keys) if any(k is not None for k in keys) else None

    def prepare_step(self, batch):
        # every branch's arrays under its own step key, as the branch will look them up
        out = {}
        for i, b in enumerate(self.branches):
            if b.step_key() is not None:
                for name, array in b.prepare_step(batch).items():
                    out[f"{i}:{name}"] = array
        return out

    def param_specs(self):
        if self.combine == "weighted_sum":
            return {}
        return {f"{name}.out": ParamSpec.single(f"{name}.{self.out_name}", (self.hidden_size,), kind="vector",
                                                init="one_plus_normal") for name in self.branch_names}

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        mine = ctx.prepared.get(self.step_key(), {}) if self.step_key() is not None else {}
        outs = []
        for i, (b, binding) in enumerate(zip(self.branches, cache.parts)):
            key = b.step_key()
            if key is not None and key not in ctx.prepared:
                ctx.prepared[key] = {name.split(":", 1)[1]: t for name, t in mine.items() if name.startswith(f"{i}:")}
            outs.append(ops.materialize(b.forward(ctx, x, binding)))
        if self.combine == "weighted_sum":
            return ScaledSum(outs, self.scales)
        out = torch.empty((x.shape[0], self.hidden_size), dtype=x.dtype, device=x.device)
        return ops.mean_of_norms(outs, [self.params[f"{name}.out"] for name in self.branch_names], self.norm_eps, out)


MIXERS.register("parallel", ParallelMixer)
