"""What a model does to its stream where a pass over a run of repeated layers begins.

``concat_projection``: ``x <- W [x ; x0]`` with x the residual stream, x0 the embedding's output and W
[width, 2 width] (x's columns first).  The stream's pending summand is added on the way in; the product's float32
result starts the stream anew.

``add_first``: ``x <- x + x0``.
"""

from __future__ import annotations

import torch

from .base import JOINS, Join, ParamSpec


class ConcatProjection(Join):
    def __init__(self, hidden_size: int, prefix: str = "", weight_name: str = "weight"):
        super().__init__(prefix)
        self.hidden_size = hidden_size
        self.weight_name = weight_name

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.hidden_size, 2 * self.hidden_size))}

    def forward(self, ctx, hidden, residual, first):
        ops = ctx.ops
        hidden = ops.materialize(hidden)
        both = torch.empty((hidden.shape[0], 2 * self.hidden_size), dtype=ctx.dtype, device=hidden.device)
        ops.sum_concat(hidden, residual, first, both)
        return ops.linear(both, self.params["weight"], None, out_dtype=torch.float32), None


class AddFirst(Join):
    """``x <- x + x0``: the embedding's output joins the stream again.  The stream's pending summand is added
    first; the embedding's output is handed on as the new pending summand, so the norm that follows adds it."""

    def __init__(self, hidden_size: int, prefix: str = ""):
        super().__init__(prefix)
        self.hidden_size = hidden_size

    def forward(self, ctx, hidden, residual, first):
        if residual is None:
            raise ValueError("the embedding's output can only be added to a stream that has begun")
        ctx.ops.stream_add(residual, hidden)
        return first, residual


JOINS.register("concat_projection", ConcatProjection)
JOINS.register("add_first", AddFirst)
