"""Token shift around a mixer: what the mixer reads is ``h + (h' - h) * mu`` with h' the previous token's row as it
was before the blend (zeros before a request's first token) and ``mu`` a weight per entry.  The previous row is
part of a request's memory: one float32 row per state slot, bound together with whatever the wrapped mixer keeps.

The weight's checkpoint name is ``<prefix>.<weight_name>`` and the wrapped mixer lives under
``<prefix>.<inner_name>``, so a block gives this mixer the layer's own prefix.
"""

from __future__ import annotations

import torch

from .base import MIXERS, Mixer, ParamSpec, PartChoice, StateNeed
from .parallel import JointNeed


class ShiftedMixer(Mixer):
    reads_stream = True     # the blend is formed from the float32 rows where there are any

    def __init__(self, hidden_size: int, inner: PartChoice, prefix: str = "", inner_name: str = "mix",
                 weight_name: str = "shift"):
        super().__init__(prefix)
        self.hidden_size, self.weight_name = hidden_size, weight_name
        self.inner = inner.build(MIXERS, prefix=self.full_name(inner_name))
        self.graph_safe = self.inner.graph_safe

    def children(self):
        return [self.inner]

    def param_specs(self):
        return {"mu": ParamSpec.single(self.weight_name, (self.hidden_size,), kind="vector")}

    def cache_need(self):
        return JointNeed((StateNeed((self.hidden_size,), torch.float32), self.inner.cache_need()))

    def page_size_problem(self, page_size):
        return self.inner.page_size_problem(page_size)

    def step_key(self):
        return self.inner.step_key()

    def prepare_step(self, batch):
        return self.inner.prepare_step(batch)

    def forward(self, ctx, x, cache):
        blended = torch.empty(tuple(x.shape), dtype=ctx.dtype, device=x.device)
        ctx.ops.shift_rows(x, self.params["mu"], blended, cache.parts[0].state, 0, ctx.cu_seqlens_q, ctx.slot_of_seq,
                           ctx.token_seq)
        return self.inner.forward(ctx, blended, cache.parts[1])


MIXERS.register("token_shifted", ShiftedMixer)
