"""Grouped-query attention without rotation, whose values have a size of their own.

``q = W_q x``, ``k = W_k x`` (heads of ``head_dim``), ``v = W_v x`` (heads of ``value_dim``), no biases.
Options: ``unit_norm`` (every q and k head is divided by its root mean square, no weight), ``temperature`` =
(coef, every): the query at position p is multiplied by ``1 + coef ln(floor((p + 1) / every) + 1)``, ``window``
(a query sees itself and the ``window - 1`` tokens before it).  ``score = (q . k) * scale``, ordinary softmax.

The pages and the attention kernels have one head size for keys and values, so both are laid out with
``padded_dim`` entries, the smallest size the matrix-core kernels take that holds both (or the larger of the two
where there is none): the extra entries are zeros and change neither a score nor a weighted sum.  One kernel
norms, scales and writes q, k and v from the float32 packed product.
"""

from __future__ import annotations

import torch

from .attention import GroupedQueryAttention
from .base import MIXERS, KVCacheNeed, ParamSpec

# head sizes the matrix-core attention kernels are built for
_KERNEL_HEAD_SIZES = (16, 32, 64, 96, 128, 256)


class PlainAttention(GroupedQueryAttention):
    graph_safe = True
    accepts_deferred = False

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, unit_norm: bool = False, temperature: tuple | None = None, window: int | None = None,
                 norm_eps: float = 1e-6, prefix: str = "", names: dict[str, str] | None = None):
        need = max(head_dim, value_dim)
        self.padded_dim = next((s for s in _KERNEL_HEAD_SIZES if s >= need), need)
        self.key_dim, self.value_dim = head_dim, value_dim
        super().__init__(hidden_size, num_heads, num_kv_heads, self.padded_dim, norm_eps=norm_eps, scale=scale,
                         window=window, position_encoding=None, prefix=prefix)
        self.unit_norm = bool(unit_norm)
        if temperature is not None and int(temperature[1]) <= 0:
            raise ValueError("the query temperature's step must be positive")
        self.temperature = (float(temperature[0]), int(temperature[1])) if temperature is not None else None
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", **(names or {})}

    def cache_need(self):
        return KVCacheNeed(self.num_kv_heads, self.padded_dim, self.window)

    def param_specs(self):
        n = self.names
        q_rows, k_rows, v_rows = (self.num_heads * self.key_dim, self.num_kv_heads * self.key_dim,
                                  self.num_kv_heads * self.value_dim)
        return {"qkv.weight": ParamSpec.stacked([(n["q"], q_rows), (n["k"], k_rows), (n["v"], v_rows)], (self.hidden_size,)),
                "o.weight": ParamSpec.single(n["o"], (self.hidden_size, self.num_heads * self.value_dim))}

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        tokens = x.shape[0]
        H, G, DP = self.num_heads, self.num_kv_heads, self.padded_dim
        proj = ops.linear(x, self.params["qkv.weight"], None, out_dtype=torch.float32)
        meta = self._meta(ctx, cache.group)
        q = torch.empty((tokens, H, DP), dtype=x.dtype, device=x.device)
        ops.qkv_plain_write(proj, q, cache.k_cache, cache.v_cache, ctx.positions, ctx.slot_mappings[cache.group], H, G,
                            self.key_dim, self.value_dim, meta.page_size, self.unit_norm, self.norm_eps,
                            temperature=self.temperature, write_kv=cache.writes)
        out = torch.empty((tokens, H, DP), dtype=x.dtype, device=x.device)
        ops.paged_attention(q, cache.k_cache, cache.v_cache, out, meta, self.scale, self.window)
        return ops.linear(ops.narrow_heads(out, self.value_dim), self.params["o.weight"], None, defer=True)


MIXERS.register("plain_attention", PlainAttention)
