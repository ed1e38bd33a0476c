"""Softmax attention whose heads are worked through together, with the options that need it or come with it:

    ``qkv_bias`` / ``out_bias``   biases of the projections (``<name>.b``)
    ``conv_taps``                 a short causal convolution over time on every channel of q, k and v right after
                                  the projection (``<name>.conv`` [channels, taps], last column the current token's;
                                  the last ``taps - 1`` projected rows are carried per request)
    ``qk_norm``                   RMS norm of every q and k head with a weight per entry shared by the heads
    ``position_encoding``         rotation of q and k (a part that offers ``freq`` and ``dims``: pairs (i, i + dims / 2))
    ``head_temperature``          a learned factor per head on the scaled scores (``temp``)
    ``sink``                      a learned number per head whose exponential joins the softmax's denominator, with
                                  no key and no value (``sink``)
    ``talk``                      after the softmax the heads' weights are mixed, ``w_h <- sum_g T[h, g] w_g``
                                  (``talk`` [heads, heads]); head h applies its mixed weights to the values of its own
                                  key/value head
    ``value_mix``                 "source": this layer's values are kept for the step; "blend": ``v <- (1 - l) v +
                                  l v_source`` with ``l`` a learned number (``vmix``) and v_source the source layer's
                                  values of the same token; the blended values are what the pages hold
    ``value_dim``                 value heads of another size than key heads: the value pages are laid out for it

``score = (q . k) * scale``.  Keys live in pages [pages, G, page, dim], values in pages [pages, G, vdim, page].  The
projection's sums stay float32 through convolution, norm and rotation; q and the pages take the step's type.

Without head mixing and temperature, and with values of the keys' size, nothing needs the heads together: the step
then runs the paged attention kernels of ``GroupedQueryAttention`` (one walk over the keys; the sink is where a row's
running maximum and sum start) where they take the sizes, and this mixer prepares their tiles of query rows.
"""

from __future__ import annotations

import torch

from .attention import GroupedQueryAttention
from .base import MIXERS, POSITION_ENCODINGS, KVCacheNeed, Mixer, ParamSpec, PartChoice, StateNeed
from .parallel import JointNeed


class TogetherAttention(GroupedQueryAttention):
    """Shares with ``GroupedQueryAttention`` only what the paged kernels want to know about a step (``step_key``,
    ``prepare_step``, the batch record); parameters, memory and the forward pass are its own."""

    graph_safe = True
    accepts_deferred = False

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                 value_dim: int | None = None, norm_eps: float = 1e-6, qkv_bias: bool = False, out_bias: bool = False,
                 conv_taps: int | None = None, qk_norm: bool = False, position_encoding: PartChoice | None = None,
                 head_temperature: bool = False, sink: bool = False, talk: bool = False,
                 value_mix: str | None = None, window: int | None = None, prefix: str = "",
                 names: dict[str, str] | None = None):
        Mixer.__init__(self, prefix)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        if value_mix not in (None, "source", "blend"):
            raise ValueError(f"value_mix is None, 'source' or 'blend', got {value_mix!r}")
        if conv_taps is not None and conv_taps < 1:
            raise ValueError("the short convolution needs at least one tap")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim = head_dim, value_dim if value_dim is not None else head_dim
        self.scale, self.norm_eps, self.window = float(scale), float(norm_eps), window
        self.qkv_bias, self.out_bias, self.qk_norm = bool(qkv_bias), bool(out_bias), bool(qk_norm)
        self.conv_taps = conv_taps
        self.head_temperature, self.sink, self.talk, self.value_mix = bool(head_temperature), bool(sink), bool(talk), value_mix
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "bias": "b", "conv": "conv", "norm": "norm",
                      "temp": "temp", "sink": "sink", "talk": "talk", "vmix": "vmix", **(names or {})}
        self.rope = position_encoding.build(POSITION_ENCODINGS, head_dim=head_dim) if position_encoding else None

    def children(self):
        return [self.rope] if self.rope is not None else []

    @property
    def one_walk(self) -> bool:
        """Whether nothing in this mixer needs a token's heads together."""
        return not self.talk and not self.head_temperature and self.value_dim == self.head_dim

    def step_key(self):
        return super().step_key() if self.one_walk else None

    def prepare_step(self, batch):
        return super().prepare_step(batch) if self.one_walk else {}

    @property
    def channels(self) -> int:
        return (self.num_heads + self.num_kv_heads) * self.head_dim + self.num_kv_heads * self.value_dim

    def cache_need(self):
        pages = KVCacheNeed(self.num_kv_heads, self.head_dim, self.window, None,
                            self.value_dim if self.value_dim != self.head_dim else None)
        if not self.conv_taps:
            return pages
        # one tap carries nothing; its row of one number keeps the convolution's kernel one for all tap counts
        return JointNeed((pages, StateNeed((max(1, (self.conv_taps - 1) * self.channels),), torch.float32)))

    def param_specs(self):
        n, h = self.names, self.hidden_size
        rows = [("q", self.num_heads * self.head_dim), ("k", self.num_kv_heads * self.head_dim),
                ("v", self.num_kv_heads * self.value_dim)]
        specs = {"qkv.weight": ParamSpec.stacked([(n[r], c) for r, c in rows], (h,)),
                 "o.weight": ParamSpec.single(n["o"], (h, self.num_heads * self.value_dim))}
        if self.qkv_bias:
            specs["qkv.bias"] = ParamSpec.stacked([(f"{n[r]}.{n['bias']}", c) for r, c in rows], (), kind="vector")
        if self.out_bias:
            specs["o.bias"] = ParamSpec.single(f"{n['o']}.{n['bias']}", (h,), kind="vector")
        if self.conv_taps:
            specs["conv.weight"] = ParamSpec.stacked([(f"{n[r]}.{n['conv']}", c) for r, c in rows], (self.conv_taps,))
        if self.qk_norm:
            for r in ("q", "k"):
                specs[f"{r}_norm.weight"] = ParamSpec.single(f"{n[r]}.{n['norm']}", (self.head_dim,), kind="vector",
                                                             init="one_plus_normal")
        if self.head_temperature:
            specs["temp"] = ParamSpec.single(n["temp"], (self.num_heads,), kind="vector", init="one_plus_normal")
        if self.sink:
            specs["sink"] = ParamSpec.single(n["sink"], (self.num_heads,), kind="vector")
        if self.talk:
            specs["talk"] = ParamSpec.single(n["talk"], (self.num_heads, self.num_heads), kind="vector")
        if self.value_mix is not None:
            specs["vmix"] = ParamSpec.scalar(n["vmix"])     # the source layer's is loaded and not used
        return specs

    def forward(self, ctx, x, cache):
        ops = ctx.ops
        T = x.shape[0]
        H, G, D, DV = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        pages, carried = (cache.parts if hasattr(cache, "parts") else (cache, None))
        if not pages.writes:
            raise ValueError("this attention writes its own pages; it cannot read another run's")
        proj = ops.linear(x, self.params["qkv.weight"], self.p("qkv.bias"), out_dtype=torch.float32)
        if carried is not None:
            qkv = torch.empty((T, self.channels), dtype=torch.float32, device=x.device)
            ops.conv_silu_state(proj, self.channels, self.params["conv.weight"], carried.state, ctx.cu_seqlens_q,
                                ctx.slot_of_seq, qkv, max_q_len=ctx.max_q_len, activation="none")
        else:
            qkv = proj
        source = keep = None
        if self.value_mix == "source":
            keep = ctx.memo["source values"] = torch.empty((T, G * DV), dtype=torch.float32, device=x.device)
        elif self.value_mix == "blend":
            source = ctx.memo.get("source values")
            if source is None or tuple(source.shape) != (T, G * DV):
                raise ValueError("values are blended with those of an earlier layer, and no layer has left any")
        q = torch.empty((T, H, D), dtype=ctx.dtype, device=x.device)
        group = pages.group
        rope = self.rope
        ops.qkv_rot_write(qkv, q, pages.k_cache, pages.v_cache, self.p("q_norm.weight"), self.p("k_norm.weight"),
                          rope.freq if rope is not None else None, rope.dims if rope is not None else 0, ctx.positions,
                          ctx.slot_mappings[group], H, G, D, DV, ctx.page_sizes[group], self.norm_eps,
                          v_source=source, v_blend=self.p("vmix") if source is not None else None, v_keep=keep)
        out = torch.empty((T, H, DV), dtype=ctx.dtype, device=x.device)
        takes = getattr(ops, "takes_sink", None)
        if self.one_walk and takes is not None and takes(ctx.dtype, D, DV, ctx.page_sizes[group], H // G):
            ops.paged_attention(q, pages.k_cache, pages.v_cache, out, self._meta(ctx, group), self.scale, self.window,
                                sink=self.p("sink"))
            return ops.linear(out.view(T, H * DV), self.params["o.weight"], self.p("o.bias"), out_dtype=torch.float32)
        ops.attention_together(q, pages.k_cache, pages.v_cache, out, ctx.token_seq, ctx.positions,
                               ctx.block_tables[group], self.scale, head_scale=self.p("temp"), sink=self.p("sink"),
                               talk=self.p("talk"), window=self.window, max_context_len=ctx.max_context_len,
                               cu_seqlens_q=ctx.cu_seqlens_q, max_q_len=ctx.max_q_len)
        return ops.linear(out.view(T, H * DV), self.params["o.weight"], self.p("o.bias"), out_dtype=torch.float32)


MIXERS.register("together_attention", TogetherAttention)
