"""The pre-norm residual block: norm, mixer, norm, feed-forward, with the residual sum
folded into the norm that follows it (atom/models/qwen3.py:240-258): the block hands
on its feed-forward output and the residual stream, and the next norm adds them."""

from __future__ import annotations

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, PartChoice, ScaledSum


class PreNormBlock(Block):
    def __init__(self, mixer: PartChoice, feed_forward: PartChoice | None, norm: PartChoice, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        n = {"mixer_norm": "input_layernorm", "mixer": "self_attn", "ffn_norm": "post_attention_layernorm",
             "ffn": "mlp", **(names or {})}
        sub = lambda name: f"{prefix}.{n[name]}" if prefix else n[name]  # noqa: E731
        self.mixer_norm = norm.build(NORMS, prefix=sub("mixer_norm"))
        self._mixer = mixer.build(MIXERS, prefix=sub("mixer"))
        # ``feed_forward`` None: the layer is its mixer alone, and hands on the mixer's output
        self.ffn = feed_forward.build(FEED_FORWARDS, prefix=sub("ffn")) if feed_forward is not None else None
        self.ffn_norm = norm.build(NORMS, prefix=sub("ffn_norm")) if self.ffn is not None else None

    @property
    def mixer(self):
        return self._mixer

    def children(self):
        return [self.mixer_norm, self._mixer] + ([self.ffn_norm, self.ffn] if self.ffn is not None else [])

    def forward(self, ctx, hidden, residual, cache):
        if not self.mixer_norm.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden, residual = self.mixer_norm.forward_residual(ctx, hidden, residual)
        if not self._mixer.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden = self._mixer.forward(ctx, hidden, cache)
        if self.ffn is None:
            return hidden, residual
        if not self.ffn_norm.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden, residual = self.ffn_norm.forward_residual(ctx, hidden, residual)
        if not self.ffn.accepts_deferred:
            hidden = ctx.ops.materialize(hidden)
        hidden = self.ffn.forward(ctx, hidden)
        return hidden, residual


class SandwichBlock(Block):
    """Norms before and after each sublayer: ``x += post1(mixer(pre1(x)))``, then ``x += post2(ffn(pre2(x)))``;
    ``feed_forward`` None leaves the second sublayer out.  As in the pre-norm block, the block hands on its last
    summand (float32, not yet added) beside the stream, and the norm that follows adds it.  The sum of the mixer's
    normed output and the norm before the feed-forward are one kernel where the norm offers ``forward_post``."""

    def __init__(self, mixer: PartChoice, feed_forward: PartChoice | None, norm: PartChoice, prefix: str = "",
                 names: dict[str, str] | None = None):
        super().__init__(prefix)
        n = {"mixer_pre": "norm1", "mixer": "mix", "mixer_post": "norm1b", "ffn_pre": "norm2", "ffn": "mlp",
             "ffn_post": "norm2b", **(names or {})}
        sub = lambda name: f"{prefix}.{n[name]}" if prefix else n[name]  # noqa: E731
        self.mixer_pre = norm.build(NORMS, prefix=sub("mixer_pre"))
        self._mixer = mixer.build(MIXERS, prefix=sub("mixer"))
        self.mixer_post = norm.build(NORMS, prefix=sub("mixer_post"))
        self.ffn = feed_forward.build(FEED_FORWARDS, prefix=sub("ffn")) if feed_forward is not None else None
        self.ffn_pre = norm.build(NORMS, prefix=sub("ffn_pre")) if self.ffn is not None else None
        self.ffn_post = norm.build(NORMS, prefix=sub("ffn_post")) if self.ffn is not None else None

    @property
    def mixer(self):
        return self._mixer

    def children(self):
        parts = [self.mixer_pre, self._mixer, self.mixer_post]
        if self.ffn is not None:
            parts += [self.ffn_pre, self.ffn, self.ffn_post]
        return parts

    def forward(self, ctx, hidden, residual, cache):
        ops = ctx.ops
        if not self.mixer_pre.accepts_deferred:
            hidden = ops.materialize(hidden)
        hidden, residual = self.mixer_pre.forward_residual(ctx, hidden, residual)
        if not self._mixer.accepts_deferred:
            hidden = ops.materialize(hidden)
        mixed = ops.materialize(self._mixer.forward(ctx, hidden, cache))
        if self.ffn is None:
            return self.mixer_post.forward(ctx, mixed, out_dtype=torch.float32), residual
        post = getattr(self.mixer_post, "forward_post", None)
        if post is not None:
            hidden = post(ctx, mixed, residual, self.ffn_pre)
        else:
            hidden, residual = self.ffn_pre.forward_residual(ctx, self.mixer_post.forward(ctx, mixed), residual)
        if not self.ffn.accepts_deferred:
            hidden = ops.materialize(hidden)
        out = ops.materialize(self.ffn.forward(ctx, hidden))
        return self.ffn_post.forward(ctx, out, out_dtype=torch.float32), residual


class PostNormBlock(Block):
    """Norms on the sublayers' outputs only: ``x += norm1(mixer(x))``, then ``x += norm2(ffn(x))``
    (``feed_forward`` None leaves it out), then, where the layer has one, a ``side`` part (kind from the
    FEED_FORWARDS registry) that is handed the stream and adds to it itself.  The sublayers read the stream, which
    is float32; the block keeps it whole (nothing pending) and hands it on as ``hidden`` with no residual.  A
    copy of the stream in the step's type, for the products that read it, comes out of the kernel that adds to
    it."""

    def __init__(self, mixer: PartChoice, feed_forward: PartChoice | None, norm: PartChoice,
                 side: PartChoice | None = None, prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        n = {"mixer": "mix", "mixer_post": "norm1", "ffn": "mlp", "ffn_post": "norm2", "side": "side", **(names or {})}
        sub = lambda name: f"{prefix}.{n[name]}" if prefix else n[name]  # noqa: E731
        self._mixer = mixer.build(MIXERS, prefix=sub("mixer"))
        self.mixer_post = norm.build(NORMS, prefix=sub("mixer_post"))
        self.ffn = feed_forward.build(FEED_FORWARDS, prefix=sub("ffn")) if feed_forward is not None else None
        self.ffn_post = norm.build(NORMS, prefix=sub("ffn_post")) if self.ffn is not None else None
        self.side = side.build(FEED_FORWARDS, prefix=sub("side")) if side is not None else None
        for post in (self.mixer_post, self.ffn_post):
            if post is not None and not hasattr(post, "forward_post"):
                raise ValueError(f"{type(post).__name__} cannot add its output to the stream (no forward_post)")

    @property
    def mixer(self):
        return self._mixer

    def children(self):
        parts = [self._mixer, self.mixer_post]
        if self.ffn is not None:
            parts += [self.ffn, self.ffn_post]
        if self.side is not None:
            parts.append(self.side)
        return parts

    def forward(self, ctx, hidden, residual, cache):
        ops = ctx.ops
        if residual is not None:
            raise ValueError("this block takes the whole stream, with nothing pending beside it")
        stream = ops.materialize(hidden)
        if stream.dtype != torch.float32:
            raise ValueError("this block keeps a float32 stream: the embedding before it must write float32")
        # the stream in the step's type, as the products read it: left by the block before this one, or made now
        reads = ctx.memo.pop(("stream copy", stream.data_ptr()), None)
        if reads is None:
            reads = stream if ctx.dtype == torch.float32 else ops.cast_rows(stream, ctx.dtype)
        mixed = ops.materialize(self._mixer.forward(ctx, reads, cache))
        reads = self.mixer_post.forward_post(ctx, mixed, stream)
        if self.ffn is not None:
            out = ops.materialize(self.ffn.forward(ctx, reads))
            reads = self.ffn_post.forward_post(ctx, out, stream)
        if self.side is not None:
            reads = self.side.forward_stream(ctx, reads, stream)
        ctx.memo[("stream copy", stream.data_ptr())] = reads
        return stream, None


class NormedSumBlock(Block):
    """The norm comes after the sum and its result is the stream: ``x <- norm1(alpha x + mixer(x))``, then
    ``x <- norm2(alpha x + ffn(x))`` (``feed_forward`` None leaves the second step out).  The sublayers read the
    stream, which is float32 and kept whole (nothing pending); its rows in the step's type, for the products that
    read them, come out of the kernel that norms it.  A mixer with ``reads_stream`` is handed the float32 rows.
    ``names["mixer"]`` may be empty: the mixer then takes the layer's own prefix.  A checkpoint that holds the second
    norm's weight for a layer without feed-forward gets the second step with nothing added: ``x <- norm2(alpha x)``."""

    def __init__(self, mixer: PartChoice, feed_forward: PartChoice | None, norm: PartChoice, alpha: float = 1.0,
                 prefix: str = "", names: dict[str, str] | None = None):
        super().__init__(prefix)
        n = {"mixer": "mix", "mixer_norm": "norm1", "ffn": "mlp", "ffn_norm": "norm2", **(names or {})}
        sub = lambda name: (f"{prefix}.{n[name]}" if prefix else n[name]) if n[name] else prefix  # noqa: E731
        self._norm_choice, self._ffn_norm_prefix, self._ffn_norm_name = norm, sub("ffn_norm"), n["ffn_norm"]
        self.alpha = float(alpha)
        self._mixer = mixer.build(MIXERS, prefix=sub("mixer"))
        self.mixer_norm = norm.build(NORMS, prefix=sub("mixer_norm"))
        self.ffn = feed_forward.build(FEED_FORWARDS, prefix=sub("ffn")) if feed_forward is not None else None
        self.ffn_norm = norm.build(NORMS, prefix=sub("ffn_norm")) if self.ffn is not None else None
        for post in (self.mixer_norm, self.ffn_norm):
            if post is not None and not hasattr(post, "forward_sum"):
                raise ValueError(f"{type(post).__name__} cannot norm a sum into the stream (no forward_sum)")

    @property
    def mixer(self):
        return self._mixer

    def children(self):
        return ([self._mixer, self.mixer_norm] + ([self.ffn] if self.ffn is not None else [])
                + ([self.ffn_norm] if self.ffn_norm is not None else []))

    def adopt_shapes(self, shape_of):
        named = shape_of(self._ffn_norm_name) is not None or shape_of(f"{self._ffn_norm_name}.weight") is not None
        if self.ffn is None and self.ffn_norm is None and named:
            self.ffn_norm = self._norm_choice.build(NORMS, prefix=self._ffn_norm_prefix)

    @staticmethod
    def _summands(ops, y):
        if isinstance(y, ScaledSum):
            return [ops.materialize(t) for t in y.terms], y.scales
        return [ops.materialize(y)], [1.0]

    def forward(self, ctx, hidden, residual, cache):
        ops = ctx.ops
        if residual is not None:
            raise ValueError("this block takes the whole stream, with nothing pending beside it")
        stream = ops.materialize(hidden)
        if stream.dtype != torch.float32:
            raise ValueError("this block keeps a float32 stream: the embedding before it must write float32")
        reads = ctx.memo.pop(("stream copy", stream.data_ptr()), None)
        if self._mixer.reads_stream:
            reads = stream
        elif reads is None:
            reads = stream if ctx.dtype == torch.float32 else ops.cast_rows(stream, ctx.dtype)
        terms, scales = self._summands(ops, self._mixer.forward(ctx, reads, cache))
        # the copy is for the feed-forward, or for the next block's mixer where that reads one
        reads = self.mixer_norm.forward_sum(ctx, terms, scales, stream, self.alpha,
                                            copy=self.ffn is not None or not self._mixer.reads_stream)
        if self.ffn is not None:
            terms, scales = self._summands(ops, self.ffn.forward(ctx, reads))
            reads = self.ffn_norm.forward_sum(ctx, terms, scales, stream, self.alpha, copy=not self._mixer.reads_stream)
        elif self.ffn_norm is not None:
            reads = self.ffn_norm.forward_sum(ctx, [], [], stream, self.alpha, copy=not self._mixer.reads_stream)
        if reads is not stream:
            ctx.memo[("stream copy", stream.data_ptr())] = reads
        return stream, None


BLOCKS.register("prenorm", PreNormBlock)
BLOCKS.register("normed_sum", NormedSumBlock)
BLOCKS.register("sandwich", SandwichBlock)
BLOCKS.register("postnorm", PostNormBlock)
