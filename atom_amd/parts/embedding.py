"""Token embedding and the language-model head (atom/model_ops/embed_head.py:138-178,
225-263).  The head may share the embedding's table (atom/models/qwen3.py:339-340);
it is applied only to the rows whose logits are asked for (embed_head.py:249-252)."""

from __future__ import annotations

import torch

from .base import EMBEDDINGS, HEADS, Embedding, Head, ParamSpec, StateNeed


class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, prefix: str = "", weight_name: str = "weight"):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.weight_name = weight_name   # the table's checkpoint name under the prefix (empty: the prefix itself)

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.vocab_size, self.hidden_size))}

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=ctx.dtype, device=ids.device)
        return ctx.ops.embedding(self.params["weight"], ids, out)


class ScaledEmbedding(TokenEmbedding):
    """``table[ids] * scale`` as float32 rows: the start of a float32 residual stream, not rounded to the
    serving type on the way."""

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, prefix: str = "",
                 weight_name: str = "weight"):
        super().__init__(vocab_size, hidden_size, prefix, weight_name)
        self.scale = float(scale)

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        return ctx.ops.embedding_scaled(self.params["weight"], ids, out, self.scale)


class PositionedEmbedding(TokenEmbedding):
    """``table[id] + rows[position]`` as float32 rows: a learned row per position (``max_positions`` of them,
    positions counted from 0 in each request) added to the token's row, unscaled."""

    def __init__(self, vocab_size: int, hidden_size: int, max_positions: int, prefix: str = "",
                 weight_name: str = "weight", position_name: str = "pos"):
        super().__init__(vocab_size, hidden_size, prefix, weight_name)
        if max_positions <= 0:
            raise ValueError("a learned position table needs at least one row")
        self.max_positions = int(max_positions)
        self.position_name = position_name

    def param_specs(self):
        return {**super().param_specs(),
                "positions": ParamSpec.single(self.position_name, (self.max_positions, self.hidden_size))}

    def forward(self, ctx, ids: torch.Tensor) -> torch.Tensor:
        out = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        return ctx.ops.embedding_positions(self.params["weight"], self.params["positions"], ids, ctx.positions, out)


class BigramEmbedding(TokenEmbedding):
    """``table[id] + pairs[(previous id * mul_prev + id * mul_cur) mod buckets]`` as float32 rows; a request's
    first token, which has no previous one, takes row ``buckets`` (the last) of ``pairs``.  The previous token of a
    request's next token is part of its state: an int32 per state slot that holds the last token + 1 (0, what a
    fresh slot holds: none yet), so that single tokens and portions cut anywhere find it, also in a replayed graph
    whose token ids exist on the device only."""

    def __init__(self, vocab_size: int, hidden_size: int, buckets: int, mul_prev: int, mul_cur: int, prefix: str = "",
                 weight_name: str = "weight", bigram_name: str = "bigram"):
        super().__init__(vocab_size, hidden_size, prefix, weight_name)
        if buckets <= 0:
            raise ValueError("the pair table needs at least one bucket")
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.bigram_name = bigram_name

    def param_specs(self):
        return {**super().param_specs(),
                "pairs": ParamSpec.single(self.bigram_name, (self.buckets + 1, self.hidden_size))}

    def cache_need(self):
        return StateNeed((1,), torch.int32)

    def forward(self, ctx, ids: torch.Tensor, cache=None) -> torch.Tensor:
        if cache is None:
            raise ValueError("the pair embedding needs its per-request state (the previous token)")
        out = torch.empty((ids.numel(), self.hidden_size), dtype=torch.float32, device=ids.device)
        return ctx.ops.embedding_bigram(self.params["weight"], self.params["pairs"], ids, cache.state,
                                        ctx.cu_seqlens_q, ctx.slot_of_seq, ctx.token_seq, out, self.buckets,
                                        self.mul_prev, self.mul_cur)


class LMHead(Head):
    """``logits = (x @ W.T) * scale`` in float32 out.  ``tied_to`` names the embedding whose table it shares."""

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding | None = None, prefix: str = "",
                 weight_name: str = "weight", scale: float = 1.0):
        super().__init__(prefix)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.tied_to = tied_to
        self.weight_name = weight_name
        self.scale = float(scale)     # the float32 logits are multiplied by it

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec.single(self.weight_name, (self.vocab_size, self.hidden_size))}

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.params["weight"] if self.tied_to is not None else self.params["weight"]

    def forward(self, ctx, x: torch.Tensor) -> torch.Tensor:
        logits = ctx.ops.linear(x, self.weight, None, out_dtype=torch.float32)
        return logits if self.scale == 1.0 else ctx.ops.scale_rows(logits, self.scale)


EMBEDDINGS.register("token_embedding", TokenEmbedding)
EMBEDDINGS.register("scaled_f32_embedding", ScaledEmbedding)
EMBEDDINGS.register("bigram_embedding", BigramEmbedding)
EMBEDDINGS.register("positioned_f32_embedding", PositionedEmbedding)
HEADS.register("lm_head", LMHead)
