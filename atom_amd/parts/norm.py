"""RMS norm: ``x * rsqrt(mean(x^2) + eps) * w`` in float32, with the residual stream
(float32) added first when asked.  atom/model_ops/layernorm.py:57-75,450-460.
Layer norm (mean taken off, weight and bias) with the same three entry points, and a fourth that
sums a normed sublayer output into the stream and norms the stream for the next sublayer."""

from __future__ import annotations

import torch

from .base import NORMS, Norm, ParamSpec


class RMSNorm(Norm):
    accepts_deferred = True   # the kernel adds the slices of a product that is still a sum

    def __init__(self, size: int, eps: float, prefix: str = "", weight_name: str = "weight", one_plus: bool = False):
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)
        self.weight_name = weight_name   # the checkpoint's name under the prefix (empty: the prefix itself)
        self.one_plus = bool(one_plus)   # the checkpoint stores the weight's distance from one
        self._folded = False

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.size,), kind="vector",
                                           init="normal" if self.one_plus else "one_plus_normal")}

    def finalize(self, device, dtype):
        if self.one_plus and not self._folded:
            self.params["weight"] = 1.0 + self.params["weight"]    # float32
            self._folded = True

    def forward_sum(self, ctx, summands, scales, stream, alpha: float, copy: bool = True):
        """``stream <- norm(alpha * stream + sum_i scales[i] * summands[i])`` in float32 (one or two summands of any
        type, nothing rounded on the way); returns the stream's new rows in the step's type for the sublayer that
        reads them next (``copy`` False, or a float32 step: the stream itself)."""
        out = None
        if copy and ctx.dtype != torch.float32:
            out = torch.empty(tuple(stream.shape), dtype=ctx.dtype, device=stream.device)
        ctx.ops.sum_norm(stream, float(alpha), summands, scales, self.params["weight"], self.eps, out)
        return stream if out is None else out

    def forward_post(self, ctx, x, stream, copy: bool = True):
        """``stream += norm(x)`` in float32, nothing rounded on the way; returns the stream's rows in the step's
        type for the sublayer that reads them next (``copy`` False, or a float32 step: the stream itself)."""
        out = None
        if copy and ctx.dtype != torch.float32:
            out = torch.empty(tuple(stream.shape), dtype=ctx.dtype, device=stream.device)
        ctx.ops.rmsnorm_post(x, self.params["weight"], self.eps, stream, out)
        return stream if out is None else out

    def forward(self, ctx, x):
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        return ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out)

    def forward_residual(self, ctx, x, residual):
        if isinstance(x, torch.Tensor) and x.dtype == torch.float32 and ctx.dtype != torch.float32:
            # a float32 summand (an embedding's output that starts the stream or joins it again) in a step of
            # another type: the sum is formed in the stream, which is then normed into the step's type
            init = residual is None
            if init:
                residual = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
            out = torch.empty(tuple(x.shape), dtype=ctx.dtype, device=x.device)
            return ctx.ops.stream_norm(residual, x, self.params["weight"], self.eps, out, init=init), residual
        pending = getattr(ctx.ops, "pending_norm", None)
        if pending is not None and residual is not None:
            # a product that has not been launched takes the residual sum as its epilogue and leaves the norm
            # to the product that follows
            lazy = pending(x, residual, self.params["weight"], self.eps)
            if lazy is not None:
                return lazy, residual
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        if residual is None:
            residual = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
            ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode="init")
        else:
            ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode="add")
        return out, residual

    def forward_rows(self, ctx, x, residual, rows):
        pending = getattr(ctx.ops, "pending_norm", None)
        if pending is not None and residual is not None:
            lazy = pending(x, residual, self.params["weight"], self.eps, rows)
            if lazy is not None:
                return lazy
        if residual is None and x.dtype == torch.float32 and ctx.dtype != torch.float32:
            # a float32 stream with nothing pending, normed into the step's type
            out = torch.empty((rows.numel(), self.size), dtype=ctx.dtype, device=x.device)
            return ctx.ops.rmsnorm_rows(x, self.params["weight"], self.eps, rows, out)
        out = torch.empty((rows.numel(), self.size), dtype=x.dtype, device=x.device)
        mode = "add" if residual is not None else "plain"
        return ctx.ops.rmsnorm(x, self.params["weight"], self.eps, out, residual=residual, mode=mode, rows=rows)


class LayerNorm(Norm):
    """``(x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b`` in float32, with the residual stream (float32)
    added first when asked.  ``weight_name`` / ``bias_name`` are the checkpoint's names under the prefix (an
    empty name: the prefix itself)."""

    def __init__(self, size: int, eps: float, prefix: str = "", weight_name: str = "weight", bias_name: str = "bias"):
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)
        self.weight_name, self.bias_name = weight_name, bias_name

    def param_specs(self):
        return {"weight": ParamSpec.single(self.weight_name, (self.size,), kind="vector", init="one_plus_normal"),
                "bias": ParamSpec.single(self.bias_name, (self.size,), kind="vector")}

    def forward(self, ctx, x, out_dtype=None):
        out = torch.empty(tuple(x.shape), dtype=out_dtype or ctx.dtype, device=x.device)
        return ctx.ops.layernorm(x, self.params["weight"], self.params["bias"], self.eps, out)

    def forward_residual(self, ctx, x, residual):
        out = torch.empty(tuple(x.shape), dtype=ctx.dtype, device=x.device)
        if residual is None:
            residual = torch.empty(tuple(x.shape), dtype=torch.float32, device=x.device)
            mode = "init"
        else:
            mode = "add"
        ctx.ops.layernorm(x, self.params["weight"], self.params["bias"], self.eps, out, residual=residual, mode=mode)
        return out, residual

    def forward_post(self, ctx, x, residual, following: "LayerNorm | None"):
        """The norm of ``x`` joins the residual stream without being rounded on the way, and the stream is
        normed by ``following`` for the sublayer that comes next (None: the sum alone).  One kernel."""
        out = None
        if following is not None:
            out = torch.empty(tuple(x.shape), dtype=ctx.dtype, device=x.device)
        ctx.ops.layernorm(x, self.params["weight"], self.params["bias"], self.eps, out, residual=residual, mode="post",
                          next_weight=following.params["weight"] if following is not None else None,
                          next_bias=following.params["bias"] if following is not None else None)
        return out

    def forward_rows(self, ctx, x, residual, rows):
        out = torch.empty((rows.numel(), self.size), dtype=ctx.dtype, device=x.device)
        mode = "add" if residual is not None else "plain"
        return ctx.ops.layernorm(x, self.params["weight"], self.params["bias"], self.eps, out, residual=residual,
                                 mode=mode, rows=rows)


NORMS.register("rmsnorm", RMSNorm)
NORMS.register("layernorm", LayerNorm)
