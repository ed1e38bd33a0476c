"""A plain, slow Savidra: one function per mechanism, whole sequences at once or token by token, float64 unless
told otherwise.  It shares nothing with the engine: weights come as a dict of tensors by checkpoint name, the
configuration as the dict a config.json holds.

The design: ``x = embed[t]``; every layer is ``x <- norm1(alpha x + mixer(shift(x)))`` and then
``x <- norm2(alpha x + ff(x))`` with RMS norms whose weight is stored as its distance from one; ``shift`` blends a
token's row with the previous token's; the mixer is softmax attention with a sink and values blended with those of
an earlier layer (``attention``), or two mixers side by side (``parallel``): attention behind short convolutions,
with a temperature per head and the heads' weights mixed after the softmax, and a gated delta rule with a decay per
key channel; the feed-forward is ``W_down (relu(W_gate x) * W_up x)``.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def one_plus_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1 + w)


def plain_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def token_shift(x, mu, prev):
    """x [T, W]; prev [W] is the row before x[0] (zeros at a sequence's start).  Returns the blend and the new prev."""
    before = torch.cat([prev[None], x[:-1]], 0)
    return x + (before - x) * mu, x[-1].clone()


def short_conv(u, w, carried):
    """u [T, C], w [C, taps] with the last column the current token's; carried [taps - 1, C] are the inputs before
    u[0].  Returns y [T, C] and the inputs to carry on."""
    taps = w.shape[1]
    full = torch.cat([carried, u], 0)
    T = u.shape[0]
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + full[j:j + T] * w[:, j]
    return y, full[full.shape[0] - (taps - 1):].clone()


def rotate_half(x, positions, dims, base, factor=1.0):
    """x [T, heads, dim]: entry i of the first ``dims`` is paired with i + dims / 2."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=F)
    a = positions.to(F)[:, None] * f[None]            # [T, half]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def softmax_weights(q, k, positions_q, positions_k, scale, sink=None, temp=None, window=None):
    """q [Tq, H, D], k [Tk, G, D] -> weights [H, Tq, Tk], causal by position, an optional sink in the denominator;
    ``window``: a query sees itself and the ``window - 1`` positions before it (the design has none; the engine's
    kernels offer it)."""
    H, G = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if temp is not None:
        s = s * temp[:, None, None]
    seen = positions_k[None, :] <= positions_q[:, None]
    if window:
        seen = seen & (positions_k[None, :] > positions_q[:, None] - window)
    s = s.masked_fill(~seen[None], -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None, None])
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink[:, None, None] - m)
    return e / den


def apply_weights(w, v, H):
    """w [H, Tq, Tk], v [Tk, G, dv] -> [Tq, H * dv]; head h reads the values of head h // (H / G)."""
    G = v.shape[1]
    vv = v.repeat_interleave(H // G, dim=1)
    return torch.einsum("hij,jhd->ihd", w, vv).reshape(w.shape[1], -1)


def delta_rule(q, k, v, beta, g, S):
    """q, k [T, H, dk] (unit length, q scaled), v [T, H, dv], beta [T, H], g [T, H, dk], S [H, dk, dv]."""
    out = []
    for t in range(q.shape[0]):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - torch.einsum("hkv,hk->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out.append(torch.einsum("hkv,hk->hv", S, q[t]))
    return torch.stack(out), S


def silu(x):
    return x * torch.sigmoid(x)


class PlainSavidra:
    """Keeps a sequence's memory between calls of ``forward``, so a prompt can be fed whole, in portions or token
    by token."""

    def __init__(self, config: dict, weights: dict, dtype=F):
        self.cfg = config
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.dtype = dtype
        self.eps = config["norm"]["eps"]
        self.alpha = config["postln_alpha"]
        self.width = config["width"]
        self.reset()

    def reset(self):
        self.pos = 0
        self.mem = [dict() for _ in self.cfg["layers"]]

    # ---- mixers

    def _project(self, m, h, positions, mem, p, biased=True, conv=True):
        w, eps = self.w, self.eps
        H, G, D, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        parts = {}
        for n in "qkv":
            y = h @ w[f"{p}.{n}"].T
            if biased:
                y = y + w[f"{p}.{n}.b"]
            if conv:
                taps = m["conv"]
                carried = mem.setdefault(f"conv_{n}", torch.zeros(taps - 1, y.shape[1], dtype=self.dtype))
                y, mem[f"conv_{n}"] = short_conv(y, w[f"{p}.{n}.conv"], carried)
            parts[n] = y
        q = plain_norm(parts["q"].view(T, H, D), w[f"{p}.q.norm"], eps)
        k = plain_norm(parts["k"].view(T, G, D), w[f"{p}.k.norm"], eps)
        v = parts["v"].view(T, G, dv)
        rot = m.get("rot")
        if rot is not None:
            factor = (rot.get("scaling") or {}).get("factor", 1.0)
            q = rotate_half(q, positions, rot["dims"], rot["base"], factor)
            k = rotate_half(k, positions, rot["dims"], rot["base"], factor)
        return q, k, v

    def _attend(self, mem, q, k, v, positions, scale, H, sink=None, temp=None, talk=None):
        keys = torch.cat([mem["k"], k], 0) if "k" in mem else k
        vals = torch.cat([mem["v"], v], 0) if "v" in mem else v
        mem["k"], mem["v"] = keys, vals
        pk = torch.arange(keys.shape[0])
        wts = softmax_weights(q, keys, positions, pk, scale, sink=sink, temp=temp)
        if talk is not None:
            wts = torch.einsum("hg,gij->hij", talk, wts)
        return apply_weights(wts, vals, H)

    def _right(self, m, h, mem, p):
        w = self.w
        H, G, D, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        parts = {}
        for n in "qkv":
            y = h @ w[f"{p}.{n}"].T
            carried = mem.setdefault(f"rconv_{n}", torch.zeros(m["conv"] - 1, y.shape[1], dtype=self.dtype))
            y, mem[f"rconv_{n}"] = short_conv(y, w[f"{p}.{n}.conv"], carried)
            parts[n] = silu(y)
        unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)  # noqa: E731
        q = unit(parts["q"].view(T, G, D)) * D ** -0.5
        k = unit(parts["k"].view(T, G, D))
        q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
        v = parts["v"].view(T, H, dv)
        beta = torch.sigmoid(h @ w[f"{p}.b"].T)
        raw = (h @ w[f"{p}.a1"].T) @ w[f"{p}.a2"].T + w[f"{p}.dt_bias"]
        g = torch.exp(-torch.exp(w[f"{p}.A_log"])[None, :, None] * torch.nn.functional.softplus(raw).view(T, H, D))
        S = mem.setdefault("S", torch.zeros(H, D, dv, dtype=self.dtype))
        o, mem["S"] = delta_rule(q, k, v, beta, g, S)
        o = plain_norm(o, w[f"{p}.norm"], self.eps)
        gate = torch.sigmoid((h @ w[f"{p}.g1"].T) @ w[f"{p}.g2"].T).view(T, H, dv)
        return (o * gate).reshape(T, H * dv) @ w[f"{p}.o"].T

    def _mixer(self, i, layer, h, positions, shared):
        w, mem, m = self.w, self.mem[i], layer["mixer"]
        p = f"l{i}.mix"
        if layer["type"] == "attention":
            q, k, v = self._project(m, h, positions, mem, p, biased=False, conv=False)
            if m.get("v_mix"):
                if "v_first" in shared:
                    lam = w[f"{p}.vmix"]
                    v = (1 - lam) * v + lam * shared["v_first"]
                else:
                    shared["v_first"] = v
            o = self._attend(mem, q, k, v, positions, m["scale"], m["heads"], sink=w[f"{p}.sink"])
            return o @ w[f"{p}.o"].T
        if layer["type"] != "parallel":
            raise ValueError(layer["type"])
        lm = m["left"]
        q, k, v = self._project(lm, h, positions, mem, f"{p}.left")
        o = self._attend(mem, q, k, v, positions, lm["scale"], lm["heads"], temp=w[f"{p}.left.temp"],
                         talk=w[f"{p}.left.talk"])
        left = o @ w[f"{p}.left.o"].T + w[f"{p}.left.o.b"]
        right = self._right(m["right"], h, mem, f"{p}.right")
        return m["left_scale"] * left + m["right_scale"] * right

    def _ff(self, i, x):
        w = self.w
        return (torch.relu(x @ w[f"l{i}.mlp.gate"].T) * (x @ w[f"l{i}.mlp.up"].T)) @ w[f"l{i}.mlp.down"].T

    # ---- the model

    def forward(self, tokens, layers_out: list | None = None):
        """Feeds the next tokens of the sequence; returns logits [T, vocab]."""
        w = self.w
        T = len(tokens)
        positions = torch.arange(self.pos, self.pos + T)
        self.pos += T
        x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
        shared = {}
        for i, layer in enumerate(self.cfg["layers"]):
            prev = self.mem[i].setdefault("shift", torch.zeros(self.width, dtype=self.dtype))
            h, self.mem[i]["shift"] = token_shift(x, w[f"l{i}.shift"], prev)
            x = one_plus_norm(self.alpha * x + self._mixer(i, layer, h, positions, shared), w[f"l{i}.norm1"], self.eps)
            if layer.get("mlp") is not None:
                x = one_plus_norm(self.alpha * x + self._ff(i, x), w[f"l{i}.norm2"], self.eps)
            elif f"l{i}.norm2" in w:      # a second norm without a feed-forward: nothing is added
                x = one_plus_norm(self.alpha * x, w[f"l{i}.norm2"], self.eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        x = one_plus_norm(x, w["final.norm"], self.eps)
        return x @ w["head"].T
