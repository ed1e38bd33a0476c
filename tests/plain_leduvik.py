"""A plain, slow implementation of the Leduvik design in float64, one function per mechanism, written from the
design's equations and sharing no code with the engine.  Recurrent mixers walk the tokens one by one; attention
builds the whole score matrix.  ``forward`` takes a request's tokens (or a further portion of them together with
what the earlier portions ``carried``) and returns the logits at every position.

Notation: T tokens, W the model width, H heads, G key/value heads (or groups), K a head's key size, V its value
size, N the state size of the state-space mixer.
"""

from __future__ import annotations

import json
import math
import os

import torch

WIDE = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def unit_rms(x, eps):
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def relu_squared(z):
    return torch.clamp(z, min=0) ** 2


# ------------------------------------------------------------------ embedding


def embed_rows(ids, positions, table, pos_table):
    """Token row plus the learned row of the token's position."""
    return table[ids] + pos_table[positions]


# ------------------------------------------------------------------ attention


def query_temperature(positions, coef: float, every: int):
    """The factor on a query at position p: 1 + coef ln(floor((p + 1) / every) + 1)."""
    steps = torch.div(positions + 1, every, rounding_mode="floor").to(WIDE)
    return 1 + coef * torch.log(steps + 1)


def may_see(i: int, j: int, window: int | None) -> bool:
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    return window is None or i - j < window


def softmax_attention(q, k, v, q_pos, k_pos, scale: float, window: int | None):
    """q [Tq, H, K], k [Tk, G, K], v [Tk, G, V]; query head h reads key/value head h // (H / G)."""
    Tq, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(Tq, H, v.shape[2], dtype=WIDE)
    mask = torch.tensor([[may_see(int(i), int(j), window) for j in k_pos] for i in q_pos])
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_mixer(h, positions, w, m, eps, carried=None, unit_qk=False, temperature=None, window=None):
    """w: the mixer's tensors by their names (q, k, v, o); carried: (k, v, positions) of the tokens before."""
    T = h.shape[0]
    H, G, K, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, K)
    k = (h @ w["k"].T).reshape(T, G, K)
    v = (h @ w["v"].T).reshape(T, G, V)
    if unit_qk:
        q, k = unit_rms(q, eps), unit_rms(k, eps)
    if temperature is not None:
        q = q * query_temperature(positions, temperature["coef"], temperature["every"])[:, None, None]
    k_pos = positions
    if carried is not None:
        k, v, k_pos = torch.cat((carried[0], k)), torch.cat((carried[1], v)), torch.cat((carried[2], positions))
    o = softmax_attention(q, k, v, positions, k_pos, m["scale"], window)
    return o.reshape(T, H * V) @ w["o"].T, (k, v, k_pos)


# ------------------------------------------------------------------ the time-mixing recurrence with a bonus


def bonus_recurrence(r, k, v, decay, bonus, S):
    """Per head: o_t = (S + diag(bonus) k_t v_t^T)^T r_t, then S <- diag(decay_t) S + k_t v_t^T.
    r, k, decay [T, H, K]; v [T, H, V]; bonus [H, K]; S [H, K, V]."""
    T, H, _ = r.shape
    out = torch.zeros(T, H, v.shape[2], dtype=WIDE)
    S = S.clone()
    for t in range(T):
        for h in range(H):
            kv = torch.outer(k[t, h], v[t, h])
            out[t, h] = (S[h] + bonus[h][:, None] * kv).T @ r[t, h]
            S[h] = decay[t, h][:, None] * S[h] + kv
    return out, S


def time_mix_mixer(h, w, m, eps, carried=None):
    """w: r, k, v, g, w1, w2, w0, u, norm, o and mu.{r,k,v,g,w}; carried: (the previous token's h, S)."""
    T, W = h.shape
    H, K = m["heads"], m["dim"]
    last, S = carried if carried is not None else (torch.zeros(W, dtype=WIDE), torch.zeros(H, K, K, dtype=WIDE))
    before = torch.cat((last[None], h[:-1]))
    mix = {s: h + (before - h) * w[f"mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ w["r"].T).reshape(T, H, K)
    k = (mix["k"] @ w["k"].T).reshape(T, H, K)
    v = (mix["v"] @ w["v"].T).reshape(T, H, K)
    gate = silu(mix["g"] @ w["g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w["w1"].T) @ w["w2"].T + w["w0"])).reshape(T, H, K)
    o, S = bonus_recurrence(r, k, v, decay, w["u"], S)
    o = unit_rms(o, eps).reshape(T, H * K) * w["norm"] * gate
    return o @ w["o"].T, (h[-1], S)


# ------------------------------------------------------------------ the state-space mixer


def short_convolution(x, taps_w, bias, before=None):
    """x [T, C]; taps_w [C, taps], the last column weighs the current token; ``before`` [taps - 1, C]: the inputs
    ahead of x (zeros at a request's start).  Returns (y [T, C], the last taps - 1 inputs)."""
    taps = taps_w.shape[1]
    if before is None:
        before = torch.zeros(taps - 1, x.shape[1], dtype=x.dtype)
    padded = torch.cat((before, x), dim=0)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(taps):
            y[t] += padded[t + j] * taps_w[:, j]
    return y + bias, padded[padded.shape[0] - (taps - 1):]


def state_space_recurrence(x, B, C, dt, A, D, S):
    """Per head h with group g = h // (H / G): S <- exp(-A_h dt) S + dt B_g x^T, y = S^T C_g + D_h x.
    x [T, H, V]; B, C [T, G, N]; dt [T, H]; A, D [H]; S [H, N, V]."""
    T, H, V = x.shape
    G = B.shape[1]
    y = torch.zeros(T, H, V, dtype=WIDE)
    S = S.clone()
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            S[h] = torch.exp(-A[h] * dt[t, h]) * S[h] + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S[h].T @ C[t, g] + D[h] * x[t, h]
    return y, S


def state_space_mixer(h, w, m, eps, carried=None):
    """w: in, conv, conv.b, dt_bias, A_log, D, norm, o; carried: (conv inputs, S)."""
    T = h.shape[0]
    H, V, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * V
    z, xBC, dt = torch.split(h @ w["in"].T, [inner, inner + 2 * G * N, H], dim=-1)
    before, S = carried if carried is not None else (None, torch.zeros(H, N, V, dtype=WIDE))
    xBC, tail = short_convolution(xBC, w["conv"], w["conv.b"], before)
    x, B, C = torch.split(silu(xBC), [inner, G * N, G * N], dim=-1)
    dt = softplus(dt + w["dt_bias"])
    y, S = state_space_recurrence(x.reshape(T, H, V), B.reshape(T, G, N), C.reshape(T, G, N), dt,
                                  torch.exp(w["A_log"]), w["D"], S)
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T, (tail, S)


# ------------------------------------------------------------------ two mixers side by side


def parallel_mixer(h, positions, w, m, eps, carried=None):
    """Half the sum of the two branches' outputs, each RMS-normed over the model width with its own weight."""
    left_c, right_c = carried if carried is not None else (None, None)
    left, left_c = attention_mixer(h, positions, sub(w, "left"), m["left"], eps, left_c,
                                   temperature=m["left"].get("q_temp"))
    right, right_c = time_mix_mixer(h, sub(w, "right"), m["right"], eps, right_c)
    return 0.5 * (rms_norm(left, w["left.out"], eps) + rms_norm(right, w["right.out"], eps)), (left_c, right_c)


def dense_ff(h, w):
    return relu_squared(h @ w["up"].T) @ w["down"].T


# ------------------------------------------------------------------ the model


def sub(tensors, prefix):
    return {k[len(prefix) + 1:]: v for k, v in tensors.items() if k.startswith(prefix + ".")}


def running_order(cfg) -> list[tuple[int, bool]]:
    """(layer, whether the embedding's output is added before it) in running order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["times"] <= 1 or loop["stop"] <= loop["start"]:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        runs += [(i, p > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def mixer(layer, h, positions, w, eps, carried):
    kind, m = layer["type"], layer["mixer"]
    if kind == "attention":
        return attention_mixer(h, positions, w, m, eps, carried, unit_qk=True,
                               window=(m.get("mask") or {}).get("size"))
    if kind == "mamba2":
        return state_space_mixer(h, w, m, eps, carried)
    if kind == "parallel":
        return parallel_mixer(h, positions, w, m, eps, carried)
    raise ValueError(f"unknown layer type {kind!r}")


def forward(cfg, tensors, ids, carried=None, trail=None):
    """Logits [T, vocab] of the tokens ``ids`` that follow what ``carried`` holds (None: a request's start), and
    what to carry on.  ``trail``, a list, receives the stream after every run of a layer."""
    eps = cfg["norm"]["eps"]
    ids = torch.as_tensor(ids, dtype=torch.long)
    order = running_order(cfg)
    done, memory = carried if carried is not None else (0, [None] * len(order))
    positions = torch.arange(done, done + len(ids))
    x = first = embed_rows(ids, positions, tensors["embed"], tensors["pos"])
    memory = list(memory)
    for run, (i, adds_first) in enumerate(order):
        layer = cfg["layers"][i]
        if adds_first:
            x = x + first
        out, memory[run] = mixer(layer, rms_norm(x, tensors[f"l{i}.norm1"], eps), positions,
                                 sub(tensors, f"l{i}.mix"), eps, memory[run])
        x = x + out
        if layer.get("mlp") is not None:
            x = x + dense_ff(rms_norm(x, tensors[f"l{i}.norm2"], eps), sub(tensors, f"l{i}.mlp"))
        if trail is not None:
            trail.append(x.clone())
    logits = rms_norm(x, tensors["final.norm"], eps) @ tensors["head"].T * cfg.get("logit_scale", 1.0)
    return logits, (done + len(ids), memory)


def load_folder(folder: str):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(WIDE) if t.is_floating_point() else t
    return cfg, tensors
