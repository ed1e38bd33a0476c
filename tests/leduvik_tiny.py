"""Tiny Leduvik configurations for the tests, as raw config.json dictionaries, and model folders with weights drawn
so that every mechanism shows in the logits: position rows, decays, bonus, convolution taps and biases, skip
weights, mixing weights and norm weights of a size that moves the result when they are dropped or misplaced.

The configurations differ from each other in every size.  Key and value sizes of attention differ (both ways) or
not, query heads outnumber key heads or not, windows are smaller than, equal to and larger than a cache page, the
state-space mixer has one or two groups and one, two or three norm parts, the convolution two to five taps, the
layers come in different orders, a layer has no feed-forward, the loop runs one, two or three times over different
runs of layers or is absent, and the constant on the logits is 1 in one model.
"""

from __future__ import annotations

import functools
import json
import os
import tempfile
import zlib

import torch

# inner size of the decay's two products in a time-mixing branch: a tensor's shape says it, the configuration does not
RANKS = {"A": 3, "B": 7, "C": 16, "D": 5, "X": 24}


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _attn(heads, kv_heads, dim, vdim, scale, window=None, temp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return m


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# A: side by side first, three passes over the first two layers, a window smaller than a page, sizes that fit nothing
LEDU_A = {
    "architecture": "Leduvik", "vocab": 101, "width": 40, "max_positions": 400, "norm": {"eps": 3e-5},
    "logit_scale": 0.7, "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        {"type": "parallel", "mixer": {"left": _attn(4, 2, 10, 6, 0.4, temp=(0.25, 7)), "right": {"heads": 5, "dim": 8}},
         "mlp": _dense(56)},
        {"type": "mamba2", "mixer": _ssm(4, 6, 5, 2, 2, 2), "mlp": None},
        {"type": "attention", "mixer": _attn(6, 3, 6, 10, 0.5, window=9), "mlp": _dense(48)},
    ],
}

# B: attention first with as many key heads as query heads and a window of a page; the loop over the middle two
# layers; five taps; three norm parts; no constant on the logits
LEDU_B = {
    "architecture": "Leduvik", "vocab": 131, "width": 48, "max_positions": 512, "norm": {"eps": 1e-6},
    "logit_scale": 1.0, "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "attention", "mixer": _attn(3, 3, 8, 8, 0.35, window=16), "mlp": _dense(40)},
        {"type": "mamba2", "mixer": _ssm(3, 12, 20, 1, 5, 3), "mlp": _dense(32)},
        {"type": "parallel", "mixer": {"left": _attn(2, 1, 12, 4, 0.3, temp=(0.5, 16)), "right": {"heads": 2, "dim": 20}},
         "mlp": None},
        {"type": "attention", "mixer": _attn(4, 1, 6, 6, 0.5, window=40), "mlp": _dense(24)},
    ],
}

# C: sizes the matrix-core kernels take; no loop
LEDU_C = {
    "architecture": "Leduvik", "vocab": 160, "width": 64, "max_positions": 1024, "norm": {"eps": 1e-5},
    "logit_scale": 2.0,
    "layers": [
        {"type": "mamba2", "mixer": _ssm(4, 32, 64, 2, 4, 1), "mlp": _dense(96)},
        {"type": "attention", "mixer": _attn(4, 2, 64, 32, 0.11, window=48), "mlp": _dense(64)},
        {"type": "parallel", "mixer": {"left": _attn(2, 1, 32, 128, 0.17, temp=(0.3, 32)), "right": {"heads": 2, "dim": 64}},
         "mlp": _dense(80)},
    ],
}

# X: wide enough that prompts of 5, 40, 130 and 300 tokens reach every kernel the engine has for matrix products;
# the first layer runs twice
LEDU_X = {
    "architecture": "Leduvik", "vocab": 1000, "width": 384, "max_positions": 640, "norm": {"eps": 1e-6},
    "logit_scale": 0.5, "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [
        {"type": "parallel", "mixer": {"left": _attn(6, 2, 64, 96, 0.125, temp=(0.2, 50)), "right": {"heads": 6, "dim": 64}},
         "mlp": _dense(1056)},
        {"type": "mamba2", "mixer": _ssm(12, 64, 128, 1, 4, 2), "mlp": _dense(1056)},
        {"type": "attention", "mixer": _attn(6, 3, 128, 64, 0.09, window=200), "mlp": _dense(1056)},
    ],
}

# D: odd sizes throughout (a width that is no multiple of 8, heads of 7, 9 and 11 entries, as many groups as heads in
# the state-space mixer), attention first, the loop over the last two layers
LEDU_D = {
    "architecture": "Leduvik", "vocab": 77, "width": 52, "max_positions": 300, "norm": {"eps": 1e-5},
    "logit_scale": 1.3, "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        {"type": "attention", "mixer": _attn(5, 5, 7, 9, 0.4, window=11), "mlp": _dense(30)},
        {"type": "mamba2", "mixer": _ssm(3, 7, 9, 3, 3, 1), "mlp": _dense(34)},
        {"type": "parallel", "mixer": {"left": _attn(3, 1, 9, 5, 0.3, temp=(0.4, 5)), "right": {"heads": 3, "dim": 11}},
         "mlp": None},
    ],
}

CONFIGS = {"A": LEDU_A, "B": LEDU_B, "C": LEDU_C, "D": LEDU_D, "X": LEDU_X}
SEEDS = {"A": 7, "B": 17, "C": 29, "D": 5, "X": 41}


def _draw(name: str, shape, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    last = name.rsplit(".", 1)[-1]
    z = torch.randn(shape, generator=g)
    if name.endswith(".conv"):
        return 0.5 * z
    if name.endswith(".conv.b"):
        return 0.3 * z
    if ".mu." in name:
        return torch.sigmoid(z)
    if last == "dt_bias":
        return 0.3 + 0.7 * z
    if last == "A_log":
        return 0.6 * z - 0.5
    if last == "w0":
        return z - 1.0
    if last == "u":
        return 0.5 * z
    if last == "pos":
        return 0.5 * z
    if last == "embed":
        return z
    if len(shape) == 1:                       # norm weights, skip weights
        return 1.0 + 0.2 * z
    return z / shape[-1] ** 0.5               # matrices: outputs of unit size


def _attention_shapes(p, m, w):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    return {p + "q": (H * D, w), p + "k": (G * D, w), p + "v": (G * V, w), p + "o": (w, H * V)}


def shapes(which: str) -> dict:
    """Every tensor a checkpoint of configuration ``which`` holds, by name, written out here from the design
    (not taken from the engine's own list): the tests compare the two."""
    cfg = CONFIGS[which]
    w, v = cfg["width"], cfg["vocab"]
    out = {"embed": (v, w), "pos": (cfg["max_positions"], w), "final.norm": (w,), "head": (v, w)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        if layer["type"] == "mamba2":
            H, V, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * V, H * V + 2 * G * N
            out.update({p + "mix.in": (2 * inner + 2 * G * N + H, w), p + "mix.conv": (ch, m["conv"]),
                        p + "mix.conv.b": (ch,), p + "mix.dt_bias": (H,), p + "mix.A_log": (H,), p + "mix.D": (H,),
                        p + "mix.norm": (inner,), p + "mix.o": (w, inner)})
        elif layer["type"] == "attention":
            out.update(_attention_shapes(p + "mix.", m, w))
        else:
            out.update(_attention_shapes(p + "mix.left.", m["left"], w))
            H, K, r = m["right"]["heads"], m["right"]["dim"], RANKS[which]
            c, q = H * K, p + "mix.right."
            out.update({q + f"mu.{s}": (w,) for s in "rkvgw"})
            out.update({q + "r": (c, w), q + "k": (c, w), q + "v": (c, w), q + "g": (c, w), q + "w1": (r, w),
                        q + "w2": (c, r), q + "w0": (c,), q + "u": (H, K), q + "norm": (c,), q + "o": (w, c),
                        p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (w,), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return out


@functools.lru_cache(maxsize=None)
def folder(which: str, stored: str = "bfloat16") -> str:
    """A model folder (config.json + model.safetensors) of configuration ``which``."""
    from safetensors.torch import save_file

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored]
    path = os.path.join(_TMP.name, f"ledu_{which}_{stored}")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(CONFIGS[which], f)
    tensors = {name: _draw(name, shape, SEEDS[which]).to(dtype).contiguous() for name, shape in shapes(which).items()}
    save_file(tensors, os.path.join(path, "model.safetensors"))
    return path


@functools.lru_cache(maxsize=None)
def tensors(which: str, stored: str = "bfloat16") -> dict:
    from safetensors.torch import load_file

    loaded = load_file(os.path.join(folder(which, stored), "model.safetensors"))
    return {k: v.double() for k, v in loaded.items()}


def ids(which: str, n: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[which]["vocab"], (n,), generator=g).tolist()


_ORACLE: dict = {}


def oracle(which: str, tokens: list[int], stored: str = "bfloat16") -> torch.Tensor:
    import plain_leduvik as pl

    key = (which, stored, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = pl.forward(CONFIGS[which], tensors(which, stored), tokens)[0]
    return _ORACLE[key]


def float32_error(which: str, tokens: list[int], stored: str = "bfloat16") -> torch.Tensor:
    """Per position, how far the plain implementation run in float32 is from itself in float64 (largest difference
    of a logit): what rounding alone does at that token with these weights."""
    import plain_leduvik as pl

    key = (which, stored, tuple(tokens), "float32")
    if key not in _ORACLE:
        wide = pl.WIDE
        pl.WIDE = torch.float32
        try:
            narrow = pl.forward(CONFIGS[which], {k: v.float() for k, v in tensors(which, stored).items()}, tokens)[0]
        finally:
            pl.WIDE = wide
        _ORACLE[key] = (narrow.double() - oracle(which, tokens, stored)).abs().amax(dim=1)
    return _ORACLE[key]


def core(which: str, dtype: str, ops, device: str, num_pages: int = 64, max_num_seqs: int = 4, page_size: int = 16,
         graph_sizes=None, stored: str = "bfloat16"):
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model

    model, _ = load_model(folder(which, stored), dtype=TORCH_DTYPES[dtype], device=device)
    return build_core(model, ops, dtype=TORCH_DTYPES[dtype], device=device, page_size=page_size, num_pages=num_pages,
                      max_num_seqs=max_num_seqs, max_model_len=num_pages * page_size, graph_sizes=graph_sizes)


_TMP = tempfile.TemporaryDirectory(prefix="atom_amd_leduvik_")
