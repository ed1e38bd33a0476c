"""Tiny Savidra configurations for the tests, as raw config.json dictionaries, and model folders with weights drawn
so that every mechanism shows in the logits: shift weights, sinks, temperatures, head mixing, value blending,
convolution taps, biases, decays and norm weights of a size that moves the result when they are dropped or misplaced.

The configurations differ from each other in every size.  Key and value sizes differ (both ways) or not, query heads
outnumber key heads or not, the rotated part is a head's whole, a part of it or nothing, positions are stretched or
not, convolutions have two to five taps, the layers come in different orders, a layer has no feed-forward, the first
layer that blends values is the first layer or a later one, the constant on the stream is 1 in one model and the
branches' constants are 1 in another.
"""

from __future__ import annotations

import functools
import json
import os
import tempfile
import zlib

import torch

from plain_savidra import PlainSavidra

# inner sizes of the delta branch's decay and gate products: a tensor's shape says them, the configuration does not
RANKS = {"A": (3, 5), "B": (6, 2), "C": (16, 8), "D": (4, 4), "E": (2, 3)}
# layers without a feed-forward whose checkpoint nevertheless holds a second norm
BARE_SECOND_NORM = {("E", 1)}


def _rot(dims, base, factor=None):
    r = {"dims": dims, "base": base}
    if factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def _attn(heads, kv_heads, dim, vdim, scale, rot, v_mix=None, conv=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot}
    if v_mix is not None:
        m["v_mix"] = v_mix
    if conv is not None:
        m["conv"] = conv
    return m


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _side(left, right, ls, rs):
    return {"left": left, "right": right, "left_scale": ls, "right_scale": rs}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# A: attention first (it is the source of the blended values), sizes that fit nothing, a layer without feed-forward
SAVI_A = {
    "architecture": "Savidra", "vocab": 97, "width": 40, "norm": {"eps": 3e-5}, "postln_alpha": 1.5,
    "layers": [
        {"type": "attention", "mixer": _attn(4, 2, 10, 6, 0.4, _rot(6, 1000.0), v_mix=True), "mlp": _dense(56)},
        {"type": "parallel", "mixer": _side(_attn(6, 3, 6, 4, 0.5, _rot(6, 300.0, 4.0), conv=2), _delta(4, 2, 5, 7, 3),
                                            0.7, 1.2), "mlp": None},
        {"type": "attention", "mixer": _attn(2, 2, 12, 6, 0.3, _rot(4, 50.0), v_mix=True), "mlp": _dense(48)},
        {"type": "attention", "mixer": _attn(3, 3, 8, 5, 0.35, _rot(8, 10000.0), v_mix=False), "mlp": _dense(32)},
    ],
}

# B: side by side first, the source of the blended values in the middle, constants of 1, five taps, no stretch
SAVI_B = {
    "architecture": "Savidra", "vocab": 131, "width": 48, "norm": {"eps": 1e-6}, "postln_alpha": 1.0,
    "layers": [
        {"type": "parallel", "mixer": _side(_attn(2, 1, 12, 20, 0.3, _rot(8, 500.0), conv=5), _delta(3, 3, 9, 6, 2),
                                            1.0, 1.0), "mlp": _dense(40)},
        {"type": "attention", "mixer": _attn(4, 1, 6, 9, 0.5, _rot(6, 100.0), v_mix=True), "mlp": None},
        {"type": "parallel", "mixer": _side(_attn(3, 3, 7, 7, 0.4, _rot(2, 20.0, 2.0), conv=3), _delta(2, 1, 12, 10, 4),
                                            0.5, 1.5), "mlp": _dense(24)},
        {"type": "attention", "mixer": _attn(3, 1, 10, 9, 0.45, _rot(10, 777.0), v_mix=True), "mlp": _dense(36)},
    ],
}

# C: sizes that matrix-core kernels take; one attention layer whose values have the keys' size, one whose have not
SAVI_C = {
    "architecture": "Savidra", "vocab": 160, "width": 64, "norm": {"eps": 1e-5}, "postln_alpha": 2.5,
    "layers": [
        {"type": "parallel", "mixer": _side(_attn(4, 2, 64, 64, 0.17, _rot(32, 10000.0, 6.0), conv=4),
                                            _delta(2, 1, 32, 64, 4), 0.8, 0.9), "mlp": _dense(96)},
        {"type": "attention", "mixer": _attn(4, 2, 64, 64, 0.11, _rot(32, 50000.0), v_mix=True), "mlp": _dense(64)},
        {"type": "attention", "mixer": _attn(2, 2, 128, 64, 0.09, _rot(64, 1000.0), v_mix=True), "mlp": _dense(80)},
    ],
}

# D: one layer of each kind, one head, no rotated part in the attention layer
SAVI_D = {
    "architecture": "Savidra", "vocab": 61, "width": 36, "norm": {"eps": 1e-5}, "postln_alpha": 3.0,
    "layers": [
        {"type": "attention", "mixer": _attn(1, 1, 9, 11, 0.33, _rot(0, 10.0)), "mlp": _dense(30)},
        {"type": "parallel", "mixer": _side(_attn(1, 1, 14, 3, 0.27, _rot(14, 64.0, 1.0), conv=3), _delta(1, 1, 7, 9, 5),
                                            1.3, 0.4), "mlp": _dense(20)},
    ],
}

# E: convolutions of one tap (nothing carried), a second norm in a layer without feed-forward, no key sizes named
SAVI_E = {
    "architecture": "Savidra", "vocab": 53, "width": 24, "norm": {"eps": 1e-6}, "postln_alpha": 0.5,
    "layers": [
        {"type": "parallel", "mixer": _side(_attn(2, 2, 6, 6, 0.4, _rot(6, 30.0), conv=1), _delta(2, 2, 4, 4, 1), 1.0, 0.9),
         "mlp": _dense(16)},
        {"type": "attention", "mixer": _attn(2, 1, 8, 8, 0.35, None), "mlp": None},
    ],
}

CONFIGS = {"A": SAVI_A, "B": SAVI_B, "C": SAVI_C, "D": SAVI_D, "E": SAVI_E}
SEEDS = {"A": 3, "B": 13, "C": 23, "D": 43, "E": 53}


def _draw(name: str, shape, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
    last = name.rsplit(".", 1)[-1]
    z = torch.randn(shape, generator=g)
    if last == "conv":
        return 0.5 * z
    if last == "shift":
        return torch.sigmoid(z)
    if last == "dt_bias":
        return 0.3 + 0.7 * z
    if last == "A_log":
        return 0.6 * z - 0.5
    if last == "temp":
        return 1.0 + 0.3 * z
    if last == "talk":
        return torch.eye(shape[0]) + 0.3 * z
    if last == "sink":
        return 1.5 * z
    if last == "vmix":
        return torch.tensor(0.35) + 0.1 * z
    if last in ("norm1", "norm2") or name == "final.norm":
        return 0.2 * z                          # stored as the distance from one
    if last == "embed":
        return z
    if last == "b" and len(shape) == 1:
        return 0.3 * z
    if len(shape) == 1:                       # plain norm weights
        return 1.0 + 0.2 * z
    return z / shape[-1] ** 0.5               # matrices: outputs of unit size


def _attention_shapes(p, m, w, side):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    out = {p + "q": (H * D, w), p + "k": (G * D, w), p + "v": (G * V, w), p + "o": (w, H * V),
           p + "q.norm": (D,), p + "k.norm": (D,)}
    if side:
        out.update({p + "q.b": (H * D,), p + "k.b": (G * D,), p + "v.b": (G * V,), p + "o.b": (w,),
                    p + "q.conv": (H * D, m["conv"]), p + "k.conv": (G * D, m["conv"]), p + "v.conv": (G * V, m["conv"]),
                    p + "talk": (H, H), p + "temp": (H,)})
    else:
        out[p + "sink"] = (H,)
        if m.get("v_mix"):
            out[p + "vmix"] = ()
    return out


def shapes(which: str) -> dict:
    """Every tensor a checkpoint of configuration ``which`` holds, by name, written out here from the design
    (not taken from the engine's own list): the tests compare the two."""
    cfg = CONFIGS[which]
    w, v = cfg["width"], cfg["vocab"]
    out = {"embed": (v, w), "final.norm": (w,), "head": (v, w)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (w,)
        out[p + "shift"] = (w,)
        if layer["type"] == "attention":
            out.update(_attention_shapes(p + "mix.", m, w, False))
        else:
            out.update(_attention_shapes(p + "mix.left.", m["left"], w, True))
            r, q = m["right"], p + "mix.right."
            H, G, D, V = r["heads"], r["kv_heads"], r["dim"], r["vdim"]
            ra, rg = RANKS[which]
            out.update({q + "q": (G * D, w), q + "k": (G * D, w), q + "v": (H * V, w),
                        q + "q.conv": (G * D, r["conv"]), q + "k.conv": (G * D, r["conv"]), q + "v.conv": (H * V, r["conv"]),
                        q + "b": (H, w), q + "A_log": (H,), q + "norm": (V,), q + "a1": (ra, w), q + "a2": (H * D, ra),
                        q + "dt_bias": (H * D,), q + "g1": (rg, w), q + "g2": (H * V, rg), q + "o": (w, H * V)})
        if (which, i) in BARE_SECOND_NORM:
            out[p + "norm2"] = (w,)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out.update({p + "norm2": (w,), p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
    return out


@functools.lru_cache(maxsize=None)
def folder(which: str, stored: str = "bfloat16") -> str:
    """A model folder (config.json + model.safetensors) of configuration ``which``."""
    from safetensors.torch import save_file

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[stored]
    path = os.path.join(_TMP.name, f"savi_{which}_{stored}")
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(CONFIGS[which], f)
    made = {name: _draw(name, shape, SEEDS[which]).to(dtype).contiguous() for name, shape in shapes(which).items()}
    save_file(made, os.path.join(path, "model.safetensors"))
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
    key = (which, stored, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = PlainSavidra(CONFIGS[which], tensors(which, stored)).forward(tokens)
    return _ORACLE[key]


def core(which: str, dtype: str, ops, device: str, num_pages: int = 64, max_num_seqs: int = 4, page_size: int = 16,
         graph_sizes=None, stored: str = "bfloat16"):
    from atom_amd.engine.core import TORCH_DTYPES, build_core, load_model

    model, _ = load_model(folder(which, stored), dtype=TORCH_DTYPES[dtype], device=device)
    return build_core(model, ops, dtype=TORCH_DTYPES[dtype], device=device, page_size=page_size, num_pages=num_pages,
                      max_num_seqs=max_num_seqs, max_model_len=num_pages * page_size, graph_sizes=graph_sizes)


_TMP = tempfile.TemporaryDirectory(prefix="atom_amd_savidra_")
