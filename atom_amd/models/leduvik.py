"""Leduvik as a ``ModelSpec``.

The stream starts as the token's embedding row plus a learned row for its position, float32 throughout.  Every
layer is a pre-norm block with RMS norms: ``x += mixer(norm1(x))``, then ``x += ff(norm2(x))`` where the layer has
a feed-forward.  The mixer is a selective state-space recurrence (``mamba2``), grouped-query attention over a
sliding window with unit-norm queries and keys and no rotation (``attention``), or two mixers side by side
(``parallel``): causal attention whose queries are scaled by a temperature that grows with position, and a
time-mixing recurrence with a decay per key channel; their outputs are RMS-normed and averaged.  The feed-forward
is ``W_down relu(W_up h)^2``.  Layers ``start .. stop - 1`` of ``loop`` run ``times`` times in a row with the same
weights, each pass with memory of its own; before every pass but the first the embedding's output is added to the
stream.  A final RMS norm, an untied head, and a constant on the logits.

Checkpoint names: ``embed``, ``pos``, ``l<i>.norm1`` / ``.norm2`` (weights), ``l<i>.mix.*``, ``l<i>.mlp.{up,down}``,
``final.norm``, ``head``; matrices carry no ``.weight`` suffix, biases end in ``.b``.
"""

from __future__ import annotations

from ..config.model_config import LeduvikConfig
from ..parts.base import PartChoice
from .model import LayerRun, ModelSpec


def _attention(cfg: LeduvikConfig, m: dict, unit_norm: bool) -> PartChoice:
    temp = m.get("q_temp")
    return PartChoice("plain_attention", {
        "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "value_dim": m["vdim"], "scale": m["scale"], "unit_norm": unit_norm, "norm_eps": cfg.norm_eps,
        "temperature": (temp["coef"], temp["every"]) if temp is not None else None,
        "window": (m.get("mask") or {}).get("size")})


def _mixer(cfg: LeduvikConfig, layer: dict) -> PartChoice:
    m = layer["mixer"]
    if layer["type"] == "mamba2":
        return PartChoice("state_space", {
            "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "value_dim": m["vdim"], "state_size": m["state"],
            "groups": m["groups"], "conv_taps": m["conv"], "norm_groups": m["norm_groups"], "norm_eps": cfg.norm_eps})
    if layer["type"] == "attention":
        return _attention(cfg, m, unit_norm=True)
    right = m["right"]
    return PartChoice("parallel", {
        "hidden_size": cfg.hidden_size, "norm_eps": cfg.norm_eps,
        "branches": [("left", _attention(cfg, m["left"], unit_norm=False)),
                     ("right", PartChoice("time_mix", {"hidden_size": cfg.hidden_size, "num_heads": right["heads"],
                                                       "head_dim": right["dim"], "norm_eps": cfg.norm_eps,
                                                       # the checkpoint's tensors say it; a configuration may name
                                                       # it for weights that are drawn, not loaded
                                                       "decay_rank": right.get("decay_rank")}))]})


def _feed_forward(cfg: LeduvikConfig, layer: dict) -> PartChoice | None:
    mlp = layer.get("mlp")
    if mlp is None:
        return None
    return PartChoice("dense_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": mlp["ff"],
                                    "activation": "relu_squared"})


def leduvik_order(num_layers: int, loop: tuple | None) -> list[LayerRun]:
    """Every pass over the repeated layers but the first begins with the model's join."""
    if loop is None:
        return [LayerRun(i) for i in range(num_layers)]
    start, stop, times = loop
    runs = [LayerRun(i) for i in range(start)]
    for p in range(times):
        runs += [LayerRun(i, enters=(p > 0 and i == start)) for i in range(start, stop)]
    return runs + [LayerRun(i) for i in range(stop, num_layers)]


def leduvik_spec(cfg: LeduvikConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight_name": ""})
    names = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "ffn": "mlp"}
    blocks = [PartChoice("prenorm", {"mixer": _mixer(cfg, layer), "feed_forward": _feed_forward(cfg, layer),
                                     "norm": norm, "names": names}) for layer in cfg.layers]
    order = leduvik_order(len(cfg.layers), cfg.loop)
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, blocks=blocks, final_norm=norm,
        tie_word_embeddings=False,
        embedding=PartChoice("positioned_f32_embedding", {"max_positions": cfg.max_position_embeddings,
                                                          "weight_name": "embed", "position_name": "pos"}),
        head=PartChoice("lm_head", {"weight_name": "", "scale": cfg.logit_scale}),
        order=order, join=PartChoice("add_first") if any(r.enters for r in order) else None,
        max_positions=cfg.max_position_embeddings,
        embedding_prefix="", layer_prefix="l{}", final_norm_prefix="final.norm", head_prefix="head")
