"""Savidra as a ``ModelSpec``.

The stream starts as the token's embedding row, float32 throughout, and is normed after every sum: a layer is
``x <- norm1(alpha x + mixer(shift(x)))``, then ``x <- norm2(alpha x + ff(x))`` where it has a feed-forward, with
RMS norms whose weight the checkpoint stores as its distance from one.  ``shift`` blends a token's row with the
previous token's, entry by entry (``l<i>.shift``).  The mixer is softmax attention with per-head norms of q and k,
rotation of a leading part of every head, a sink per head and, in layers that say so, values blended with those of
the first such layer (``attention``), or two mixers side by side whose outputs are added with a constant each
(``parallel``): attention with biases, short convolutions on q, k and v, stretched positions, a temperature per
head and the heads' weights mixed after the softmax; and a gated delta rule with a decay per key channel, low-rank
decay and gate projections and a sigmoid gate.  The feed-forward is ``W_down (relu(W_gate x) * W_up x)``.  A final
norm of the same kind and an untied head.

Checkpoint names: ``embed``, ``l<i>.norm1`` / ``.norm2`` / ``.shift``, ``l<i>.mix.*``, ``l<i>.mlp.{gate,up,down}``,
``final.norm``, ``head``; matrices carry no ``.weight`` suffix, biases end in ``.b``.
"""

from __future__ import annotations

from ..config.model_config import SavidraConfig
from ..parts.base import PartChoice
from .model import ModelSpec


def _attention(cfg: SavidraConfig, m: dict, **options) -> PartChoice:
    rot = m.get("rot")
    encoding = None
    if rot is not None and rot["dims"] > 0:
        encoding = PartChoice("half_rotary", {"dims": rot["dims"], "base": rot["base"],
                                              "factor": (rot.get("scaling") or {}).get("factor")})
    return PartChoice("together_attention", {
        "hidden_size": cfg.hidden_size, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
        "value_dim": m["vdim"], "scale": m["scale"], "norm_eps": cfg.norm_eps, "qk_norm": True,
        "position_encoding": encoding, **options})


def _mixer(cfg: SavidraConfig, i: int, layer: dict, first_mixing: int | None) -> PartChoice:
    m = layer["mixer"]
    if layer["type"] == "attention":
        mix = None
        if m.get("v_mix"):
            mix = "source" if i == first_mixing else "blend"
        return _attention(cfg, m, sink=True, value_mix=mix)
    left, right = m["left"], m["right"]
    delta = PartChoice("gated_delta", {
        "hidden_size": cfg.hidden_size, "num_heads": right["heads"], "num_kv_heads": right["kv_heads"],
        "head_dim": right["dim"], "value_dim": right["vdim"], "conv_taps": right["conv"], "norm_eps": cfg.norm_eps,
        "decay": "channel", "decay_low_rank": True, "gate_low_rank": True, "gate_activation": "sigmoid",
        # the tensors of a checkpoint say the inner sizes; a configuration may name them for weights that are drawn
        "decay_rank": right.get("decay_rank"), "gate_rank": right.get("gate_rank")})
    return PartChoice("parallel", {
        "hidden_size": cfg.hidden_size, "norm_eps": cfg.norm_eps, "combine": "weighted_sum",
        "scales": [m["left_scale"], m["right_scale"]],
        "branches": [("left", _attention(cfg, left, qkv_bias=True, out_bias=True, conv_taps=left.get("conv"),
                                         head_temperature=True, talk=True)),
                     ("right", delta)]})


def savidra_spec(cfg: SavidraConfig) -> ModelSpec:
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight_name": "", "one_plus": True})
    first_mixing = next((i for i, layer in enumerate(cfg.layers)
                         if layer["type"] == "attention" and layer["mixer"].get("v_mix")), None)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        mlp = layer.get("mlp")
        ffn = None
        if mlp is not None:
            ffn = PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": mlp["ff"],
                                           "activation": "relu", "weight_suffix": "",
                                           "names": {"gate": "gate", "up": "up", "down": "down"}})
        shifted = PartChoice("token_shifted", {"hidden_size": cfg.hidden_size,
                                               "inner": _mixer(cfg, i, layer, first_mixing)})
        blocks.append(PartChoice("normed_sum", {"mixer": shifted, "feed_forward": ffn, "norm": norm,
                                                "alpha": cfg.postln_alpha, "names": {"mixer": ""}}))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, blocks=blocks, final_norm=norm,
        tie_word_embeddings=False,
        embedding=PartChoice("scaled_f32_embedding", {"scale": 1.0, "weight_name": ""}),
        head=PartChoice("lm_head", {"weight_name": ""}),
        max_positions=0, embedding_prefix="embed", layer_prefix="l{}", final_norm_prefix="final.norm", head_prefix="head")
