"""Typed model configurations read from a checkpoint's own ``config.json`` keys.

Every size and constant a model needs comes from here; no model code holds one.
The fields and fallbacks follow what ATOM reads from the HF config for
``Qwen3ForCausalLM`` (atom/models/qwen3.py:211-239, atom/config.py:1708-1753).
"""

from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that cannot describe a model this engine can run."""


_MISSING = object()


def _take(raw: dict, key: str, kind, default=_MISSING):
    if key not in raw or raw[key] is None:
        if default is _MISSING:
            raise ConfigError(f"config.json lacks the required key '{key}'")
        return default
    value = raw[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if kind is int and isinstance(value, bool) or not isinstance(value, kind):
        raise ConfigError(f"config.json key '{key}' must be {kind.__name__}, got {value!r}")
    return value


@dataclass(frozen=True)
class ModelConfig:
    """What every architecture's configuration has in common."""

    architecture: str
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    torch_dtype: str
    bos_token_id: int | None
    eos_token_id: int | list[int] | None

    #: keys of config.json each subclass understands, for the round trip in to_dict()
    model_type: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: dict) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> dict:
        raise NotImplementedError

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)

    def replace(self, **changes) -> "ModelConfig":
        return type(self).from_dict({**self.to_dict(), **changes})


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    """``Qwen3ForCausalLM``: grouped-query attention with per-head q/k norms, rotary
    positions, a SiLU-gated dense feed-forward and RMS norms."""

    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    hidden_act: str = "silu"
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    attention_bias: bool = False
    use_sliding_window: bool = False
    sliding_window: int | None = None
    layer_types: tuple[str, ...] | None = None

    model_type: ClassVar[str] = "qwen3"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        archs = raw.get("architectures") or [None]
        hidden = _take(raw, "hidden_size", int)
        heads = _take(raw, "num_attention_heads", int)
        # atom/models/qwen3.py:85,221: head_dim falls back to hidden_size // heads
        head_dim = _take(raw, "head_dim", int, hidden // heads)
        # atom/config.py:1708-1722: rope_theta may live under rope_parameters
        rope = raw.get("rope_parameters") or {}
        theta = rope.get("rope_theta", raw.get("rope_theta"))
        if theta is None:
            raise ConfigError("config.json lacks 'rope_theta' (or rope_parameters.rope_theta)")
        scaling = raw.get("rope_scaling")
        rope_type = (scaling or {}).get("rope_type", (scaling or {}).get("type", rope.get("rope_type", "default")))
        if rope_type not in ("default", None):
            raise ConfigError(f"rope scaling of type {rope_type!r} is not supported for {archs[0]}")
        layers = _take(raw, "num_hidden_layers", int)
        layer_types = raw.get("layer_types")
        if layer_types is not None:
            layer_types = tuple(layer_types)
        cfg = cls(
            architecture=archs[0] or "Qwen3ForCausalLM",
            vocab_size=_take(raw, "vocab_size", int),
            hidden_size=hidden,
            num_hidden_layers=layers,
            # atom/config.py:1745-1753: 8192 when the checkpoint names none
            max_position_embeddings=_take(raw, "max_position_embeddings", int, 8192),
            tie_word_embeddings=_take(raw, "tie_word_embeddings", bool, False),
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            num_attention_heads=heads,
            num_key_value_heads=_take(raw, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            intermediate_size=_take(raw, "intermediate_size", int),
            hidden_act=_take(raw, "hidden_act", str, "silu"),
            rms_norm_eps=_take(raw, "rms_norm_eps", float, 1e-6),
            rope_theta=float(theta),
            attention_bias=_take(raw, "attention_bias", bool, False),
            use_sliding_window=_take(raw, "use_sliding_window", bool, False),
            sliding_window=raw.get("sliding_window"),
            layer_types=layer_types,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        def positive(name):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")

        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            positive(name)
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim must be even for rotary pairs, got {self.head_dim}")
        if self.hidden_act != "silu":  # atom/models/qwen3.py:191
            raise ConfigError(f"hidden_act must be 'silu', got {self.hidden_act!r}")
        if self.rms_norm_eps <= 0:
            raise ConfigError("rms_norm_eps must be positive")
        if self.layer_types is not None and len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(
                f"layer_types has {len(self.layer_types)} entries for {self.num_hidden_layers} layers")
        if self.use_sliding_window and self.layer_types and "sliding_attention" in self.layer_types:
            if not self.sliding_window or self.sliding_window <= 0:
                raise ConfigError("sliding layers need a positive sliding_window")

    def window_of_layer(self, layer: int) -> int | None:
        """The attention window of a layer or None for all keys: ``layer_types`` read
        as atom/models/llama.py:187-191 does, and only when ``use_sliding_window``."""
        if self.use_sliding_window and self.layer_types and self.layer_types[layer] == "sliding_attention":
            return self.sliding_window
        return None

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": self.model_type,
        }
        for f in dataclasses.fields(self):
            if f.name == "architecture":
                continue
            value = getattr(self, f.name)
            if isinstance(value, tuple):
                value = list(value)
            out[f.name] = value
        return out


def _need(raw: dict, key: str, kind, where: str):
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ConfigError(f"config.json lacks '{key}' in {where}")
    value = raw[key]
    if kind is float and isinstance(value, int) and not isinstance(value, bool):
        value = float(value)
    if (kind is int and isinstance(value, bool)) or not isinstance(value, kind):
        raise ConfigError(f"config.json: '{key}' in {where} must be {kind.__name__}, got {value!r}")
    return value


@dataclass(frozen=True)
class LotoraxConfig(ModelConfig):
    """``Lotorax``: layers listed one by one, each a mixer (attention over cached latents, or the gated delta
    rule) and an optional feed-forward (dense, or routed experts) between layer norms; a run of layers may be
    repeated with the same weights.  config.json keys: ``vocab``, ``width``, ``embedding.scale``, ``norm.eps``,
    ``layers`` (``type``, ``mixer``, ``mlp``), ``loop`` (``start``, ``stop``, ``times``)."""

    layers: tuple = ()                # the entries of config.json's 'layers', as they are
    loop: tuple | None = None         # (start, stop, times)
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0

    model_type: ClassVar[str] = "lotorax"
    MIXER_TYPES: ClassVar[tuple] = ("latent_attention", "delta")
    MLP_KINDS: ClassVar[tuple] = ("dense", "moe")

    @classmethod
    def from_dict(cls, raw: dict) -> "LotoraxConfig":
        layers = _need(raw, "layers", list, "the model")
        loop = raw.get("loop")
        if loop is not None:
            loop = tuple(_need(loop, k, int, "'loop'") for k in ("start", "stop", "times"))
        cfg = cls(
            architecture=raw.get("architecture") or (raw.get("architectures") or ["Lotorax"])[0],
            vocab_size=_need(raw, "vocab", int, "the model"),
            hidden_size=_need(raw, "width", int, "the model"),
            num_hidden_layers=len(layers),
            # the design names no position limit: angles are formed from positions as they come
            max_position_embeddings=_take(raw, "max_position_embeddings", int, 1 << 20),
            tie_word_embeddings=False,
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            layers=tuple(layers),
            loop=loop,
            norm_eps=_need(raw.get("norm"), "eps", float, "'norm'"),
            embedding_scale=_need(raw.get("embedding"), "scale", float, "'embedding'"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind not in self.MIXER_TYPES:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {self.MIXER_TYPES}")
            m = _need(layer, "mixer", dict, where)
            if kind == "latent_attention":
                for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank"):
                    if _need(m, key, int, f"{where}'s mixer") <= 0:
                        raise ConfigError(f"{where}: {key} must be positive")
                _need(m, "scale", float, f"{where}'s mixer")
                rot = _need(m, "rot", dict, f"{where}'s mixer")
                dims = _need(rot, "dims", int, f"{where}'s rot")
                _need(rot, "base", float, f"{where}'s rot")
                if dims % 2 or dims > m["rot_dim"]:
                    raise ConfigError(f"{where}: rot.dims must be even and at most rot_dim")
                if rot.get("scaling") is not None:
                    for key in ("factor", "original", "fast", "slow"):
                        _need(rot["scaling"], key, float, f"{where}'s rot.scaling")
            else:
                for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    if _need(m, key, int, f"{where}'s mixer") <= 0:
                        raise ConfigError(f"{where}: {key} must be positive")
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", str, f"{where}'s mlp")
                if mk not in self.MLP_KINDS:
                    raise ConfigError(f"{where}: unknown mlp kind {mk!r}; known: {self.MLP_KINDS}")
                if mk == "dense":
                    _need(mlp, "ff", int, f"{where}'s mlp")
                else:
                    _need(_need(mlp, "expert", dict, f"{where}'s mlp"), "ff", int, f"{where}'s mlp.expert")
                    router = _need(mlp, "router", dict, f"{where}'s mlp")
                    if not 0 < _need(router, "top", int, f"{where}'s router") <= _need(router, "experts", int, f"{where}'s router"):
                        raise ConfigError(f"{where}: the router's top must lie in 1 .. experts")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times < 1:
                raise ConfigError(f"loop {self.loop} does not fit {len(self.layers)} layers")

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architecture": self.architecture, "model_type": self.model_type, "vocab": self.vocab_size,
            "width": self.hidden_size, "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": [dict(layer) for layer in self.layers],
        }
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.max_position_embeddings != 1 << 20:
            out["max_position_embeddings"] = self.max_position_embeddings
        for key in ("bos_token_id", "eos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out


@dataclass(frozen=True)
class RalitarConfig(ModelConfig):
    """``Ralitar``: a token embedding plus a hashed bigram embedding; layers listed one by one, each a mixer (a
    real-gated linear recurrence, the gated delta rule with a decay per key channel, or chunked attention whose
    values are its keys) and an optional dense feed-forward, RMS-normed on their way into the stream, then a small
    per-layer input that depends on the token itself.  config.json keys: ``vocab``, ``width``, ``norm.eps``,
    ``embedding.bigram`` (``buckets``, ``mul_prev``, ``mul_cur``), ``token_side.dim``, ``layers`` (``type``,
    ``mixer``, ``mlp``)."""

    layers: tuple = ()
    norm_eps: float = 1e-6
    bigram: tuple | None = None       # (buckets, mul_prev, mul_cur)
    side_dim: int = 0                 # columns of the per-layer token input (0: the model has none)

    model_type: ClassVar[str] = "ralitar"
    MIXER_TYPES: ClassVar[tuple] = ("rglru", "channel_delta", "attention")
    MLP_KINDS: ClassVar[tuple] = ("dense",)

    @classmethod
    def from_dict(cls, raw: dict) -> "RalitarConfig":
        layers = _need(raw, "layers", list, "the model")
        bigram = (raw.get("embedding") or {}).get("bigram")
        if bigram is not None:
            bigram = tuple(_need(bigram, k, int, "'embedding.bigram'") for k in ("buckets", "mul_prev", "mul_cur"))
        side = raw.get("token_side")
        cfg = cls(
            architecture=raw.get("architecture") or (raw.get("architectures") or ["Ralitar"])[0],
            vocab_size=_need(raw, "vocab", int, "the model"),
            hidden_size=_need(raw, "width", int, "the model"),
            num_hidden_layers=len(layers),
            max_position_embeddings=_take(raw, "max_position_embeddings", int, 1 << 20),
            tie_word_embeddings=False,
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            layers=tuple(layers),
            norm_eps=_need(raw.get("norm"), "eps", float, "'norm'"),
            bigram=bigram,
            side_dim=_need(side, "dim", int, "'token_side'") if side is not None else 0,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")
        if self.bigram is not None and self.bigram[0] <= 0:
            raise ConfigError("embedding.bigram.buckets must be positive")
        if self.side_dim < 0:
            raise ConfigError("token_side.dim must not be negative")

        def positive(m, keys, where):
            for key in keys:
                if _need(m, key, int, where) <= 0:
                    raise ConfigError(f"{where}: {key} must be positive")

        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind not in self.MIXER_TYPES:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {self.MIXER_TYPES}")
            m = _need(layer, "mixer", dict, where)
            mw = f"{where}'s mixer"
            if kind == "rglru":
                positive(m, ("width", "blocks", "conv"), mw)
                if m["width"] % m["blocks"]:
                    raise ConfigError(f"{where}: width must be a multiple of blocks")
            elif kind == "channel_delta":
                positive(m, ("heads", "kv_heads", "dim", "vdim", "conv"), mw)
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
            else:
                positive(m, ("heads", "kv_heads", "dim", "vdim"), mw)
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
                if m["vdim"] != m["dim"]:
                    raise ConfigError(f"{where}: the values are the keys, so vdim must equal dim")
                _need(m, "scale", float, mw)
                if m.get("softcap") is not None and _need(m, "softcap", float, mw) <= 0:
                    raise ConfigError(f"{where}: softcap must be positive")
                mask = m.get("mask")
                if mask is not None and _need(mask, "size", int, f"{where}'s mask") <= 0:
                    raise ConfigError(f"{where}: mask.size must be positive")
                rot = m.get("rot")
                if rot is not None:
                    dims = _need(rot, "dims", int, f"{where}'s rot")
                    _need(rot, "base", float, f"{where}'s rot")
                    if dims % 2 or dims < 0 or dims > m["dim"]:
                        raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                    if rot.get("scaling") is not None:
                        for key in ("factor", "low", "high", "original"):
                            _need(rot["scaling"], key, float, f"{where}'s rot.scaling")
                        if rot["scaling"]["high"] == rot["scaling"]["low"]:
                            raise ConfigError(f"{where}: rot.scaling needs high and low to differ")
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", str, f"{where}'s mlp")
                if mk not in self.MLP_KINDS:
                    raise ConfigError(f"{where}: unknown mlp kind {mk!r}; known: {self.MLP_KINDS}")
                positive(mlp, ("ff",), f"{where}'s mlp")

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architecture": self.architecture, "model_type": self.model_type, "vocab": self.vocab_size,
            "width": self.hidden_size, "norm": {"eps": self.norm_eps},
            "layers": [dict(layer) for layer in self.layers],
        }
        if self.bigram is not None:
            out["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.max_position_embeddings != 1 << 20:
            out["max_position_embeddings"] = self.max_position_embeddings
        for key in ("bos_token_id", "eos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out


@dataclass(frozen=True)
class LeduvikConfig(ModelConfig):
    """``Leduvik``: token rows plus learned position rows; pre-norm layers listed one by one, each a mixer (a
    selective state-space recurrence, windowed attention with unit-norm queries and keys, or attention and a
    time-mixing recurrence side by side) and an optional dense feed-forward; a run of layers may be passed several
    times, the embedding's output joining the stream again before every pass but the first.  config.json keys:
    ``vocab``, ``width``, ``max_positions``, ``norm.eps``, ``logit_scale``, ``layers`` (``type``, ``mixer``,
    ``mlp``), ``loop`` (``start``, ``stop``, ``times``)."""

    layers: tuple = ()
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    loop: tuple | None = None         # (start, stop, times)

    model_type: ClassVar[str] = "leduvik"
    MIXER_TYPES: ClassVar[tuple] = ("mamba2", "attention", "parallel")
    MLP_KINDS: ClassVar[tuple] = ("dense",)

    @classmethod
    def from_dict(cls, raw: dict) -> "LeduvikConfig":
        layers = [cls._with_defaults(layer) for layer in _need(raw, "layers", list, "the model")]
        loop = raw.get("loop")
        if loop is not None:
            loop = tuple(_need(loop, k, int, "'loop'") for k in ("start", "stop", "times"))
            if loop[0] == loop[1] or loop[2] == 1:
                loop = None           # an empty run of layers, or a single pass: nothing is repeated
        cfg = cls(
            architecture=raw.get("architecture") or (raw.get("architectures") or ["Leduvik"])[0],
            vocab_size=_need(raw, "vocab", int, "the model"),
            hidden_size=_need(raw, "width", int, "the model"),
            num_hidden_layers=len(layers),
            max_position_embeddings=_need(raw, "max_positions", int, "the model"),
            tie_word_embeddings=False,
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            layers=tuple(layers),
            norm_eps=_need(raw.get("norm"), "eps", float, "'norm'"),
            logit_scale=_take(raw, "logit_scale", float, 1.0),
            loop=loop,
        )
        cfg.validate()
        return cfg

    @staticmethod
    def _with_defaults(layer):
        """A layer's entry with the sizes that have an obvious value where the file leaves them out: as many
        key/value heads as query heads, values of the keys' size, one group, one norm part."""
        if not isinstance(layer, dict) or not isinstance(layer.get("mixer"), dict):
            return layer

        def attention(m):
            m = dict(m)
            if "heads" in m:
                m.setdefault("kv_heads", m["heads"])
            if "dim" in m:
                m.setdefault("vdim", m["dim"])
            return m

        layer, m = dict(layer), dict(layer["mixer"])
        if layer.get("type") == "mamba2":
            m.setdefault("groups", 1)
            m.setdefault("norm_groups", 1)
        elif layer.get("type") == "attention":
            m = attention(m)
        elif layer.get("type") == "parallel" and isinstance(m.get("left"), dict):
            m["left"] = attention(m["left"])
        layer["mixer"] = m
        return layer

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.max_position_embeddings <= 0:
            raise ConfigError("max_positions must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")

        def positive(m, keys, where):
            for key in keys:
                if _need(m, key, int, where) <= 0:
                    raise ConfigError(f"{where}: {key} must be positive")

        def attention(m, where):
            positive(m, ("heads", "kv_heads", "dim", "vdim"), where)
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
            _need(m, "scale", float, where)
            mask = m.get("mask")
            if mask is not None and _need(mask, "size", int, f"{where}'s mask") <= 0:
                raise ConfigError(f"{where}: mask.size must be positive")
            temp = m.get("q_temp")
            if temp is not None:
                _need(temp, "coef", float, f"{where}'s q_temp")
                if _need(temp, "every", int, f"{where}'s q_temp") <= 0:
                    raise ConfigError(f"{where}: q_temp.every must be positive")

        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind not in self.MIXER_TYPES:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {self.MIXER_TYPES}")
            m = _need(layer, "mixer", dict, where)
            mw = f"{where}'s mixer"
            if kind == "mamba2":
                positive(m, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), mw)
                if m["heads"] % m["groups"]:
                    raise ConfigError(f"{where}: heads must be a multiple of groups")
                if (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ConfigError(f"{where}: heads * vdim must be a multiple of norm_groups")
            elif kind == "attention":
                attention(m, mw)
            else:
                attention(_need(m, "left", dict, mw), f"{mw}'s left")
                positive(_need(m, "right", dict, mw), ("heads", "dim"), f"{mw}'s right")
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", str, f"{where}'s mlp")
                if mk not in self.MLP_KINDS:
                    raise ConfigError(f"{where}: unknown mlp kind {mk!r}; known: {self.MLP_KINDS}")
                positive(mlp, ("ff",), f"{where}'s mlp")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times < 1:
                raise ConfigError(f"loop {self.loop} does not fit {len(self.layers)} layers")

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architecture": self.architecture, "model_type": self.model_type, "vocab": self.vocab_size,
            "width": self.hidden_size, "max_positions": self.max_position_embeddings, "norm": {"eps": self.norm_eps},
            "logit_scale": self.logit_scale, "layers": [dict(layer) for layer in self.layers],
        }
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        for key in ("bos_token_id", "eos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out


@dataclass(frozen=True)
class SavidraConfig(ModelConfig):
    """``Savidra``: token rows start a float32 stream that is normed after every sum, ``x <- norm(alpha x +
    sublayer(x))``; the mixer reads a blend of a token's row and the previous token's; layers are listed one by
    one, each softmax attention with a sink per head and values blended with an earlier layer's (``attention``)
    or attention behind short convolutions, with a temperature per head and the heads' weights mixed, side by side
    with a gated delta rule (``parallel``), and an optional ReLU-gated dense feed-forward.  config.json keys:
    ``vocab``, ``width``, ``norm.eps``, ``postln_alpha``, ``layers`` (``type``, ``mixer``, ``mlp``)."""

    layers: tuple = ()
    norm_eps: float = 1e-6
    postln_alpha: float = 1.0

    model_type: ClassVar[str] = "savidra"
    MIXER_TYPES: ClassVar[tuple] = ("attention", "parallel")
    MLP_KINDS: ClassVar[tuple] = ("dense",)

    @classmethod
    def from_dict(cls, raw: dict) -> "SavidraConfig":
        layers = [cls._with_defaults(layer) for layer in _need(raw, "layers", list, "the model")]
        cfg = cls(
            architecture=raw.get("architecture") or (raw.get("architectures") or ["Savidra"])[0],
            vocab_size=_need(raw, "vocab", int, "the model"),
            hidden_size=_need(raw, "width", int, "the model"),
            num_hidden_layers=len(layers),
            max_position_embeddings=_take(raw, "max_position_embeddings", int, 1 << 20),
            tie_word_embeddings=False,
            torch_dtype=str(raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            layers=tuple(layers),
            norm_eps=_need(raw.get("norm"), "eps", float, "'norm'"),
            postln_alpha=_take(raw, "postln_alpha", float, 1.0),
        )
        cfg.validate()
        return cfg

    @staticmethod
    def _with_defaults(layer):
        """As many key/value heads as query heads and values of the keys' size where an entry leaves them out."""
        if not isinstance(layer, dict) or not isinstance(layer.get("mixer"), dict):
            return layer

        def heads(m):
            m = dict(m)
            if "heads" in m:
                m.setdefault("kv_heads", m["heads"])
            if "dim" in m:
                m.setdefault("vdim", m["dim"])
            return m

        layer, m = dict(layer), dict(layer["mixer"])
        if layer.get("type") == "attention":
            m = heads(m)
        elif layer.get("type") == "parallel":
            for side in ("left", "right"):
                if isinstance(m.get(side), dict):
                    m[side] = heads(m[side])
        layer["mixer"] = m
        return layer

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or not self.layers:
            raise ConfigError("vocab, width and the number of layers must be positive")
        if self.norm_eps <= 0:
            raise ConfigError("norm.eps must be positive")

        def positive(m, keys, where):
            for key in keys:
                if _need(m, key, int, where) <= 0:
                    raise ConfigError(f"{where}: {key} must be positive")

        def heads(m, where):
            positive(m, ("heads", "kv_heads", "dim", "vdim"), where)
            if m["heads"] % m["kv_heads"]:
                raise ConfigError(f"{where}: heads must be a multiple of kv_heads")

        def attention(m, where):
            heads(m, where)
            _need(m, "scale", float, where)
            rot = m.get("rot")
            if rot is not None:
                dims = _need(rot, "dims", int, f"{where}'s rot")
                _need(rot, "base", float, f"{where}'s rot")
                if dims % 2 or dims < 0 or dims > m["dim"]:
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                if rot.get("scaling") is not None and _need(rot["scaling"], "factor", float, f"{where}'s rot.scaling") <= 0:
                    raise ConfigError(f"{where}: rot.scaling.factor must be positive")
            if m.get("conv") is not None and _need(m, "conv", int, where) <= 0:
                raise ConfigError(f"{where}: conv must be positive")

        mixed_values = None
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            kind = _need(layer, "type", str, where)
            if kind not in self.MIXER_TYPES:
                raise ConfigError(f"{where}: unknown type {kind!r}; known: {self.MIXER_TYPES}")
            m = _need(layer, "mixer", dict, where)
            mw = f"{where}'s mixer"
            if kind == "attention":
                attention(m, mw)
                if m.get("v_mix"):
                    size = (m["kv_heads"], m["vdim"])
                    if mixed_values is not None and size != mixed_values:
                        raise ConfigError(f"{where}: layers that blend their values need value heads of one number and size")
                    mixed_values = size
            else:
                attention(_need(m, "left", dict, mw), f"{mw}'s left")
                right = _need(m, "right", dict, mw)
                heads(right, f"{mw}'s right")
                positive(right, ("conv",), f"{mw}'s right")
                for key in ("left_scale", "right_scale"):
                    _need(m, key, float, mw)
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = _need(mlp, "kind", str, f"{where}'s mlp")
                if mk not in self.MLP_KINDS:
                    raise ConfigError(f"{where}: unknown mlp kind {mk!r}; known: {self.MLP_KINDS}")
                positive(mlp, ("ff",), f"{where}'s mlp")

    def to_dict(self) -> dict:
        out: dict[str, Any] = {
            "architecture": self.architecture, "model_type": self.model_type, "vocab": self.vocab_size,
            "width": self.hidden_size, "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha,
            "layers": [dict(layer) for layer in self.layers],
        }
        if self.max_position_embeddings != 1 << 20:
            out["max_position_embeddings"] = self.max_position_embeddings
        for key in ("bos_token_id", "eos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder!r}")
    with open(path) as f:
        return json.load(f)
