"""Rotary position encoding: float32 cos/sin tables [max_positions, rotary_dim / 2].

atom/model_ops/rotary_embedding.py:58-80: ``inv_freq_j = base ** (-2j / rotary_dim)``,
``angle = position * inv_freq`` and its cos and sin, all float32.  The reference then
casts the tables to the model's type (:48-50); here they stay float32 and the rotation
is done in float32 by the kernel that also norms q/k and writes the cache.
"""

from __future__ import annotations

import math

import torch

from .base import POSITION_ENCODINGS, PositionEncoding

_TABLES: dict = {}


class RotaryEncoding(PositionEncoding):
    """NeoX-style rotation of the first ``rotary_dim`` elements of each head."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, rotary_dim: int | None = None,
                 prefix: str = ""):
        super().__init__(prefix)
        self.head_dim = head_dim
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not (0 < self.rotary_dim <= head_dim):
            raise ValueError(f"rotary_dim must be even and in (0, head_dim], got {self.rotary_dim}")
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def finalize(self, device, dtype):
        key = (self.rotary_dim, self.theta, self.max_positions, str(device))
        if key not in _TABLES:
            inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim))
            t = torch.arange(self.max_positions, dtype=torch.float32)
            freqs = torch.einsum("i,j->ij", t, inv_freq)
            _TABLES[key] = (freqs.cos().contiguous().to(device), freqs.sin().contiguous().to(device))
        self.cos, self.sin = _TABLES[key]


class ScaledRotary(PositionEncoding):
    """Rotation of interleaved pairs (2i, 2i + 1) of the first ``dims`` entries by ``position * f_i``, with the
    frequencies optionally stretched for contexts longer than the ``original`` one (YaRN; Peng et al., "YaRN:
    Efficient Context Window Extension of Large Language Models"): with ``where(t) = dims * ln(original / (2 pi t))
    / (2 ln base)``, ``lo = max(floor(where(fast)), 0)``, ``hi = min(ceil(where(slow)), dims - 1)`` and ``ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``, pair i turns at ``f_i / factor * ramp_i + f_i * (1 - ramp_i)``
    where ``f_i = base^(-2i / dims)``, and cosine and sine are multiplied by ``0.1 ln(factor) + 1``.

    The kernels form angles in float64 from ``freq`` (float64 [dims / 2]), so there is no table over positions and
    no position limit; ``mult`` is the multiplier of cosine and sine."""

    def __init__(self, dims: int, base: float, factor: float | None = None, original: float | None = None,
                 fast: float | None = None, slow: float | None = None, prefix: str = ""):
        super().__init__(prefix)
        if dims % 2 or dims < 0:
            raise ValueError(f"rotated dimensions come in pairs, got {dims}")
        self.dims = int(dims)
        self.base = float(base)
        self.scaling = None
        if factor is not None:
            if None in (original, fast, slow):
                raise ValueError("stretched rotation needs factor, original, fast and slow")
            self.scaling = (float(factor), float(original), float(fast), float(slow))
        self.freq: torch.Tensor | None = None
        self.mult = 1.0

    def frequencies(self) -> tuple[torch.Tensor, float]:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(self.dims, 1))
        if self.scaling is None:
            return f, 1.0
        factor, original, fast, slow = self.scaling

        def where(turns: float) -> float:
            return self.dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(self.base))

        lo = max(math.floor(where(fast)), 0)
        hi = min(math.ceil(where(slow)), self.dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0

    def finalize(self, device, dtype):
        freq, self.mult = self.frequencies()
        self.freq = freq.to(device)


class BandedRotary(PositionEncoding):
    """Rotation of interleaved pairs (2i, 2i + 1) of the first ``dims`` entries by ``position * f_i``,
    ``f_i = base^(-2i / dims)``, with the frequencies scaled by the band their wavelength ``l = 2 pi / f`` falls in
    (the scheme of the Llama 3.1 models): unchanged where ``l < original / high``, divided by ``factor`` where
    ``l > original / low``, and between the two ``(1 - s) f / factor + s f`` with ``s = (original / l - low) /
    (high - low)``.  Without ``factor`` the frequencies are plain.

    Offers what ``ScaledRotary`` offers: ``freq`` (float64 [dims / 2], on the device), ``mult`` (1 here) and
    ``dims``; kernels form the angle in float64 from the position, so there is no table and no position limit."""

    def __init__(self, dims: int, base: float, factor: float | None = None, low: float | None = None,
                 high: float | None = None, original: float | None = None, head_dim: int | None = None,
                 prefix: str = ""):
        super().__init__(prefix)
        if dims % 2 or dims < 0 or (head_dim is not None and dims > head_dim):
            raise ValueError(f"rotated dimensions come in pairs within a head, got {dims}")
        self.dims = int(dims)
        self.base = float(base)
        self.scaling = None
        if factor is not None:
            if None in (low, high, original):
                raise ValueError("banded scaling needs factor, low, high and original")
            if float(high) == float(low):
                raise ValueError("banded scaling needs high and low to differ")
            self.scaling = (float(factor), float(low), float(high), float(original))
        self.freq: torch.Tensor | None = None
        self.mult = 1.0

    def frequencies(self) -> torch.Tensor:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(self.dims, 1))
        if self.scaling is None:
            return f
        factor, low, high, original = self.scaling
        length = 2 * math.pi / f
        s = (original / length - low) / (high - low)
        between = (1 - s) * f / factor + s * f
        return torch.where(length < original / high, f, torch.where(length > original / low, f / factor, between))

    def finalize(self, device, dtype):
        self.freq = self.frequencies().to(device)


class HalfRotary(PositionEncoding):
    """Rotation of the pairs (i, i + dims / 2) of the first ``dims`` entries of a head by ``position * f_i``,
    ``f_i = base^(-2i / dims) / factor`` (``factor``: positions stretched linearly; None: 1).  Offers what
    ``ScaledRotary`` offers (``freq`` float64 [dims / 2] on the device, ``mult``, ``dims``): kernels form the angle
    in float64 from the position, so there is no table and no position limit."""

    def __init__(self, dims: int, base: float, factor: float | None = None, head_dim: int | None = None,
                 prefix: str = ""):
        super().__init__(prefix)
        if dims % 2 or dims < 0 or (head_dim is not None and dims > head_dim):
            raise ValueError(f"rotated dimensions come in pairs within a head, got {dims}")
        if factor is not None and not float(factor) > 0:
            raise ValueError("the stretch of positions must be positive")
        self.dims, self.base = int(dims), float(base)
        self.factor = float(factor) if factor is not None else 1.0
        self.freq: torch.Tensor | None = None
        self.mult = 1.0

    def frequencies(self) -> torch.Tensor:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        return self.base ** (-2.0 * i / max(self.dims, 1)) / self.factor

    def finalize(self, device, dtype):
        self.freq = self.frequencies().to(device)


POSITION_ENCODINGS.register("half_rotary", HalfRotary)
POSITION_ENCODINGS.register("rotary", RotaryEncoding)
POSITION_ENCODINGS.register("scaled_rotary", ScaledRotary)
POSITION_ENCODINGS.register("banded_rotary", BandedRotary)
