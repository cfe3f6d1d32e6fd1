"""Rotary position encoding: the tables.

``inv_freq[i] = 1 / theta^(2i/dim)``, ``angle[p, i] = p * inv_freq[i]`` in float32,
``cos``/``sin`` of the angles, cast to the activation dtype (reference:
engine/dryft_qwen3/model.py:49-57). The reference stores ``cat(angle, angle)``; its two
halves are equal, so only ``[positions, dim/2]`` is kept here. The rotation itself
(pairs ``(j, j + dim/2)``, model.py:35-41) is applied by the attention part's fused kernel.
Tables are made once on the host with the float32 routines any plain implementation
would use, then uploaded.
"""

from __future__ import annotations

import math

import torch

from . import register_part
from .base import PositionEncoding


class RotaryPositions(PositionEncoding):
    def __init__(self, dim: int, theta: float):
        if dim % 2:
            raise ValueError(f"rotary width must be even, got {dim}")
        self.dim, self.theta = int(dim), float(theta)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.n_positions = 0

    def prepare(self, n_positions: int, dtype: torch.dtype, device) -> None:
        if self.cos is not None and n_positions <= self.n_positions and self.cos.dtype == dtype:
            return
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.dim, 2, dtype=torch.int64).to(torch.float32) / self.dim))
        pos = torch.arange(n_positions, dtype=torch.float32)
        angle = pos[:, None] * inv_freq[None, :]
        self.cos = angle.cos().to(dtype).to(device).contiguous()
        self.sin = angle.sin().to(dtype).to(device).contiguous()
        self.n_positions = n_positions


class PairRotaryPositions(PositionEncoding):
    """Rotary tables for a rotation over neighbouring pairs ``(2i, 2i + 1)`` of the first ``dims`` features, kept in
    float32 whatever the activation dtype: ``cos``/``sin`` are ``[positions, dims / 2]`` of the angles
    ``p * f_i``, ``f_i = base^(-2i / dims)``.

    With ``scaling`` (YaRN: ``factor``, ``original`` context length, ``fast`` and ``slow`` turn counts) the slow
    pairs are stretched and the fast ones left alone: with ``d(t) = dims * ln(original / (2 pi t)) / (2 ln base)``,
    ``lo = max(floor(d(fast)), 0)``, ``hi = min(ceil(d(slow)), dims - 1)`` and
    ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)`` the frequency becomes
    ``f_i / factor * ramp_i + f_i * (1 - ramp_i)``, and cos and sin are both multiplied by ``0.1 ln(factor) + 1``
    (the tables carry that factor). Angles are formed in float64 on the host and rounded once."""

    def __init__(self, dims: int, base: float, scaling: dict | None = None):
        if dims % 2 or dims < 0:
            raise ValueError(f"the rotated width must be even, got {dims}")
        self.dims, self.base = int(dims), float(base)
        self.scaling = dict(scaling) if scaling else None
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.n_positions = 0

    def frequencies(self) -> tuple[torch.Tensor, float]:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / max(self.dims, 1))
        if not self.scaling:
            return f, 1.0
        factor, original = float(self.scaling["factor"]), float(self.scaling["original"])

        def pair_of(turns: float) -> float:
            return self.dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(self.base))

        lo = max(math.floor(pair_of(float(self.scaling["fast"]))), 0)
        hi = min(math.ceil(pair_of(float(self.scaling["slow"]))), self.dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0

    def prepare(self, n_positions: int, dtype: torch.dtype, device) -> None:
        if self.cos is not None and n_positions <= self.n_positions:
            return
        f, both = self.frequencies()
        angle = torch.arange(n_positions, dtype=torch.float64)[:, None] * f[None, :]
        self.cos = (angle.cos() * both).to(torch.float32).to(device).contiguous()
        self.sin = (angle.sin() * both).to(torch.float32).to(device).contiguous()
        self.n_positions = n_positions


class HalfRotaryPositions(PositionEncoding):
    """Float32 tables for a rotation that pairs feature ``i`` with feature ``i + dims/2`` of the first ``dims``
    features of a vector: ``cos``/``sin`` are ``[positions, dims / 2]`` of the angles ``p * f_i``,
    ``f_i = base^(-2i / dims)``, formed in float64 on the host and rounded once, whatever the activation dtype.

    With ``scaling`` (``factor``, ``low``, ``high``, ``original``: the wavelength rule of Llama 3.1) a frequency whose
    wavelength ``l = 2 pi / f`` is shorter than ``original / high`` stays, one whose wavelength is longer than
    ``original / low`` becomes ``f / factor``, and between the two, with ``s = (original / l - low) / (high - low)``,
    it becomes ``(1 - s) f / factor + s f``."""

    def __init__(self, dims: int, base: float, scaling: dict | None = None):
        if dims % 2 or dims <= 0:
            raise ValueError(f"the rotated width must be even and positive, got {dims}")
        self.dims, self.base = int(dims), float(base)
        self.scaling = dict(scaling) if scaling else None
        if self.scaling:
            missing = [k for k in ("factor", "low", "high", "original") if k not in self.scaling]
            if missing or float(self.scaling["high"]) == float(self.scaling["low"]):
                raise ValueError(f"frequency scaling needs factor, low, high (not equal) and original; got {self.scaling}")
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.n_positions = 0

    def frequencies(self) -> torch.Tensor:
        f = self.base ** (-2.0 * torch.arange(self.dims // 2, dtype=torch.float64) / self.dims)
        if not self.scaling:
            return f
        factor, low, high, original = (float(self.scaling[k]) for k in ("factor", "low", "high", "original"))
        wave = 2.0 * math.pi / f
        blend = ((original / wave - low) / (high - low))
        mixed = (1.0 - blend) * f / factor + blend * f
        return torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor, mixed))

    def prepare(self, n_positions: int, dtype: torch.dtype, device) -> None:
        if self.cos is not None and n_positions <= self.n_positions:
            return
        angle = torch.arange(n_positions, dtype=torch.float64)[:, None] * self.frequencies()[None, :]
        self.cos = angle.cos().to(torch.float32).to(device).contiguous()
        self.sin = angle.sin().to(torch.float32).to(device).contiguous()
        self.n_positions = n_positions


register_part("rotary", RotaryPositions)
register_part("half_rotary", HalfRotaryPositions)
register_part("pair_rotary", PairRotaryPositions)
