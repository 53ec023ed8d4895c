"""Position encodings.

``rope_interleaved``: rotary embedding over adjacent pairs ``(x[2j], x[2j+1])``
(``llama4/llama4_jax/model.py:722-728``) with frequencies
``theta ** -(2j / head_dim)`` (``model.py:706-708``) and, if the configuration has
``rope_scaling``, the llama3 correction (``model.py:654-672``).  Angles are formed
in float32 from integer positions inside the kernel (``model.py:710-718``: a
reduced-precision product here is catastrophic); this part says, as data, which
frequencies there are, which elements pair up and how many of a head are rotated.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import PositionEncoding, Rotation, register_position


@register_position("none")
class NoPosition(PositionEncoding):
    pass


def llama3_scaled_frequencies(inv_freq: torch.Tensor, factor: float, low_freq_factor: float,
                              high_freq_factor: float, original_max_position_embeddings: int) -> torch.Tensor:
    """Wavelengths above ``orig / low`` are stretched by ``factor``; those below
    ``orig / high`` are kept; between, the two are blended linearly in
    ``orig / wavelength``.  With ``low == high`` there is no band between."""
    old = float(original_max_position_embeddings)
    low_wl = old / low_freq_factor
    high_wl = old / high_freq_factor
    wavelen = 2.0 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_wl, inv_freq / factor, inv_freq)
    if high_freq_factor != low_freq_factor:
        smooth = (old / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        blended = (1.0 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < high_wl) & ~(wavelen > low_wl)
        scaled = torch.where(medium, blended, scaled)
    return scaled


@register_position("rope_interleaved")
class RopeInterleaved(PositionEncoding):
    def inv_freq(self) -> Optional[torch.Tensor]:
        dh = self.head_dim
        fraction = torch.arange(0, dh, 2, dtype=torch.float32) / dh
        inv = 1.0 / (torch.tensor(float(self.spec.theta), dtype=torch.float32) ** fraction)
        scaling = self.spec.get("scaling")
        if scaling:
            inv = llama3_scaled_frequencies(
                inv,
                float(scaling["factor"]),
                float(scaling["low_freq_factor"]),
                float(scaling["high_freq_factor"]),
                int(scaling["original_max_position_embeddings"]),
            )
        return inv.to(torch.float32)

    def rotation(self) -> Rotation:
        return Rotation(self.inv_freq(), pairing="adjacent", rotary_dim=self.head_dim)


@register_position("rope_half")
class RopeHalf(PositionEncoding):
    """Rotary embedding over half-split pairs: element ``j`` pairs with ``j + rotary_dim / 2`` for ``j`` below
    ``rotary_dim / 2``; the pair ``(u, v)`` at position ``p`` becomes ``(u cos a - v sin a, v cos a + u sin a)``
    with ``a = p * theta ** (-2 j / rotary_dim)``.  ``rotary_dim`` leading elements of the vector turn (default:
    all), the rest pass unchanged."""

    def rotation(self) -> Rotation:
        rd = int(self.spec.get("rotary_dim") or self.head_dim)
        if rd % 2 or not 0 < rd <= self.head_dim:
            raise ValueError(f"rotary_dim must be even and at most {self.head_dim}, got {rd}")
        j = torch.arange(0, rd // 2, dtype=torch.float64)
        inv = torch.tensor(float(self.spec.theta), dtype=torch.float64) ** (-2.0 * j / rd)
        return Rotation(inv.to(torch.float32), pairing="half", rotary_dim=rd)


def yarn_scaled_frequencies(inv_freq: torch.Tensor, base: float, dims: int, factor: float, original: float,
                            fast: float, slow: float) -> torch.Tensor:
    """Pairs that turn fewer than ``slow`` times over ``original`` positions are slowed by ``factor``, pairs that
    turn more than ``fast`` times are kept, and between the two the mix goes linearly with the pair's index: the
    pair that turns ``t`` times has the (fractional) index ``dims ln(original / (2 pi t)) / (2 ln base)``; the ramp
    runs from the floor of that index for ``fast`` to its ceiling for ``slow`` (clipped to the pairs there are)."""
    where = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(fast)), 0)
    hi = min(math.ceil(where(slow)), dims - 1)
    i = torch.arange(inv_freq.numel(), dtype=torch.float64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return inv_freq / factor * ramp + inv_freq * (1.0 - ramp)


@register_position("rope_yarn")
class RopeYarn(PositionEncoding):
    """Rotary embedding over adjacent pairs of the leading ``rotary_dim`` elements (default: all; with the option
    ``pairing = "half"`` element ``j`` pairs with ``j + rotary_dim / 2`` instead) with frequencies
    ``theta ** (-2 j / rotary_dim)``, optionally stretched (``scaling = (factor, original, fast, slow)``, see
    :func:`yarn_scaled_frequencies`); with a scaling the sines and cosines are also multiplied by
    ``0.1 ln(factor) + 1`` (``Rotation.magnitude``)."""

    def rotation(self) -> Rotation:
        rd = int(self.spec.get("rotary_dim") or self.head_dim)
        if rd % 2 or not 0 < rd <= self.head_dim:
            raise ValueError(f"rotary_dim must be even and at most {self.head_dim}, got {rd}")
        theta = float(self.spec.theta)
        j = torch.arange(0, rd // 2, dtype=torch.float64)
        inv = torch.tensor(theta, dtype=torch.float64) ** (-2.0 * j / rd)
        magnitude = 1.0
        scaling = self.spec.get("scaling")
        if scaling:
            factor, original, fast, slow = (float(v) for v in scaling)
            inv = yarn_scaled_frequencies(inv, theta, rd, factor, original, fast, slow)
            magnitude = 0.1 * math.log(factor) + 1.0
        pairing = str(self.spec.get("pairing") or "adjacent")
        if pairing not in ("adjacent", "half"):
            raise ValueError(f"pairs are 'adjacent' or 'half', not {pairing!r}")
        return Rotation(inv.to(torch.float32), pairing=pairing, rotary_dim=rd, magnitude=magnitude)
