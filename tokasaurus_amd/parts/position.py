"""Rotary position encoding: the inverse frequencies (with the scaling rules a
checkpoint may ask for) and the cos/sin tables.

The reference builds cos/sin for every position up to
``max_position_embeddings`` once, in 32-bit, and looks rows up by position
(tokasaurus/model/llama.py:559-570,576-577); the generator itself is delegated
there to an installed package.  Definition used here: inv_freq_j = theta^(-2j/d);
``llama3`` scaling leaves wavelengths shorter than orig/high_freq_factor alone,
divides those longer than orig/low_freq_factor by ``factor`` and blends linearly
in between; ``linear`` divides all by ``factor``.
"""

from __future__ import annotations

import math

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import POSITION_ENCODINGS, PositionEncoding


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """[d/2] float32 on the host (a handful of numbers computed once at set-up)."""
    exponent = torch.arange(0, head_dim, 2, dtype=torch.int64).to(torch.float32) / head_dim
    inv_freq = 1.0 / (theta**exponent)
    if scaling is None or scaling["rope_type"] == "default":
        return inv_freq
    kind = scaling["rope_type"]
    factor = float(scaling["factor"])
    if kind == "linear":
        return inv_freq / factor
    if kind == "llama3":
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        orig = float(scaling["original_max_position_embeddings"])
        wavelen = 2 * math.pi / inv_freq
        long_wave = wavelen > orig / low
        short_wave = wavelen < orig / high
        smooth = (orig / wavelen - low) / (high - low)
        blended = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        out = torch.where(long_wave, inv_freq / factor, inv_freq)
        return torch.where(~long_wave & ~short_wave, blended, out)
    raise ValueError(f"unknown rope scaling {kind!r}")


@POSITION_ENCODINGS.register("rotary")
class RotaryEncoding(PositionEncoding):
    """cos/sin tables [max_positions, d/2] in 32-bit on the device; lane j of a
    head pairs with lane j + d/2."""

    def __init__(self, head_dim: int, theta: float, max_positions: int, scaling: dict | None = None):
        if head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {head_dim}")
        self.head_dim = head_dim
        self.theta = float(theta)
        self.max_positions = int(max_positions)
        self.scaling = scaling
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    def prepare(self, device: torch.device) -> None:
        if self.cos is not None:
            return
        inv_freq = inverse_frequencies(self.head_dim, self.theta, self.scaling).to(device)
        self.cos, self.sin = ops.rope_table(inv_freq, self.max_positions)
