"""Rotary position encoding with the llama3 wavelength-band scaling.

Inverse frequencies are derived in 64-bit, stored in 32-bit, and the cos/sin
tables are evaluated in 64-bit from the stored 32-bit frequencies, as the
reference does (src/kernels.cpp:114-187). The table holds one half of each row
(the reference's two halves are equal) for positions up to `max_position`; the
reference stops at min(max_position_embeddings, original max, 8192)
(include/llmengine/config.hpp:39-45), this table does not.
"""
from __future__ import annotations

import math

import torch

from .base import Placement, PositionEncoding
from .registry import register_part


def inverse_frequencies(rotary_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """[rotary_dim / 2] float64. scaling: factor, low_freq_factor, high_freq_factor,
    original_max_position_embeddings (src/kernels.cpp:122-155); pi is the true
    double value where the reference widens a float literal."""
    half = rotary_dim // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = 1.0 / torch.pow(torch.tensor(float(theta), dtype=torch.float64), 2.0 * i / rotary_dim)
    if scaling:
        factor = float(scaling["factor"])
        low = float(scaling["low_freq_factor"])
        high = float(scaling["high_freq_factor"])
        orig = float(scaling["original_max_position_embeddings"])
        wavelen = 2.0 * math.pi / freq
        low_wavelen, high_wavelen = orig / low, orig / high
        if high != low:
            smooth = (orig / wavelen - low) / (high - low)
        else:
            smooth = torch.zeros_like(freq)
        blended = (1.0 - smooth) * freq / factor + smooth * freq
        freq = torch.where(wavelen > low_wavelen, freq / factor,
                           torch.where(wavelen < high_wavelen, freq, blended))
    return freq


class RotaryEmbedding(PositionEncoding):
    graph_safe = True

    def __init__(self, rotary_dim: int, theta: float, max_position: int, scaling: dict | None = None):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be even")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self._max_position = int(max_position)
        self.scaling = dict(scaling) if scaling else None
        self.inv_freq = inverse_frequencies(self.rotary_dim, self.theta, self.scaling).to(torch.float32)
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None

    @property
    def max_position(self) -> int:
        return self._max_position

    def materialize(self, placement: Placement) -> None:
        if self.cos is not None and self.cos.device == placement.device:
            return
        pos = torch.arange(self._max_position, dtype=torch.float64)
        angle = pos[:, None] * self.inv_freq.to(torch.float64)[None, :]
        self.cos = torch.cos(angle).to(torch.float32).to(placement.device).contiguous()
        self.sin = torch.sin(angle).to(torch.float32).to(placement.device).contiguous()

    def rotary_tables(self):
        if self.cos is None:
            raise RuntimeError("rotary tables are not on the device yet (load the model first)")
        return self.cos, self.sin, self.rotary_dim


register_part("position", "rotary", RotaryEmbedding)
