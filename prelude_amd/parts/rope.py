"""Rotary position encoding: the cos/sin tables mixers rotate by.

inv_freq_j = 1 / f32(theta^(2j/d)) with the power in 64-bit, angle
f32(p) * inv_freq_j in 32-bit, cos and sin in 32-bit
(crates/prelude-core/src/models/commons/attn_utils.rs:32-50).  The tables stay
32-bit in every mode (the reference rounds them to the engine's type).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import PartError, PositionEncoding, register_part


@register_part("position", "rope")
class RotaryEmbedding(PositionEncoding):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, rotary_dim: int, max_positions: int, theta: float):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise PartError(f"rope: rotary width {rotary_dim} must be positive and even")
        self.rotary_dim = int(rotary_dim)
        self.max_positions = int(max_positions)
        self.theta = float(theta)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def prepare(self, device):
        d = self.rotary_dim
        j = torch.arange(0, d, 2, dtype=torch.float64)
        inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), j / d).to(torch.float32)
        pos = torch.arange(self.max_positions, dtype=torch.float32).reshape(-1, 1)
        ang = pos * inv_freq.reshape(1, -1)
        self.cos = torch.cos(ang).contiguous().to(device)
        self.sin = torch.sin(ang).contiguous().to(device)


@register_part("position", "rotary_frequencies")
class RotaryFrequencies(PositionEncoding):
    """The frequencies alone, f_i = theta^(-2i/d) for i < d/2 (the power in 64-bit, rounded once to 32-bit): the
    mixers' kernels take the angle position * f_i and its cosine and sine themselves, in 32-bit, so there is no
    table and no longest position.  How the rotated dimensions are paired is the mixer's business."""
    GRAPH_SAFE_PORTIONS = True

    def __init__(self, rotary_dim: int, theta: float, long_wave_factor: float = 0.0, long_wave_low: float = 1.0,
                 long_wave_high: float = 1.0, long_wave_original: int = 0):
        """``long_wave_factor`` > 0 slows the long wavelengths down.  With lambda = 2 pi / f a frequency's wavelength,
        lambda_short = ``long_wave_original`` / ``long_wave_high`` and lambda_long = ``long_wave_original`` /
        ``long_wave_low``: waves shorter than lambda_short keep f, waves longer than lambda_long turn at f / factor,
        and those between move from the one to the other, f / factor + t (f - f / factor) with
        t = (original / lambda - low) / (high - low).  0: the plain frequencies."""
        if rotary_dim <= 0 or rotary_dim % 2:
            raise PartError(f"rotary_frequencies: rotary width {rotary_dim} must be positive and even")
        if theta <= 0:
            raise PartError(f"rotary_frequencies: base {theta} must be positive")
        self.rotary_dim = int(rotary_dim)
        self.theta = float(theta)
        self.long_wave_factor = float(long_wave_factor or 0.0)
        self.long_wave_low, self.long_wave_high = float(long_wave_low), float(long_wave_high)
        self.long_wave_original = float(long_wave_original)
        if self.long_wave_factor < 0 or (self.long_wave_factor > 0 and not (
                self.long_wave_original > 0 and self.long_wave_low > 0 and self.long_wave_high > self.long_wave_low)):
            raise PartError(f"rotary_frequencies: long waves scaled by {long_wave_factor} need an original length > 0 "
                            f"and 0 < low < high, got {long_wave_original}, {long_wave_low}, {long_wave_high}")
        self.inv_freq: Optional[torch.Tensor] = None

    def frequencies(self) -> torch.Tensor:
        """The frequencies in 64-bit, on the host."""
        d = self.rotary_dim
        i = torch.arange(0, d // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * i / d)
        if self.long_wave_factor > 0:
            length = 2.0 * math.pi / f
            orig, low, high = self.long_wave_original, self.long_wave_low, self.long_wave_high
            s = (orig / length - low) / (high - low)
            blended = (1.0 - s) * f / self.long_wave_factor + s * f
            f = torch.where(length < orig / high, f, torch.where(length > orig / low, f / self.long_wave_factor, blended))
        return f

    def prepare(self, device):
        self.inv_freq = self.frequencies().to(torch.float32).to(device)
