"""Rotary position encoding: with half-split pairs (i, i + rot/2), and with neighbouring pairs (2i, 2i + 1) and an
optional stretching of the slow pairs for contexts longer than the trained one.

Reference mini_llm/nn/rope.py:34-40 (inverse frequencies 1 / theta^(2i/d) in float32),
74-80 (angle = float32(position) * inv_freq), 110-146 (rotation).  The tables are made once
per step, in float32, and shared by every layer that uses this encoding; the rotation itself
is fused into the attention mixer's q/k kernel.
"""

from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import Part, register


class RotaryHalfSplit(Part):
    """Pairs (i, i + rotary_dim/2) turned by position * theta^(-2i/rotary_dim) / factor; `factor` (linear scaling of the
    positions: every frequency divided by it) is 1 unless given."""

    def __init__(self, rotary_dim: int, theta: float, factor: float = 1.0):
        if rotary_dim <= 0 or rotary_dim % 2 != 0:
            raise ValueError(f"rotary_dim must be a positive even integer, got {rotary_dim}")
        if theta <= 0:
            raise ValueError(f"theta must be positive, got {theta}")
        if not factor > 0:
            raise ValueError(f"factor must be positive, got {factor}")
        self.rotary_dim, self.theta, self.factor = rotary_dim, theta, float(factor)
        dims = torch.arange(0, rotary_dim, 2, dtype=torch.float32)
        self._inv_freq_host = 1.0 / (theta ** (dims / rotary_dim))
        if self.factor != 1.0:
            self._inv_freq_host = self._inv_freq_host / self.factor
        self._inv_freq = None

    def key(self):
        return ("rope_half", self.rotary_dim, self.theta, self.factor)

    def tables(self, ctx):
        """cos and sin [T, rotary_dim/2] float32 for this step's positions (made once per step)."""
        cached = ctx.memo.get(self.key())
        if cached is None:
            if self._inv_freq is None or self._inv_freq.device != ctx.positions.device:
                self._inv_freq = self._inv_freq_host.to(ctx.positions.device)
            half = self.rotary_dim // 2
            tag = f"{self.rotary_dim}_{self.theta}" + ("" if self.factor == 1.0 else f"_{self.factor}")
            cos = ctx.scratch(f"rope_cos_{tag}", (ctx.T, half), torch.float32)
            sin = ctx.scratch(f"rope_sin_{tag}", (ctx.T, half), torch.float32)
            ops.rope_table(cos, sin, ctx.positions, self._inv_freq)
            cached = ctx.memo[self.key()] = (cos, sin)
        return cached


def yarn_frequencies(rotary_dim: int, theta: float, factor: float, original: float, fast: float, slow: float) -> tuple:
    """(frequencies [rotary_dim / 2] float64, magnitude) of a rotation whose slow pairs are stretched by `factor`.

    With f_i = theta^(-2i / rotary_dim) and turns(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), the pair index
    at which a context of `original` positions makes t turns: pairs below lo = max(floor(turns(fast)), 0) keep f_i, pairs
    above hi = min(ceil(turns(slow)), rotary_dim - 1) turn `factor` times slower, and between them
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) blends: f_i / factor * ramp_i + f_i * (1 - ramp_i).
    cos and sin are both multiplied by the magnitude 0.1 ln(factor) + 1."""
    if factor <= 0 or original <= 0 or fast <= 0 or slow <= 0:
        raise ValueError(f"factor, original, fast and slow must be positive, got {factor}, {original}, {fast}, {slow}")
    index = torch.arange(0, rotary_dim // 2, dtype=torch.float64)
    plain = theta ** (-2.0 * index / rotary_dim)

    def turns(t: float) -> float:
        return rotary_dim * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(theta))

    lo = max(math.floor(turns(fast)), 0)
    hi = min(math.ceil(turns(slow)), rotary_dim - 1)
    ramp = ((index - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return plain / factor * ramp + plain * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


class RotaryInterleaved(Part):
    """Rotary positions whose pairs are neighbours, (2i, 2i + 1): the pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a) with a = p * f_i, f_i = theta^(-2i / rotary_dim).  `scaling` (a mapping with
    factor, original, fast, slow) stretches the slow pairs, see yarn_frequencies(); `factor` alone divides every frequency by a
    constant (linear scaling of the positions).  The tables are the same kind as the
    half-split part's, [T, rotary_dim / 2] float32 made once a step; the mixer's kernel pairs the dims."""

    pairing = "interleaved"

    def __init__(self, rotary_dim: int, theta: float, scaling: dict | None = None, factor: float = 1.0):
        if rotary_dim <= 0 or rotary_dim % 2 != 0:
            raise ValueError(f"rotary_dim must be a positive even integer, got {rotary_dim}")
        if theta <= 0 or theta == 1:
            raise ValueError(f"theta must be positive and not 1, got {theta}")
        if not factor > 0 or (factor != 1.0 and scaling is not None):
            raise ValueError(f"factor must be positive and comes without `scaling`, got {factor}")
        self.rotary_dim, self.theta, self.factor = rotary_dim, theta, float(factor)
        self.scaling = None if scaling is None else tuple(float(scaling[name]) for name in ("factor", "original", "fast", "slow"))
        if self.scaling is None:
            frequencies, self.magnitude = theta ** (-2.0 * torch.arange(0, rotary_dim // 2, dtype=torch.float64) / rotary_dim) / self.factor, 1.0
        else:
            frequencies, self.magnitude = yarn_frequencies(rotary_dim, theta, *self.scaling)
        self._inv_freq_host = frequencies.to(torch.float32)
        self._inv_freq = None

    def key(self):
        return ("rope_interleaved", self.rotary_dim, self.theta, self.scaling, self.factor)

    def tables(self, ctx):
        """cos and sin [T, rotary_dim/2] float32 for this step's positions, times the magnitude (made once per step)."""
        cached = ctx.memo.get(self.key())
        if cached is None:
            if self._inv_freq is None or self._inv_freq.device != ctx.positions.device:
                self._inv_freq = self._inv_freq_host.to(ctx.positions.device)
            half = self.rotary_dim // 2
            tag = f"{self.rotary_dim}_{self.theta}_{self.scaling}" + ("" if self.factor == 1.0 else f"_{self.factor}")
            cos = ctx.scratch(f"rope_pairs_cos_{tag}", (ctx.T, half), torch.float32)
            sin = ctx.scratch(f"rope_pairs_sin_{tag}", (ctx.T, half), torch.float32)
            ops.rope_table(cos, sin, ctx.positions, self._inv_freq, self.magnitude)
            cached = ctx.memo[self.key()] = (cos, sin)
        return cached


class NoPosition(Part):
    """No position signal inside the mixer."""

    def tables(self, ctx):
        return None


register("position", "rope_half", RotaryHalfSplit)
register("position", "rope_interleaved", RotaryInterleaved)
register("position", "none", NoPosition)
