"""Position encodings applied to q and k inside a mixer."""
from __future__ import annotations

import math
from typing import Optional

import torch

from .base import BuildContext, PositionEncoding


def scaled_frequencies(inv_freq: torch.Tensor, scaling) -> torch.Tensor:
    """float64 frequencies with their long wavelengths stretched (see RotaryHalfSplit)."""
    factor, low, high, original = float(scaling.factor), float(scaling.low), float(scaling.high), float(scaling.original)
    wavelength = 2.0 * math.pi / inv_freq
    share = (original / wavelength - low) / (high - low)
    mixed = (1.0 - share) * inv_freq / factor + share * inv_freq
    out = torch.where(wavelength > original / low, inv_freq / factor, mixed)
    return torch.where(wavelength < original / high, inv_freq, out)


class RotaryHalfSplit(PositionEncoding):
    """Rotary encoding with half-split pairing: element i pairs with i + rot/2,
    inv_freq_i = theta^(-2i/rot), angle = pos * inv_freq_i
      y[i] = x[i] cos - x[i + rot/2] sin,  y[i + rot/2] = x[i + rot/2] cos + x[i] sin
    (src/layers/rotary.cu:81-83, :96-116; the reference rotates the whole head,
    rot = head_dim, and computes angles on the fly with no table).  The
    frequencies are computed once in double precision and rounded to float32;
    the angle, sine and cosine are float32 in the kernel, computed once per step for
    all heads and layers."""

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None, scaling=None):
        """`scaling` (an object with `factor`, `low`, `high`, `original`, or None) stretches long
        wavelengths: with l = 2 pi / f a frequency is kept where l < original / high, divided by
        `factor` where l > original / low, and in between it is (1 - s) f / factor + s f with
        s = (original / l - low) / (high - low)."""
        self.scaling = scaling
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError("rotary_dim must be even and within the head")
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(self.theta, dtype=torch.float64), -(2.0 * i) / self.rotary_dim)
        if self.scaling is not None:
            inv = scaled_frequencies(inv, self.scaling)
        self.inv_freq = inv.to(torch.float32).to(ctx.device)

    def _scaling_key(self):
        s = self.scaling
        return None if s is None else (float(s.factor), float(s.low), float(s.high), float(s.original))

    def fused_rotary(self, step):
        # cosines and sines of this step's positions: made by the first layer that asks,
        # shared by every layer with the same rotation
        key = ("rope_table", self.theta, self.rotary_dim, self._scaling_key())
        table = step.scratch.get(key)
        if table is None:
            table = self.ctx.ops.rope_table(step.positions, self.inv_freq)
            step.scratch[key] = table
        return table, self.rotary_dim


class NoPositionEncoding(PositionEncoding):
    """q and k pass unchanged (a mixer whose order comes from elsewhere)."""

    def fused_rotary(self, step):
        return None, 0


class RotaryInterleaved(PositionEncoding):
    """Rotary encoding with neighbouring pairs: element 2i pairs with 2i + 1 for i < dims / 2,
    angle = pos * base^(-2i/dims),
      y[2i] = x[2i] cos - x[2i+1] sin,  y[2i+1] = x[2i+1] cos + x[2i] sin;
    elements from `dims` on pass unchanged.  The frequencies are computed once in double
    precision and rounded to float32; angle, sine and cosine are float32, made once per step for
    every layer with the same rotation (`table`), and applied by the mixer's own kernels."""

    def __init__(self, dims: int, base: float):
        if dims % 2 or dims < 0:
            raise ValueError("a rotation takes an even number of elements")
        self.rotary_dim = int(dims)
        self.base = float(base)
        self.inv_freq: Optional[torch.Tensor] = None

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(self.base, dtype=torch.float64), -(2.0 * i) / max(1, self.rotary_dim))
        self.inv_freq = inv.to(torch.float32).to(ctx.device)

    def table(self, step) -> Optional[torch.Tensor]:
        """float32 [N, dims / 2, 2] (cos, sin) of this step's positions; None without a rotation."""
        if self.rotary_dim == 0:
            return None
        key = ("rope_table", self.base, self.rotary_dim)
        table = step.scratch.get(key)
        if table is None:
            table = self.ctx.ops.rope_table(step.positions, self.inv_freq)
            step.scratch[key] = table
        return table
