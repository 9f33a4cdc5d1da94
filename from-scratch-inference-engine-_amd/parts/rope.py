"""Rotary position encoding."""

from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from .. import ops
from .base import PositionEncoding, register_part


@register_part("position", "rope")
class RotaryEncoding(PositionEncoding):
    """Rotate-half RoPE over ``rotary_dim`` (default: the whole head): pair (i, i + rotary_dim/2),
    frequency theta^(-2i/rotary_dim), angle = position * frequency in float64
    (src/model/nn.cpp:110-149).  Where the whole head rotates it also offers the step's table of
    cosines and sines, from which a mixer's own kernels rotate.  ``layout="interleaved"``: the pairs are
    neighbours (2i, 2i + 1) instead, the frequencies the same; ``table`` gives a mixer the step's cosines
    and sines for its own kernels, ``rotate`` turns the first ``rotary_dim`` values of every q and k head.

    ``stretch`` = (factor, original, fast, slow) rescales the frequencies for contexts beyond ``original``
    positions: with dim(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0),
    hi = min(ceil(dim(slow)), rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i
    turns at f_i / factor * ramp_i + f_i * (1 - ramp_i) (fast pairs stay, slow pairs are divided by the factor,
    a ramp between), and every cosine and sine is multiplied by 0.1 * ln(factor) + 1.  That factor only exists
    in the table: ``rotate`` refuses where it would have to compute the angles itself.

    ``bands`` = (factor, low, high, original) rescales by wavelength instead: with l_i = 2 pi / f_i, a pair whose
    wavelength is below original / high keeps f_i, one above original / low turns at f_i / factor, and between the two
    s = (original / l_i - low) / (high - low) blends them, (1 - s) f_i / factor + s f_i."""

    graph_safe = True

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None, layout: str = "half",
                 stretch: Optional[tuple] = None, bands: Optional[tuple] = None):
        if layout not in ("half", "interleaved"):
            raise ValueError(f"rope: unknown layout '{layout}' (half or interleaved)")
        self.layout = layout
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rope: rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.inv_freq = None
        self.magnitude = 1.0
        self.bands = None
        if bands is not None:
            factor, low, high, original = (float(v) for v in bands)
            if stretch is not None or not (factor > 0 and original > 0 and 0 < low < high):
                raise ValueError(f"rope: bands {bands} need a positive factor and original and 0 < low < high (and no stretch)")
            self.bands = (factor, low, high, original)
        self.stretch = None
        if stretch is not None:
            factor, original, fast, slow = (float(v) for v in stretch)
            if not (factor >= 1.0 and original > 0 and fast > 0 and slow > 0 and self.theta > 1.0):
                raise ValueError(f"rope: stretch {stretch} needs factor >= 1 and positive original, fast and slow")
            self.stretch = (factor, original, fast, slow)
            self.magnitude = 0.1 * math.log(factor) + 1.0

    def frequencies(self) -> np.ndarray:
        """float64 [rotary_dim / 2]: the angle a position adds to each pair."""
        dims = self.rotary_dim
        i = np.arange(dims // 2, dtype=np.float64)
        freq = np.power(np.float64(self.theta), -2.0 * i / dims)
        if self.bands is not None:
            factor, low, high, original = self.bands
            wavelength = 2.0 * math.pi / freq
            blend = (original / wavelength - low) / (high - low)
            mixed = (1.0 - blend) * freq / factor + blend * freq
            return np.where(wavelength < original / high, freq, np.where(wavelength > original / low, freq / factor, mixed))
        if self.stretch is None:
            return freq
        factor, original, fast, slow = self.stretch

        def dim_of(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

        lo = max(math.floor(dim_of(fast)), 0)
        hi = min(math.ceil(dim_of(slow)), dims - 1)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return freq / factor * ramp + freq * (1.0 - ramp)

    def prepare(self, device, compute_dtype) -> None:
        self.inv_freq = torch.from_numpy(self.frequencies()).to(device)

    def table(self, ctx) -> torch.Tensor:
        """The cosines and sines of this step's positions: the same in every layer, made by the
        first one that asks."""
        key = ("rope cos/sin", self.theta, self.rotary_dim, self.stretch, self.bands)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = ops.rope_table(ctx.positions, self.inv_freq, self.magnitude)
        return table

    def rotation_table(self, head_dim, ctx):
        return self.table(ctx) if self.rotary_dim == head_dim and self.layout == "half" else None

    def rotate(self, qkv, n_heads, n_kv, head_dim, ctx) -> None:
        if self.layout == "interleaved":
            # (a lane reads its neighbour's value: from a copy, so that nobody reads what another has written)
            ops.rope_pairs(qkv.clone(), 0, head_dim, qkv, 0, head_dim, n_heads + n_kv, head_dim, self.rotary_dim // 2,
                           head_dim, self.table(ctx))
            return
        cos_sin = self.table(ctx) if self.rotary_dim == head_dim and head_dim % 8 == 0 else None
        if cos_sin is None and self.magnitude != 1.0:
            raise NotImplementedError("rope: a stretched rotation of part of a head exists as a table only")
        ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq, cos_sin=cos_sin)


@register_part("position", "none")
class NoPositionEncoding(PositionEncoding):
    """No rotation: q and k stay as they are."""

    graph_safe = True
    rotates = False

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim

    def rotate(self, qkv, n_heads, n_kv, head_dim, ctx) -> None:
        return None
