"""Rotary position encoding with half-split pairs (i, i + head_dim / 2)
(simply/utils/position_encoding.py:55-110)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import POSITION_ENCODINGS
from .base import PositionEncoding


@POSITION_ENCODINGS.register("rope")
class RoPE(PositionEncoding):
    def __init__(self, head_dim: int, base: float, scale_factor: float = 1.0, min_timescale: float = 1.0):
        if head_dim % 2:
            raise ValueError(f"rope: head_dim {head_dim} must be even")
        self.head_dim = int(head_dim)
        self.base = float(base)
        self.scale_factor = float(scale_factor)
        self.min_timescale = float(min_timescale)
        self._table: torch.Tensor | None = None

    def timescale_host(self) -> torch.Tensor:
        """timescale_i = min * (max / min) ** (2 i / head_dim)   (position_encoding.py:85-88),
        computed in float64 and rounded once to float32."""
        i = torch.arange(self.head_dim // 2, dtype=torch.float64)
        ts = self.min_timescale * (self.base / self.min_timescale) ** (2.0 * i / self.head_dim)
        return ts.to(torch.float32)

    def to_device(self, device) -> None:
        self._table = self.timescale_host().to(device)

    def rotary_table(self):
        if self._table is None:
            raise RuntimeError("rope: to_device() has not been called")
        return self._table, self.scale_factor

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        if head_dim != self.head_dim:
            raise ValueError(f"rope: built for head_dim {self.head_dim}, applied to {head_dim}")
        table, sf = self.rotary_table()
        ops.rope(x, positions, table, sf, div, num_heads, head_dim)


@POSITION_ENCODINGS.register("partial_rope")
class PartialRoPE(PositionEncoding):
    """Rotation of the first `dims` dimensions of a head only, in half-split pairs (i, i + dims / 2) by the angle
    position * base ** (-2 i / dims); the other dimensions pass unchanged.  The frequencies are computed in float64
    and rounded once to float32; the angle is their 32-bit product with the position."""

    def __init__(self, head_dim: int, dims: int, base: float):
        if dims % 2 or not 0 <= dims <= head_dim:
            raise ValueError(f"partial_rope: {dims} rotated dimensions of {head_dim} (an even number, at most all)")
        if dims and base <= 0:
            raise ValueError("partial_rope: the base must be positive")
        self.head_dim, self.dims, self.base = int(head_dim), int(dims), float(base)
        self._inv_freq: torch.Tensor | None = None

    def inv_freq_host(self) -> torch.Tensor:
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        return (self.base ** (-2.0 * i / max(self.dims, 1))).to(torch.float32)

    def to_device(self, device) -> None:
        self._inv_freq = self.inv_freq_host().to(device)

    def frequencies(self) -> tuple[torch.Tensor | None, int]:
        """(float32 [dims / 2] on the device, dims): what the rotate-and-write kernel of a mixer takes."""
        if self.dims and self._inv_freq is None:
            raise RuntimeError("partial_rope: to_device() has not been called")
        return (self._inv_freq if self.dims else None), self.dims

    def apply(self, x, positions, num_heads, head_dim, div=1.0):
        if head_dim != self.head_dim:
            raise ValueError(f"partial_rope: built for head_dim {self.head_dim}, applied to {head_dim}")
        if div != 1.0:
            raise ValueError("partial_rope: no division")
        inv_freq, dims = self.frequencies()
        # (the kernel's first H heads are rotated in place; no keys, no values, no norm)
        ops.qk_norm_rope_cache_write(x, positions, inv_freq, dims, None, num_heads, 0, head_dim, 1)
