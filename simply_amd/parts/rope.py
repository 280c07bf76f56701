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
