"""Rotary position encoding."""

from __future__ import annotations

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
    cosines and sines, from which a mixer's own kernels rotate."""

    graph_safe = True

    def __init__(self, head_dim: int, theta: float, rotary_dim: Optional[int] = None):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rope: rotary_dim {self.rotary_dim} must be even and within head_dim {head_dim}")
        self.inv_freq = None

    def prepare(self, device, compute_dtype) -> None:
        i = np.arange(self.rotary_dim // 2, dtype=np.float64)
        table = np.power(np.float64(self.theta), -2.0 * i / self.rotary_dim)
        self.inv_freq = torch.from_numpy(table).to(device)

    def table(self, ctx) -> torch.Tensor:
        """The cosines and sines of this step's positions: the same in every layer, made by the
        first one that asks."""
        key = ("rope cos/sin", self.theta, self.rotary_dim)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.memo[key] = ops.rope_table(ctx.positions, self.inv_freq)
        return table

    def rotation_table(self, head_dim, ctx):
        return self.table(ctx) if self.rotary_dim == head_dim else None

    def rotate(self, qkv, n_heads, n_kv, head_dim, ctx) -> None:
        cos_sin = self.table(ctx) if self.rotary_dim == head_dim and head_dim % 8 == 0 else None
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
