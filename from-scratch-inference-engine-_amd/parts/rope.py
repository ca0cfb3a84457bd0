"""Rotary position encoding."""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import ops
from ..ops.functions import GEMM_MFMA_SKINNY_BEST_M
from .base import PositionEncoding, register_part


class KVStore:
    """Where a position encoding hands keys and values: the pools of one layer and, per token,
    the slot to write (negative = not stored)."""

    __slots__ = ("k_pool", "v_pool", "slots", "page_size")

    def __init__(self, k_pool, v_pool, slots, page_size):
        self.k_pool, self.v_pool, self.slots, self.page_size = k_pool, v_pool, slots, page_size


@register_part("position", "rope")
class RotaryEncoding(PositionEncoding):
    """Rotate-half RoPE over ``rotary_dim`` (default: the whole head): pair (i, i + rotary_dim/2),
    frequency theta^(-2i/rotary_dim), angle = position * frequency in float64
    (src/model/nn.cpp:110-149).  Fused with the q/k/v bias and the write into the cache."""

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

    def apply(self, qkv, n_heads, n_kv, head_dim, ctx, store: Optional[KVStore], bias=None) -> None:
        cos_sin = self.table(ctx) if self.rotary_dim == head_dim and head_dim % 8 == 0 else None
        if store is None:
            ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq, bias=bias, cos_sin=cos_sin)
        else:
            ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq, slots=store.slots,
                              k_pool=store.k_pool, v_pool=store.v_pool, page_size=store.page_size, bias=bias,
                              cos_sin=cos_sin)

    def apply_sums(self, parts, n_heads, n_kv, head_dim, ctx, store: Optional[KVStore], bias=None):
        if self.rotary_dim != head_dim or head_dim % 8:
            return None
        qkv = torch.empty(parts.shape[1:], dtype=ctx.compute_dtype, device=parts.device)
        kw = {} if store is None else dict(slots=store.slots, k_pool=store.k_pool, v_pool=store.v_pool,
                                           page_size=store.page_size)
        return ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq, bias=bias,
                                 cos_sin=self.table(ctx), parts=parts, **kw)

    def project(self, x, weight, bias, n_heads, n_kv, head_dim, ctx, store: Optional[KVStore]):
        """For a few rows of bfloat16 (decoding) the projection's own epilogue rotates and stores."""
        if (x.dtype != torch.bfloat16 or not 0 < x.shape[0] <= GEMM_MFMA_SKINNY_BEST_M or x.shape[1] % 8
                or head_dim % 16 or self.rotary_dim != head_dim):
            return None
        table = self.table(ctx)
        if store is None:
            return ops.gemm_mfma_skinny_rope(x, weight, bias, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq,
                                             cos_sin=table)
        return ops.gemm_mfma_skinny_rope(x, weight, bias, ctx.positions, n_heads, n_kv, head_dim, self.inv_freq,
                                         slots=store.slots, k_pool=store.k_pool, v_pool=store.v_pool,
                                         page_size=store.page_size, cos_sin=table)


@register_part("position", "none")
class NoPositionEncoding(PositionEncoding):
    """No rotation: only the bias and the write into the cache."""

    graph_safe = True

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim

    def apply(self, qkv, n_heads, n_kv, head_dim, ctx, store: Optional[KVStore], bias=None) -> None:
        if store is None:
            ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, None, bias=bias)
        else:
            ops.rope_kv_write(qkv, ctx.positions, n_heads, n_kv, head_dim, None, slots=store.slots,
                              k_pool=store.k_pool, v_pool=store.v_pool, page_size=store.page_size, bias=bias)
