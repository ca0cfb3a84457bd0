"""y = x . W^T (+ b): the matrix product every part uses."""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from ..ops.tuning import library_mm
from ..ops.functions import (GEMM_MFMA_SKINNY_BEST_M, GEMM_MFMA_SKINNY_MAX_M, GEMM_MFMA_WIDE_MAX_M,
                             GEMM_SKINNY_MAX_M)


class Linear:
    """Holds ``weight`` [N, K] in the compute dtype and an optional float32 ``bias`` [N].

    float32: the engine's own kernels only (true 32-bit products and sums): vector FMA kernels,
    and for 3 to 64 rows (decoding) the matrix cores' float32 instruction, which rounds nothing.
    bfloat16: up to 16 rows (decoding) the engine's matrix-core kernel that streams the weight
    once; its sibling that shares x through LDS for float32 results of 8 to 64 rows (the logits;
    beyond 64 rows the library with a float32 result), for the residual projections
    (``for_residual``: 17 to 64 rows, and any number where K is long) and for the partial sums of
    other projections of 17 to 64 rows (``partial_sums``); everything else the library product
    (hipBLASLt through torch, where the reference's engine calls cuBLAS) with float32
    accumulation, the bias added by a kernel of the engine.  A large weight has a second copy in
    the order of the matrix instruction's fragments (``prepare``, ``streamed``), from which the
    sibling takes every product of up to 64 rows."""

    float32_on_matrix_cores = True  # up to 64 rows of float32: v_mfma_f32_16x16x4_f32 instead of vector FMAs
    # A bfloat16 weight of at least this many bytes is kept a second time, in the order of the matrix
    # instruction's fragments, for the engine's own products (decoding): a wave then loads 1 KB in one
    # piece with streaming loads, where rows give it 16 pieces of 64 bytes (a compute unit draws about
    # half as much when a wave's load is pieces of rows).  From 16 MB on: the q/k/v and output
    # projections of a 7B model (33 and 26 MB) gain by it.  The rows stay for the library's products of
    # many rows.  None: no copies.
    # A copy that would leave less than ``streamed_copy_reserve`` of the device's memory free is not
    # made: a model that large keeps copies of its first layers only and runs the rest from rows.
    streamed_copy_from = 16 << 20
    streamed_copy_reserve = 0.25

    def __init__(self, in_features: int, out_features: int, bias: bool = False):
        self.in_features = in_features
        self.out_features = out_features
        self.has_bias = bias
        self._weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.streamed = None  # the weight in fragment order (ops.FragmentOrdered), if prepare() made one
        self._wide_splits: dict = {}  # tiles of rows -> slices of K (a property of the sizes alone)
        self._wide_takes: dict = {}   # (tiles, slices, gate/up) -> whether the kernel takes them from this weight

    @property
    def weight(self) -> Optional[torch.Tensor]:
        return self._weight

    @weight.setter
    def weight(self, t: Optional[torch.Tensor]) -> None:
        self._weight = t
        self.streamed = None  # a copy of the weight that was here says nothing about this one
        self._wide_takes = {}

    def prepare(self, copies: bool = True) -> None:
        """Called by the owning part once the weight is set.  ``copies=False``: no second copy."""
        w = self.weight
        self.streamed = None
        if (copies and self.streamed_copy_from is not None and w is not None and w.dtype == torch.bfloat16 and w.is_cuda
                and w.numel() * 2 >= self.streamed_copy_from and ops.gemm_mfma_wide_splits_ok(self.in_features, 1)):
            free, total = torch.cuda.mem_get_info(w.device)
            if free - w.numel() * 2 >= self.streamed_copy_reserve * total:
                self.streamed = ops.fragment_order(w)

    def drop_copy(self) -> int:
        """Forget the fragment-ordered copy (the products then read rows); returns its bytes."""
        if self.streamed is None:
            return 0
        freed = self.streamed.data.numel() * self.streamed.data.element_size()
        self.streamed = None
        self._wide_takes = {}
        return freed

    @property
    def wide_weight(self):
        """What the products that share x through LDS read: the fragment-ordered copy if there is one."""
        return self.weight if self.streamed is None else self.streamed

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                 skip_bias: bool = False) -> torch.Tensor:
        bias = None if skip_bias else self.bias
        w = self.weight
        m = x.shape[0]
        if x.dtype == torch.float32:
            if self.float32_on_matrix_cores and 2 < m <= GEMM_MFMA_SKINNY_MAX_M and self.in_features % 4 == 0:
                # decoding in the 32-bit path: W streams once into true float32 matrix instructions
                # (several times faster than the vector kernels from 8 rows on, no faster at one or two)
                return ops.gemm_mfma_fp32(x, w, bias)
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        wants_f32 = out_dtype is not None and out_dtype != x.dtype
        if (wants_f32 and bias is None and (8 if self.streamed is None else 1) <= m <= GEMM_MFMA_SKINNY_MAX_M
                and ops.gemm_mfma_wide_splits_ok(self.in_features, 1)):
            # float32 results (logits) of 8 to 64 rows: x shared through LDS; from the fragment-ordered
            # copy at any number of rows
            return ops.gemm_mfma_wide(x, self.wide_weight)
        if (wants_f32 and bias is None and m > GEMM_MFMA_SKINNY_MAX_M and out_dtype == torch.float32
                and self.in_features % 8 == 0 and self.out_features % 8 == 0):
            # logits of more rows than the engine's kernels take (a decode batch beyond 64, a replay
            # that wants every position): the library with a float32 result
            return library_mm(x, w, float32_result=True)
        if self.in_features % 8 == 0 and m <= (GEMM_MFMA_SKINNY_MAX_M if wants_f32 else GEMM_MFMA_SKINNY_BEST_M):
            return ops.gemm_mfma_skinny(x, w, bias, out_dtype=out_dtype)
        if m <= GEMM_SKINNY_MAX_M or wants_f32 or self.in_features % 8 or self.out_features % 8:
            # few rows with an odd inner size; float32 results from bfloat16 operands (logits of
            # many rows); and sizes whose rows are not 16-byte aligned, which the library is not given
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        y = library_mm(x, w)
        if bias is not None:
            ops.bias_add(y, bias)
        return y

    def for_residual(self, x: torch.Tensor, ctx) -> torch.Tensor:
        """The product as the delta of the residual stream.  For a few rows (decoding) and a
        long inner dimension the matrix-core kernel cuts K into slices with workgroups of their
        own, which fills the chip where N alone leaves too few of them, and returns their float32
        partial sums [S, T, N]; the next norm adds them up in order."""
        m = x.shape[0]
        if (getattr(ctx, "partial_sums_ok", False) and x.dtype == torch.bfloat16 and self.bias is None
                and GEMM_MFMA_SKINNY_MAX_M < m <= GEMM_MFMA_WIDE_MAX_M and self.streamed is not None):
            # 65 to 128 rows of a fragment-ordered weight: the same kernel with five to eight tiles of x,
            # where its launch shape has one
            splits = self.wide_splits(m)
            if splits > 1 and self.wide_takes(m, splits):
                return ops.gemm_mfma_wide(x, self.streamed, splits=splits)
        if (getattr(ctx, "partial_sums_ok", False) and x.dtype == torch.bfloat16 and self.bias is None
                and self.in_features % 8 == 0 and 0 < m <= GEMM_MFMA_SKINNY_MAX_M):
            # the kernel that shares x through LDS: above 16 rows, and at any number of rows where
            # K is long enough for six slices or more
            splits = self.wide_splits(m)
            if splits > 1 and (m > GEMM_MFMA_SKINNY_BEST_M or splits >= 6 or self.streamed is not None):
                return ops.gemm_mfma_wide(x, self.wide_weight, splits=splits)
            splits = self.residual_splits(m)
            if splits > 1:
                return ops.gemm_mfma_skinny(x, self.weight, splits=splits)
        return self(x)

    def partial_sums(self, x: torch.Tensor, few_rows: bool = False) -> Optional[torch.Tensor]:
        """x . W^T (no bias) of 17 to 64 rows (to 128 from a fragment-ordered copy) as float32 partial
        sums [S, T, N] of slices of K, for a consumer that adds them up itself; None where the engine's
        kernel for that does not take the sizes.  ``few_rows``: also for up to 16 rows."""
        m = x.shape[0]
        most = GEMM_MFMA_SKINNY_MAX_M if self.streamed is None else GEMM_MFMA_WIDE_MAX_M
        least = 0 if few_rows else GEMM_MFMA_SKINNY_BEST_M  # (fewer rows: for a consumer that spares a launch by it)
        if x.dtype != torch.bfloat16 or not least < m <= most:
            return None
        splits = self.wide_splits(m)
        if splits < 2 or not self.wide_takes(m, splits):
            return None
        return ops.gemm_mfma_wide(x, self.wide_weight, splits=splits)

    def wide_takes(self, m: int, splits: int, gate_up: bool = False) -> bool:
        """Whether the kernel that shares x through LDS takes ``m`` rows of this weight (beyond 64 rows
        it has kernels for some launch shapes only)."""
        key = (-(-m // 16), splits, gate_up, self.streamed is not None)
        if key not in self._wide_takes:
            self._wide_takes[key] = ops.gemm_mfma_wide_takes(m, self.wide_weight, splits, gate_up)
        return self._wide_takes[key]

    def wide_splits(self, m: int) -> int:
        """Slices of K for the kernel that shares x through LDS, by the tiles of 16 rows that ``m``
        rows make (the kernel's own rule: as many as K gives, up to 8, for up to 16 rows; from 17
        rows on the cut that gives the most workgroups the device has room for).  1 = it does
        not take this K."""
        tiles = -(-m // 16)
        if tiles not in self._wide_splits:
            self._wide_splits[tiles] = ops.gemm_mfma_wide_best_splits(m, self.out_features, self.in_features)
        return self._wide_splits[tiles]

    def residual_splits(self, m: int) -> int:
        """Slices of K for ``for_residual`` (1 = do not cut): as many as bring the workgroups to
        about three and a half per compute unit, each slice at least 512 long.  Above 16 rows only
        where K gives four slices of 1024; shorter products of that many rows are the library's."""
        groups = -(-self.out_features // 16)
        shortest = 512 if m <= GEMM_MFMA_SKINNY_BEST_M else 1024
        splits = 1
        # (about three and a half workgroups a compute unit)
        while splits < 8 and 2 * groups * splits < 7 * ops.compute_units() and self.in_features // (2 * splits) >= shortest:
            splits *= 2
        if m > GEMM_MFMA_SKINNY_BEST_M and splits < 4:
            return 1
        return splits
