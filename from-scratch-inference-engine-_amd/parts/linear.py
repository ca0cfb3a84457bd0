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
    # instruction's fragments, for the products of up to 64 rows (decoding): a wave then loads 1 KB in
    # one piece with streaming loads, where rows give it 16 pieces of 64 bytes (MI355X, 8 rows: N = 37888,
    # K = 3584, 272 MB, 43.7 against 49.3 us; N = 3584, K = 18944, 136 MB, 23.2 against 27.2; N = 152064,
    # K = 3584 179 against 194; N = K = 5120, 52 MB, 10.3 against 12.7; N = K = 4096, 34 MB, 9.3 against 7.5,
    # and N = K = 3584, 26 MB, 6.7 against 6.5, so small ones are not copied).  The
    # rows stay for the library's products of many rows (prefill).  The device has 288 GB: twice the
    # large matrices of a 32B model are 120.  None: no copies.  A copy is not made where it would leave
    # less than ``streamed_copy_reserve`` of the device's memory free (for the cache and the steps'
    # own tensors): a model that large keeps copies of its first layers only and runs the rest from rows.
    streamed_copy_from = 48 << 20
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
                # (4 layers of 3584 / 18944 and the head on MI355X, ms a step against the vector
                # kernels: 8 rows 1.9 / 2.8, 32 rows 3.1 / 23, 64 rows 5.0 / 25; one row 1.6 / 1.5)
                return ops.gemm_mfma_fp32(x, w, bias)
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        wants_f32 = out_dtype is not None and out_dtype != x.dtype
        if (wants_f32 and bias is None and (8 if self.streamed is None else 1) <= m <= GEMM_MFMA_SKINNY_MAX_M
                and ops.gemm_mfma_wide_splits_ok(self.in_features, 1)):
            # logits of 8 to 64 rows: x shared through LDS (N = 152064, K = 3584 on MI355X: 200
            # against 215 us at 8 rows, 242 against 486 at 64); from the fragment-ordered copy at any
            # number of rows (one row 164 us, the few-rows kernel on rows 176 to 198)
            return ops.gemm_mfma_wide(x, self.wide_weight)
        if (wants_f32 and bias is None and m > GEMM_MFMA_SKINNY_MAX_M and out_dtype == torch.float32
                and self.in_features % 8 == 0 and self.out_features % 8 == 0):
            # logits of more rows than the engine's kernels take (a decode batch beyond 64, a replay
            # that wants every position): the library with a float32 result (N = 152064, K = 3584
            # on MI355X at 256 rows: 0.38 ms; the engine's 64-row kernel four times 0.96, its tiled
            # float32 kernel 7)
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
            # where its launch shape has one (N = 3584, K = 18944 on MI355X at 96 rows: 35 us in 9 slices; the
            # library 95, or some 60 with its kernel chosen by timing)
            splits = self.wide_splits(m)
            if splits > 1 and self.wide_takes(m, splits):
                return ops.gemm_mfma_wide(x, self.streamed, splits=splits)
        if (getattr(ctx, "partial_sums_ok", False) and x.dtype == torch.bfloat16 and self.bias is None
                and self.in_features % 8 == 0 and 0 < m <= GEMM_MFMA_SKINNY_MAX_M):
            # the kernel that shares x through LDS: above 16 rows, and at any number of rows where
            # K is long enough for six slices or more (N = 3584, K = 18944 in 8: 26 against 28 us at 8
            # rows, 27 against 32 at 16; N = K = 3584 in 7: 7.4 against 8.4 at 8 rows)
            splits = self.wide_splits(m)
            if splits > 1 and (m > GEMM_MFMA_SKINNY_BEST_M or splits >= 6 or self.streamed is not None):
                return ops.gemm_mfma_wide(x, self.wide_weight, splits=splits)
            splits = self.residual_splits(m)
            if splits > 1:
                return ops.gemm_mfma_skinny(x, self.weight, splits=splits)
        return self(x)

    def partial_sums(self, x: torch.Tensor, few_rows: bool = False) -> Optional[torch.Tensor]:
        """x . W^T (no bias) of 17 to 64 rows (to 128 from a fragment-ordered copy) as float32 partial sums [S, T, N] of slices of K, for a
        consumer that adds them up itself; None where the engine's kernel for that does not take the
        sizes (N = 4608, K = 3584 on MI355X at 64 rows: 12.4 us, the library's whole product 18.8;
        at 32 rows 9.1 against 13.6)."""
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
        not take this K.  (64 rows on MI355X: N = 3584, K = 18944 in 9 slices 32 us, against 68 for
        the few-rows kernel and 91 for the library; N = K = 3584 in 4 slices 10.9 against the
        library's 13.7.)"""
        tiles = -(-m // 16)
        if tiles not in self._wide_splits:
            self._wide_splits[tiles] = ops.gemm_mfma_wide_best_splits(m, self.out_features, self.in_features)
        return self._wide_splits[tiles]

    def residual_splits(self, m: int) -> int:
        """Slices of K for ``for_residual`` (1 = do not cut): as many as bring the workgroups to
        about four per compute unit, each slice at least 512 long (N = K = 3584, 8 rows: 8.2 us in
        four slices, 8.8 in two).  Above 16 rows only where K gives four slices of 1024; shorter
        products of that many rows are the library's (measured on MI355X at N = 3584, K = 18944,
        64 rows: 67 us against the library's 91)."""
        groups = -(-self.out_features // 16)
        shortest = 512 if m <= GEMM_MFMA_SKINNY_BEST_M else 1024
        splits = 1
        # (about three and a half workgroups a compute unit)
        while splits < 8 and 2 * groups * splits < 7 * ops.compute_units() and self.in_features // (2 * splits) >= shortest:
            splits *= 2
        if m > GEMM_MFMA_SKINNY_BEST_M and splits < 4:
            return 1
        return splits
