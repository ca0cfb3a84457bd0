"""y = x . W^T (+ b): the matrix product every part uses."""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from ..ops.functions import GEMM_MFMA_SKINNY_BEST_M, GEMM_MFMA_SKINNY_MAX_M, GEMM_SKINNY_MAX_M


class Linear:
    """Holds ``weight`` [N, K] in the compute dtype and an optional float32 ``bias`` [N].

    float32: the engine's own kernels only (true 32-bit products and sums).
    bfloat16: up to 16 rows (decoding) the engine's matrix-core kernel that streams the weight
    once (up to 64 rows for float32 results, the logits); above that the library product (hipBLASLt through torch, where the reference's engine
    calls cuBLAS) with float32 accumulation, the bias added by a kernel of the engine."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False):
        self.in_features = in_features
        self.out_features = out_features
        self.has_bias = bias
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def __call__(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                 skip_bias: bool = False) -> torch.Tensor:
        bias = None if skip_bias else self.bias
        w = self.weight
        m = x.shape[0]
        if x.dtype == torch.float32:
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        wants_f32 = out_dtype is not None and out_dtype != x.dtype
        if self.in_features % 8 == 0 and m <= (GEMM_MFMA_SKINNY_MAX_M if wants_f32 else GEMM_MFMA_SKINNY_BEST_M):
            return ops.gemm_mfma_skinny(x, w, bias, out_dtype=out_dtype)
        if m <= GEMM_SKINNY_MAX_M or wants_f32 or self.in_features % 8 or self.out_features % 8:
            # few rows with an odd inner size; float32 results from bfloat16 operands (logits of
            # many rows); and sizes whose rows are not 16-byte aligned, which the library is not given
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        y = torch.mm(x, w.t())
        if bias is not None:
            ops.bias_add(y, bias)
        return y
