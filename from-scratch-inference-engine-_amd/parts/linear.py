"""y = x . W^T (+ b): the matrix product every part uses."""

from __future__ import annotations

from typing import Optional

import torch

from .. import ops
from ..ops.functions import GEMM_SKINNY_MAX_M


class Linear:
    """Holds ``weight`` [N, K] in the compute dtype and an optional float32 ``bias`` [N].

    float32: the engine's own kernels only (true 32-bit products and sums).
    bfloat16: the engine's skinny kernel for up to 8 rows; above that the library product
    (hipBLASLt through torch, where the reference's engine calls cuBLAS) with float32
    accumulation, the bias added by a kernel of the engine."""

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
        if x.dtype == torch.float32 or x.shape[0] <= GEMM_SKINNY_MAX_M:
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        if out_dtype is not None and out_dtype != x.dtype:
            # float32 result from bfloat16 operands (logits): the engine's tiled kernel
            return ops.gemm(x, w, bias, out_dtype=out_dtype)
        y = torch.mm(x, w.t())
        if bias is not None:
            ops.bias_add(y, bias)
        return y
