"""RMSNorm, fused with the residual sum."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import HiddenState, Norm, ParamDecl, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = (x * rsqrt(mean(x^2) + eps)) * w with x = residual + pending delta, all in float32;
    eps inside the square root, the weight multiplied last, plain w (the reference's rms_norm,
    src/model/nn.cpp:45-72, which sums in float64)."""

    adds_partial_sums = True

    graph_safe = True

    def __init__(self, hidden_size: int, eps: float):
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.hidden_size,), "vector", "norm")}

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        delta, hidden.delta = hidden.delta, None
        return ops.rmsnorm(hidden.residual, self.weight, self.eps, out_dtype, delta=delta,
                           write_back=delta is not None)

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        return ops.rmsnorm(hidden.residual, self.weight, self.eps, out_dtype, delta=hidden.delta, rows=rows)

    def plain(self, x: torch.Tensor, out=None) -> torch.Tensor:
        return ops.rmsnorm_plain(x, self.weight, self.eps, out=out)
