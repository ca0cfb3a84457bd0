"""Dense gated feed-forward."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import FeedForward, ParamDecl, register_part
from ..ops.functions import GEMM_MFMA_SKINNY_BEST_M
from .linear import Linear


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)), no biases (src/model/model.cpp:134-138).  gate and up are one
    matrix [2I, H] with their rows interleaved (gate_0, up_0, gate_1, up_1, ...): x is read once,
    and the lane that holds gate_j also holds up_j, so that for a few rows (decoding) SiLU*up
    happens in the product's epilogue and the [T, 2I] intermediate never reaches memory."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = Linear(hidden_size, 2 * intermediate_size)
        self.down = Linear(intermediate_size, hidden_size)

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"gate_up_weight": ParamDecl((2 * self.intermediate_size, self.hidden_size), layout="interleave"),
                "down_weight": ParamDecl((self.hidden_size, self.intermediate_size))}

    @property
    def gate_up_weight(self):
        return self.gate_up.weight

    @gate_up_weight.setter
    def gate_up_weight(self, t):
        self.gate_up.weight = t

    @property
    def down_weight(self):
        return self.down.weight

    @down_weight.setter
    def down_weight(self, t):
        self.down.weight = t

    def prepare(self, device, compute_dtype) -> None:
        copies = bool(self.options.get("weight_copies", True))
        self.gate_up.prepare(copies)
        self.down.prepare(copies)

    def release_optional_memory(self) -> int:
        return self.gate_up.drop_copy() + self.down.drop_copy()

    # rows up to which silu(gate) * up comes from the product that shares x through LDS when the weight
    # has a fragment-ordered copy (beyond: the library's product and a kernel for SiLU*up)
    streamed_swiglu_max_rows = 128

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        m = x.shape[0]
        if (x.dtype == torch.bfloat16 and self.gate_up.streamed is not None and 0 < m <= self.streamed_swiglu_max_rows
                and self.gate_up.wide_takes(m, 1, gate_up=True)):
            # from the fragment-ordered copy at any number of rows up to 64, and up to 128 where the
            # kernel has the launch shape for it: SiLU*up in the product's epilogue
            act = ops.gemm_mfma_wide_swiglu(x, self.gate_up.streamed)
        elif (x.dtype == torch.bfloat16 and 3 <= m <= GEMM_MFMA_SKINNY_BEST_M and self.hidden_size % 128 == 0
                and self.gate_up.out_features % 4 == 0 and self.gate_up.out_features // 64 >= ops.compute_units()):
            # three rows and more of a matrix that gives every compute unit a workgroup: the kernel that
            # shares x through LDS (one or two rows, and small matrices, are faster in the other)
            act = ops.gemm_mfma_wide_swiglu(x, self.gate_up.weight)
        elif x.dtype == torch.bfloat16 and m <= GEMM_MFMA_SKINNY_BEST_M and self.hidden_size % 8 == 0:
            act = ops.gemm_mfma_skinny(x, self.gate_up.weight, epilogue="swiglu")
        else:
            act = ops.swiglu(self.gate_up(x))
        return self.down.for_residual(act, ctx)
