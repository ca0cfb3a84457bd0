"""Dense gated feed-forward."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import FeedForward, ParamDecl, register_part
from .linear import Linear


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down(silu(gate(x)) * up(x)), no biases (src/model/model.cpp:134-138).  gate and up are one
    matrix [2I, H] (gate rows first), so x is read once."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = Linear(hidden_size, 2 * intermediate_size)
        self.down = Linear(intermediate_size, hidden_size)

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"gate_up_weight": ParamDecl((2 * self.intermediate_size, self.hidden_size)),
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

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        return self.down(ops.swiglu(self.gate_up(x)))
