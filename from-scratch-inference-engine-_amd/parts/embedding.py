"""Token embedding and the LM head."""

from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from .base import ParamDecl, Part
from .linear import Linear


class TokenEmbedding(Part):
    """x[t] = table[ids[t]] without scaling (src/model/nn.cpp:90-108), written as the float32
    residual stream."""

    kind = "embedding"
    graph_safe = True  # reads the step's token ids from the device

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight = None

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embedding(self.weight, ids)


class LMHead(Part):
    """logits = x . W^T in float32, no bias (src/model/model.cpp:144-148).  With tied embeddings
    its weight is bound to the embedding table."""

    kind = "lm_head"
    graph_safe = True

    def __init__(self, hidden_size: int, vocab_size: int):
        self.linear = Linear(hidden_size, vocab_size)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.vocab_size, self.hidden_size))}

    @property
    def weight(self):
        return self.linear.weight

    @weight.setter
    def weight(self, t):
        self.linear.weight = t

    def prepare(self, device, compute_dtype) -> None:
        self.linear.prepare(bool(self.options.get("weight_copies", True)))

    def release_optional_memory(self) -> int:
        return self.linear.drop_copy()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.linear(x, out_dtype=torch.float32)
