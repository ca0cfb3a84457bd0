"""The description of a model that an architecture builds from its configuration."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

from ..parts.base import Block, Norm, Part
from ..parts.embedding import LMHead, TokenEmbedding
from ..weights.loader import ParamBinding, TensorSpec


@dataclass(frozen=True)
class LayerCall:
    """One entry of the order in which layers run.

    ``layer`` indexes ``ModelSpec.layers`` (the same layer may be named by several calls: its
    weights are then shared, each call has a cache of its own).  ``cache_of`` = index of an
    *earlier call* whose cache this call reads instead of keeping one (its mixer then writes
    nothing); ``None`` = the call keeps its own."""

    layer: int
    cache_of: Optional[int] = None


@dataclass
class ModelSpec:
    """Parts, the order they run in, and how checkpoint tensors map to their parameters."""

    config: object
    embedding: TokenEmbedding
    layers: List[Block]
    schedule: List[LayerCall]
    final_norm: Norm
    lm_head: LMHead
    bindings: List[ParamBinding] = field(default_factory=list)
    ignore_unexpected: Sequence[str] = ()

    def all_parts(self) -> List[Part]:
        """Every part of the model once, parts before the parts they are made of."""
        out: List[Part] = []
        seen = set()

        def add(part: Part) -> None:
            if id(part) in seen:
                return
            seen.add(id(part))
            out.append(part)
            for sub in part.sub_parts().values():
                add(sub)

        for part in (self.embedding, *self.layers, self.final_norm, self.lm_head):
            add(part)
        return out

    def stream_norms(self) -> List[Norm]:
        """The norms that read the residual stream and fold its pending delta in: those a block
        names among its own parts, and the final one."""
        norms = [p for block in self.layers for p in block.sub_parts().values() if isinstance(p, Norm)]
        return norms + [self.final_norm]


def bind(bindings: List[ParamBinding], owner: Part, attr: str, sources: Sequence[TensorSpec]) -> None:
    """Declare that ``owner.attr`` is made of the checkpoint tensors ``sources`` (joined along
    dim 0 the way the part's declaration says); checks the shapes against that declaration."""
    decl = owner.param_decls()[attr]
    rows = sum(s.shape[0] for s in sources)
    tail = tuple(sources[0].shape[1:])
    if any(tuple(s.shape[1:]) != tail for s in sources) or (rows, *tail) != tuple(decl.shape):
        raise ValueError(f"{type(owner).__name__}.{attr}: sources {[s.shape for s in sources]} do not "
                         f"make up {decl.shape}")
    bindings.append(ParamBinding(owner, attr, list(sources), decl.storage, decl.layout))
