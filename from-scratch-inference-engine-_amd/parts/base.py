"""Interfaces of the parts a layer is put together from, and the registries that name them.

A part is constructed from explicit sizes and constants, declares its parameters and what it
needs from the cache, and computes on the tokens of one step.  It never sees a model
configuration and does not know which model it is in.

Kinds and their interfaces (``ctx`` is the step's ``StepContext``):

  Norm             ``normed = norm(hidden)``; ``norm.rows(hidden, rows)`` for chosen rows.
                   ``hidden`` is a ``HiddenState``: the float32 residual stream plus a pending
                   delta that the next norm folds in (fused residual sum + norm).
                   ``norm.plain(x)`` normalises a plain tensor (an output before it is added,
                   the heads of q and k).
  Mixer            ``y = mixer.forward(x, ctx, cache)``; ``cache_need()`` says what it keeps per
                   request: a need of ``cache.needs`` (``PagedNeed``: keys and values per token,
                   ``StateNeed``: fixed size, or one of its own that owns its memory) or nothing; ``planner()`` may name per-step index tables it wants built on the host.
  FeedForward      ``y = ffn.forward(x, ctx)``.
  PositionEncoding ``pos.rotate(qkv, n_heads, n_kv, head_dim, ctx)`` transforms the q and k heads
                   in place by the step's positions.  It touches nothing else: bias, norms of q
                   and k and the write into the cache are the mixer's.
  Block            the arrangement: ``block.forward(hidden, ctx, cache)``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamDecl:
    """A parameter of a part.  ``storage``: 'matrix' (compute dtype), 'vector' (float32) or
    'int_table' (int32).  ``init`` names the random-weights distribution.  ``layout`` says how
    several checkpoint tensors make up the parameter: 'concat' (one after the other along dim
    0) or 'interleave' (row i of every source in turn: a0, b0, a1, b1, ...)."""

    shape: Tuple[int, ...]
    storage: str = "matrix"
    init: str = "weight"
    layout: str = "concat"


class HiddenState:
    """The residual stream of a step: ``residual`` float32 [T, H] and a pending ``delta`` that has
    not been added yet: [T, H] in the compute dtype, or (only if every norm of the model sets
    ``adds_partial_sums``, which the step's context then says in ``partial_sums_ok``) float32
    [S, T, H], partial sums of a matrix product to be added in order."""

    __slots__ = ("residual", "delta")

    def __init__(self, residual: torch.Tensor, delta: Optional[torch.Tensor] = None):
        self.residual = residual
        self.delta = delta


class Part:
    kind: str = "part"
    # True if the part takes everything that changes from step to step from device tensors (its
    # input and the context's device tables, never ctx.host) and never waits for the device, so
    # that a captured graph of a decode step can be replayed.  A model is replayed from graphs
    # only if every part of every layer says so.  A step is executed exactly once, also the one
    # that captures a graph (the warm-up before a capture runs on rows of no request), so a part
    # whose cache is a running state may set it.
    graph_safe = False
    # what the model was loaded with (``weight_copies``: whether large matrices may be kept a second
    # time in another order); the model sets it on every part before ``prepare``
    options: Dict[str, Any] = {}

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {}

    def prepare(self, device, compute_dtype: torch.dtype) -> None:
        """Called once after the parameters are set (tables, constants on the device)."""

    def release_optional_memory(self) -> int:
        """Give back device memory that the part can work without (second copies of weights in
        another order); returns the bytes.  Called when the cache does not fit beside them."""
        return 0

    def sub_parts(self) -> Dict[str, "Part"]:
        """The parts this one is made of (a block's norms, mixer and feed-forward; a mixer's
        position encoding and the norms of its heads).  The model prepares them, asks them for
        ``graph_safe`` and lists them with the rest; their parameters are bound like any part's."""
        return {}


def prepare_parts(part: "Part", device, compute_dtype: torch.dtype, options: Optional[Dict[str, Any]] = None,
                  _seen: Optional[set] = None) -> None:
    """``prepare`` for ``part`` and every part it is made of, each once, with ``options`` set on
    them first.  The model calls it for its parts; whoever uses a part by itself calls it too."""
    seen = set() if _seen is None else _seen
    if id(part) in seen:
        return
    seen.add(id(part))
    if options is not None:
        part.options = options
    part.prepare(device, compute_dtype)
    for sub in part.sub_parts().values():
        prepare_parts(sub, device, compute_dtype, options, seen)


class Norm(Part):
    kind = "norm"
    # True if the norm also takes a pending delta that comes as float32 partial sums [S, T, H]
    adds_partial_sums = False

    def __call__(self, hidden: HiddenState, out_dtype: torch.dtype) -> torch.Tensor:
        raise NotImplementedError

    def rows(self, hidden: HiddenState, rows: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        raise NotImplementedError

    def plain(self, x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The norm of a plain tensor [T, W], away from the residual stream: a mixer's or a
        feed-forward's output before it is added (sandwich and post-norm arrangements), or the
        heads of q and k (a norm as wide as a head normalises every head of a row; ``x`` may be
        the q or k columns of a q/k/v row, and ``out`` may be ``x``)."""
        raise NotImplementedError


class Mixer(Part):
    kind = "mixer"

    def cache_need(self):
        return None

    def planner(self):
        return None

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    kind = "feed_forward"

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    kind = "position"
    # False for an encoding that leaves q and k as they are (the mixer then skips the call)
    rotates = True

    def rotate(self, qkv: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, ctx) -> None:
        """Transform the q and k heads of ``qkv`` [T, (n_heads + 2 n_kv) head_dim] in place by the
        step's positions (``ctx.positions``, int32 [T]).  The bias has been added and the heads
        normalised, if the mixer does either; the values are not touched, and nothing is written
        to the cache: that is the mixer's, after this call."""
        raise NotImplementedError

    def rotation_table(self, head_dim: int, ctx) -> Optional[torch.Tensor]:
        """Optional: if this encoding is the rotation of the pairs (i, i + head_dim / 2) of every
        q and k head by an angle per token and pair, the step's float32 table [T, head_dim / 2, 2]
        of their cosines and sines.  A mixer whose own kernels rotate (in the epilogue of the q/k/v
        product, in the kernel that writes the cache, inside attention) takes the table instead of
        calling ``rotate``; None, the default: the mixer calls ``rotate``."""
        return None


class Block(Part):
    kind = "block"

    def forward(self, hidden: HiddenState, ctx, cache) -> None:
        raise NotImplementedError


# ------------------------------------------------------------------------------ registries
_REGISTRIES: Dict[str, Dict[str, Callable[..., Part]]] = {
    "norm": {}, "mixer": {}, "feed_forward": {}, "position": {}, "block": {},
}


def register_part(kind: str, name: str):
    """Class decorator: make a part constructible by name, e.g.
    ``@register_part("mixer", "my_mixer")``.  A test or an extension can register parts of its
    own without touching the engine's files."""
    if kind not in _REGISTRIES:
        raise KeyError(f"unknown part kind '{kind}' (known: {sorted(_REGISTRIES)})")

    def deco(cls):
        _REGISTRIES[kind][name] = cls
        return cls

    return deco


def make_part(kind: str, name: str, **params) -> Part:
    table = _REGISTRIES[kind]
    if name not in table:
        raise KeyError(f"no {kind} named '{name}' (known: {sorted(table)})")
    return table[name](**params)


def known_parts(kind: str):
    return sorted(_REGISTRIES[kind])
