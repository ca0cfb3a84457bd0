"""The arrangement of a layer's parts."""

from __future__ import annotations

from typing import Dict

from .base import Block, FeedForward, HiddenState, Mixer, Norm, Part, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += ffn(norm2(x))  (src/model/model.cpp:106-139).  The sums are
    left pending in the hidden state, so the next norm (this block's second, the next block's
    first, or the model's last) adds them in the same pass that normalises."""

    graph_safe = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def sub_parts(self) -> Dict[str, Part]:
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, hidden: HiddenState, ctx, cache) -> None:
        x = self.mixer_norm(hidden, ctx.compute_dtype)
        hidden.delta = self.mixer.forward(x, ctx, cache)
        x = self.ffn_norm(hidden, ctx.compute_dtype)
        hidden.delta = self.ffn.forward(x, ctx)
