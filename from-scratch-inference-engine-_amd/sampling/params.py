"""Sampling parameters, with the reference's names and meanings."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    """include/engine/sampler.hpp:9-13: ``temperature <= 0`` selects greedy (argmax),
    ``top_k = 0`` disables top-k, ``top_p >= 1`` disables top-p."""

    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0
