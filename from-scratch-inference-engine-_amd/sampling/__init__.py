"""Greedy, temperature, top-k and top-p sampling."""

from .params import SamplingParams

__all__ = ["SamplingParams"]
