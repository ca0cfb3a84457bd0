"""Seeded random weights: in memory, or written out as a model folder."""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Sequence

import torch

from .loader import ParamBinding, TensorSpec, expected_tensors
from .safetensors_file import write_safetensors

INIT_STD = 0.02


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    """Each tensor has its own stream keyed by (seed, name), so a tensor's values do not depend
    on which other tensors exist.  Distributions: weights and biases N(0, 0.02), norm weights
    1 + N(0, 0.02).  (The reference's test fixture draws everything from N(0, 0.02),
    tests/cpp/tiny_model.hpp:46-73; norm weights near 1 keep activations at a useful scale.)"""
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_for(seed, spec.name))
    if spec.init == "int":
        return torch.randint(0, 2 ** 15, spec.shape, generator=gen, device=device, dtype=torch.int32)
    t = torch.randn(spec.shape, generator=gen, device=device, dtype=torch.float32) * INIT_STD
    if spec.init == "norm":
        t = t + 1.0
    elif spec.init not in ("weight", "bias"):
        raise ValueError(f"unknown init '{spec.init}' for {spec.name}")
    return t.to(dtype)


def random_checkpoint_tensors(bindings: Sequence[ParamBinding], seed: int,
                              dtype: torch.dtype = torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    return {name: random_tensor(spec, seed, dtype, device)
            for name, spec in expected_tensors(bindings).items()}


def write_random_model(config, seed: int, out_dir, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors`` for ``config`` (a typed
    configuration of a registered architecture) with weights drawn from ``seed``."""
    from ..models.registry import build_model_spec

    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    spec = build_model_spec(config)
    tensors = random_checkpoint_tensors(spec.bindings, seed, dtype)
    (out / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    write_safetensors(out / "model.safetensors", tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return out
