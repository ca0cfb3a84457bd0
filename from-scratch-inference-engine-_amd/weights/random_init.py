"""Seeded random weights: in memory, or written out as a model folder.

Every value is a pure function of (seed, tensor name, index of the element): a counter-based
generator, written twice, for the host (numpy) and for the device (a kernel), which give the
same bits.  A model made on the device from a configuration and a seed therefore holds exactly
the weights that ``write_random_model`` writes for them, and a tensor's values do not depend on
which other tensors exist or in which order they are made.

The generator: two 64-bit outputs of the SplitMix64 sequence started at
``splitmix64(seed) ^ first 8 bytes of sha256(name)``, numbers 2i and 2i + 1 for element i; the sum
of their eight 16-bit fields is an integer with mean 262,140 and standard deviation 53,509.9
(Irwin-Hall: close to normal, bounded by 4.9 standard deviations); centred and scaled it is a
float32 z, and the value is z * 0.02 (weights, biases) or 1 + z * 0.02 (norm weights), every
operation a single float32 operation that rounds the same everywhere.  Integer tables take 15
bits of the first output.  (The reference's test fixture draws everything from N(0, 0.02),
tests/cpp/tiny_model.hpp:46-73; norm weights near 1 keep activations at a useful scale.)
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Sequence

import numpy as np
import torch

from .loader import ParamBinding, TensorSpec, expected_tensors
from .safetensors_file import write_safetensors

INIT_STD = 0.02
_MASK = (1 << 64) - 1
_GAMMA = 0x9E3779B97F4A7C15
_SUM_MEAN = 4 * 65535                       # of eight uniform 16-bit fields
_INV_SUM_STD = np.float32(1.8688124e-05)    # 1 / sqrt(8 * (65536^2 - 1) / 12), bits 0x379cc471


def _splitmix64(x: int) -> int:
    x = (x + _GAMMA) & _MASK
    z = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def stream_key(seed: int, name: str) -> int:
    """Where the SplitMix64 sequence of a tensor starts."""
    name_bits = int.from_bytes(hashlib.sha256(name.encode()).digest()[:8], "little")
    return _splitmix64(seed & _MASK) ^ name_bits


def _outputs(key: int, first: int, count: int):
    """Numbers 2i and 2i + 1 of the sequence for i in [first, first + count), as uint64 arrays."""
    with np.errstate(over="ignore"):
        i = np.arange(first, first + count, dtype=np.uint64)
        out = []
        for k in (0, 1):
            x = np.uint64(key) + (np.uint64(2) * i + np.uint64(k) + np.uint64(1)) * np.uint64(_GAMMA)
            z = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            out.append(z ^ (z >> np.uint64(31)))
    return out


def host_values(key: int, n: int, init: str) -> np.ndarray:
    """The n values of a tensor on the host: float32, or int32 for ``init == 'int'``."""
    out = np.empty((n,), dtype=np.int32 if init == "int" else np.float32)
    chunk = 1 << 20
    for first in range(0, n, chunk):
        count = min(chunk, n - first)
        a, b = _outputs(key, first, count)
        if init == "int":
            out[first:first + count] = ((a >> np.uint64(17)) & np.uint64(0x7FFF)).astype(np.int32)
            continue
        total = np.zeros((count,), dtype=np.int64)
        for word in (a, b):
            for shift in (0, 16, 32, 48):
                total += ((word >> np.uint64(shift)) & np.uint64(0xFFFF)).astype(np.int64)
        z = (total - _SUM_MEAN).astype(np.float32) * _INV_SUM_STD
        v = z * np.float32(INIT_STD)
        out[first:first + count] = v + np.float32(1.0) if init == "norm" else v
    return out


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    """The tensor ``spec`` of the random model ``seed``: drawn by the kernel on a GPU, by numpy on
    the host, the same bits either way.  Distributions: weights and biases 0.02 z, norm weights
    1 + 0.02 z (z close to standard normal), integer tables uniform in [0, 2^15)."""
    if spec.init not in ("weight", "bias", "norm", "int"):
        raise ValueError(f"unknown init '{spec.init}' for {spec.name}")
    key = stream_key(seed, spec.name)
    n = 1
    for d in spec.shape:
        n *= int(d)
    device = torch.device(device)
    if device.type == "cuda":
        from .. import ops

        if spec.init == "int":
            return ops.random_fill(torch.empty(spec.shape, dtype=torch.int32, device=device), key, "int")
        return ops.random_fill(torch.empty(spec.shape, dtype=torch.float32, device=device), key, spec.init,
                               INIT_STD).to(dtype)
    t = torch.from_numpy(host_values(key, n, spec.init)).reshape(spec.shape)
    return t if spec.init == "int" else t.to(dtype)


def random_checkpoint_tensors(bindings: Sequence[ParamBinding], seed: int,
                              dtype: torch.dtype = torch.bfloat16, device="cpu") -> Dict[str, torch.Tensor]:
    return {name: random_tensor(spec, seed, dtype, device)
            for name, spec in expected_tensors(bindings).items()}


def write_random_model(config, seed: int, out_dir, dtype: torch.dtype = torch.bfloat16, device=None) -> Path:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors`` for ``config`` (a typed
    configuration of a registered architecture) with weights drawn from ``seed``.  ``device``: where
    the values are made (default: the GPU if there is one; the file is the same either way)."""
    from ..models.registry import build_model_spec

    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    spec = build_model_spec(config)
    if device is None:
        device = "cuda:0" if torch.cuda.is_available() else "cpu"
    tensors = {name: t.cpu() for name, t in random_checkpoint_tensors(spec.bindings, seed, dtype, device).items()}
    (out / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    write_safetensors(out / "model.safetensors", tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return out
