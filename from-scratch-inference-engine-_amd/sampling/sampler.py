"""Chooses next tokens on the device.

The reference samples on the host with one generator shared by all requests
(src/sampler/sampler.cpp:25-88), so its draws depend on what else is in the batch.  Here every
draw has its own uniform number, a pure function of (engine seed, request id, index of the
token in the request's output), and the kernel turns it into a token: what a request samples
does not depend on the batch it shares.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import SamplingParams

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_for(seed: int, request_id: int, index: int) -> float:
    """A number in [0, 1) for the ``index``-th sampled token of ``request_id``."""
    z = _splitmix64(seed & _MASK)
    z = _splitmix64(z ^ (request_id & _MASK))
    z = _splitmix64(z ^ (index & _MASK))
    return (z >> 11) / float(1 << 53)


class Sampler:
    def __init__(self, seed: int = 0):
        self.seed = int(seed)
        # the parameters of a step's rows travel in one pinned buffer and one copy
        self._pinned: Optional[torch.Tensor] = None
        self._copied: Optional[torch.cuda.Event] = None

    def _upload(self, uniform, temperature, top_k, top_p, device):
        """One host-to-device copy for the four per-row arrays: [uniform float64 | temperature
        float32 | top_k int32 | top_p float32], each n long; returns their device views."""
        n = len(uniform)
        if self._copied is not None:
            self._copied.synchronize()  # the last copy has read the buffer
        if self._pinned is None or self._pinned.numel() < 20 * n:
            self._pinned = torch.empty((max(20 * n, 4096),), dtype=torch.uint8, pin_memory=True)
        host = self._pinned.numpy()
        host[:8 * n].view(np.float64)[:] = uniform
        host[8 * n:12 * n].view(np.float32)[:] = temperature
        host[12 * n:16 * n].view(np.int32)[:] = top_k
        host[16 * n:20 * n].view(np.float32)[:] = top_p
        dev = self._pinned[:20 * n].to(device, non_blocking=True)
        if self._copied is None:
            self._copied = torch.cuda.Event()
        self._copied.record()
        return (dev[:8 * n].view(torch.float64), dev[8 * n:12 * n].view(torch.float32),
                dev[12 * n:16 * n].view(torch.int32), dev[16 * n:20 * n].view(torch.float32))

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], request_ids: Sequence[int],
               indices: Sequence[int]) -> List[int]:
        """One token per row of ``logits`` [n, vocab] (float32, on the device)."""
        if logits.shape[0] == 0:
            return []
        return self.sample_on_device(logits, params, request_ids, indices).tolist()

    def sample_on_device(self, logits: torch.Tensor, params: Sequence[SamplingParams], request_ids: Sequence[int],
                         indices: Sequence[int]) -> torch.Tensor:
        """The same, left on the device (int32 [n]) and not waited for: the caller reads it when
        it needs the ids, and the next step may take them from there meanwhile."""
        n = logits.shape[0]
        if not (len(params) == len(request_ids) == len(indices) == n):
            raise ValueError("sample: one set of parameters, request id and index per row")
        if all(p.greedy for p in params):
            return ops.sample(logits)
        uniform, temperature, top_k, top_p = self._upload(
            [uniform_for(self.seed, r, i) for r, i in zip(request_ids, indices)],
            [max(float(p.temperature), 0.0) for p in params], [int(p.top_k) for p in params],
            [float(p.top_p) for p in params], logits.device)
        return ops.sample(logits, temperature, top_k, top_p, uniform)
