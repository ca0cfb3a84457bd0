"""The engine: scheduler + step function + sampler, with the reference's surface."""

from __future__ import annotations

from typing import List, Optional, Sequence as Seq

import torch

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .context import StepEntry
from .model import Model, Runner
from .scheduler import Request, Scheduler, SeqStatus


class _Landing:
    """Token ids on their way from the device to pinned host memory."""

    def __init__(self, ids_on_device: torch.Tensor):
        self.host = torch.empty(ids_on_device.shape, dtype=ids_on_device.dtype, pin_memory=True)
        self.host.copy_(ids_on_device, non_blocking=True)
        self.event = torch.cuda.Event()
        self.event.record()

    def read(self) -> List[int]:
        self.event.synchronize()
        return self.host.tolist()


class Engine:
    """``Engine(model, block_size, num_blocks, seed=0, max_batch=256)`` with ``add_request``,
    ``step``, ``has_work``, ``output``, ``status``, ``preemptions`` and ``generate`` as in the
    reference (bindings/module.cpp:103-147, include/engine/engine.hpp:36-89).  Added:
    ``max_tokens_per_step`` (token budget of a step), ``prefill_chunk`` (longest portion of a
    prompt in one step) and ``fill_rows`` (see ``Runner``); ``num_blocks=0`` makes the pool as large
    as the device's free memory allows (``Model.pages_that_fit``).  ``enable_prefix_cache`` is accepted for compatibility; prefix caching
    is not part of this engine and the flag changes nothing."""

    def __init__(self, model: Model, block_size: int = 16, num_blocks: int = 2048, seed: int = 0,
                 max_batch: int = 256, enable_prefix_cache: bool = False, *, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None, fill_rows=None):
        self.model = model
        if num_blocks <= 0:
            num_blocks = model.pages_that_fit(block_size)
        self.runner = Runner(model, page_size=block_size, num_pages=num_blocks, max_requests=max_batch,
                             fill_rows=fill_rows)
        self.scheduler = Scheduler(self.runner.manager, max_batch=max_batch,
                                   max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk,
                                   max_position=self.runner.max_position)
        self.sampler = Sampler(seed)
        self.run_ahead = True
        self._pending = None  # (items, samples on the device) of a step that is queued but not read
        self.steps_read = 0   # steps whose samples have reached the requests' outputs

    def add_request(self, prompt: Seq[int], params: Optional[SamplingParams] = None, max_tokens: int = 16,
                    eos_id: int = -1) -> int:
        prompt = [int(t) for t in prompt]
        vocab = self.runner.vocab_size
        for t in prompt:
            if not 0 <= t < vocab:
                raise IndexError(f"Engine: token id {t} is outside the vocabulary [0, {vocab})")
        return self.scheduler.add_request(Request(prompt, params or SamplingParams(), int(max_tokens), int(eos_id)))

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def _launch(self, items, feed=None):
        """Queue the step of ``items`` and the sampling of its logits; nothing is waited for.
        ``feed``: the device tensor of the previous step's samples, for a step that runs ahead."""
        entries = [StepEntry(it.seq.cache, it.tokens, [len(it.tokens) - 1] if it.wants_logits else [])
                   for it in items]
        logits = self.runner.step(entries, keep=False, feed=feed)
        wanting = [it for it in items if it.wants_logits]
        if not wanting:
            return items, None, None
        # the index of a sample among its request's samples: those in the output plus, for a step
        # that runs ahead, the one still on its way
        ahead = 1 if feed is not None else 0
        sampled = self.sampler.sample_on_device(logits, [it.seq.request.params for it in wanting],
                                                [it.seq.id for it in wanting],
                                                [len(it.seq.output) + ahead for it in wanting])
        # the ids start their way to the host now, ahead of whatever is queued after this step
        # (a copy asked for later would wait behind the next step)
        landing = _Landing(sampled)
        return items, sampled, landing

    def _finish(self, items, landing) -> None:
        tokens = landing.read() if landing is not None else []
        sampled, k = [], 0
        for it in items:
            if it.wants_logits:
                sampled.append(tokens[k])
                k += 1
            else:
                sampled.append(None)
        self.scheduler.finish_step(items, sampled)
        self.steps_read += 1

    def _progress(self):
        return (self.runner.steps, self.steps_read, self.scheduler.preemptions)

    def step(self) -> None:
        """One model step.  While every running request decodes, the engine runs one step ahead:
        the next step is queued, with its token ids taken from the device, before the samples of
        the present one are read, so the GPU does not wait for the host between steps.  Outputs
        show a step's tokens once that step has been read, i.e. one call later than it was queued."""
        if self._pending is not None and not any(
                it.wants_logits and it.seq.status == SeqStatus.Running for it in self._pending[0]):
            self._pending = None  # nobody is left who wants that step's samples
        if self._pending is None:
            items = self.scheduler.schedule()
            if not items:
                return
            self._pending = self._launch(items)
        items, sampled, landing = self._pending
        nxt = self.scheduler.lookahead(items) if (self.run_ahead and sampled is not None) else None
        self._pending = self._launch(nxt, feed=sampled) if nxt is not None else None
        self._finish(items, landing)

    def output(self, seq_id: int) -> List[int]:
        return list(self.scheduler.sequences[seq_id].output)

    def status(self, seq_id: int) -> SeqStatus:
        return self.scheduler.sequences[seq_id].status

    def preemptions(self) -> int:
        return self.scheduler.preemptions

    def prefix_hits(self) -> int:
        return 0

    def free_blocks(self) -> int:
        return self.runner.manager.free_pages(0) if self.runner.manager.groups else 0

    def generate(self, prompt: Seq[int], params: Optional[SamplingParams] = None, max_tokens: int = 16,
                 eos_id: int = -1) -> List[int]:
        sid = self.add_request(prompt, params, max_tokens, eos_id)
        while self.status(sid) != SeqStatus.Finished:
            before = self._progress()
            self.step()
            if self._progress() == before:
                raise RuntimeError("Engine.generate: the scheduler made no progress")
        return self.output(sid)

    def generate_batch(self, prompts: Seq[Seq[int]], params: Optional[SamplingParams] = None,
                       max_tokens: int = 16, eos_id: int = -1) -> List[List[int]]:
        """All prompts submitted at once and batched by the scheduler."""
        ids = [self.add_request(p, params, max_tokens, eos_id) for p in prompts]
        while any(self.status(i) != SeqStatus.Finished for i in ids):
            before = self._progress()
            self.step()
            if self._progress() == before:
                raise RuntimeError("Engine.generate_batch: the scheduler made no progress")
        return [self.output(i) for i in ids]
