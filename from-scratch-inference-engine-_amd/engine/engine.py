"""The engine: scheduler + step function + sampler, with the reference's surface."""

from __future__ import annotations

from typing import List, Optional, Sequence as Seq

from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .context import StepEntry
from .model import Model, Runner
from .scheduler import Request, Scheduler, SeqStatus


class Engine:
    """``Engine(model, block_size, num_blocks, seed=0, max_batch=256)`` with ``add_request``,
    ``step``, ``has_work``, ``output``, ``status``, ``preemptions`` and ``generate`` as in the
    reference (bindings/module.cpp:103-147, include/engine/engine.hpp:36-89).  Added:
    ``max_tokens_per_step`` (token budget of a step) and ``prefill_chunk`` (longest portion of a
    prompt in one step).  ``enable_prefix_cache`` is accepted for compatibility; prefix caching
    is not part of this engine and the flag changes nothing."""

    def __init__(self, model: Model, block_size: int = 16, num_blocks: int = 2048, seed: int = 0,
                 max_batch: int = 256, enable_prefix_cache: bool = False, *, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None):
        self.model = model
        self.runner = Runner(model, page_size=block_size, num_pages=num_blocks, max_requests=max_batch)
        self.scheduler = Scheduler(self.runner.manager, max_batch=max_batch,
                                   max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk,
                                   max_position=self.runner.max_position)
        self.sampler = Sampler(seed)

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

    def step(self) -> None:
        items = self.scheduler.schedule()
        if not items:
            return
        entries = [StepEntry(it.seq.cache, it.tokens, [len(it.tokens) - 1] if it.wants_logits else [])
                   for it in items]
        logits = self.runner.step(entries, keep=False)
        wanting = [it for it in items if it.wants_logits]
        tokens = self.sampler.sample(logits, [it.seq.request.params for it in wanting],
                                     [it.seq.id for it in wanting], [len(it.seq.output) for it in wanting])
        sampled, k = [], 0
        for it in items:
            if it.wants_logits:
                sampled.append(tokens[k])
                k += 1
            else:
                sampled.append(None)
        self.scheduler.finish_step(items, sampled)

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
            before = (self.runner.steps, self.scheduler.preemptions)
            self.step()
            if (self.runner.steps, self.scheduler.preemptions) == before:
                raise RuntimeError("Engine.generate: the scheduler made no progress")
        return self.output(sid)

    def generate_batch(self, prompts: Seq[Seq[int]], params: Optional[SamplingParams] = None,
                       max_tokens: int = 16, eos_id: int = -1) -> List[List[int]]:
        """All prompts submitted at once and batched by the scheduler."""
        ids = [self.add_request(p, params, max_tokens, eos_id) for p in prompts]
        while any(self.status(i) != SeqStatus.Finished for i in ids):
            before = (self.runner.steps, self.scheduler.preemptions)
            self.step()
            if (self.runner.steps, self.scheduler.preemptions) == before:
                raise RuntimeError("Engine.generate_batch: the scheduler made no progress")
        return [self.output(i) for i in ids]
