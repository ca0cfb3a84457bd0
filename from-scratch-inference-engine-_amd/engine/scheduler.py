"""Continuous batching: which requests run in the next step, and with which tokens.

Pure host logic over the cache manager, so every decision can be tested without a GPU.

Policy (the reference's, src/engine/engine.cpp:53-178, plus a token budget and portions):
  * first come, first served: waiting requests are admitted in order while there is a free
    state slot, ``max_batch`` is not reached and the pool can hold the request's whole present
    context beside what the running requests still need for theirs; the first one that does
    not fit blocks those behind it;
  * a step holds at most ``max_tokens_per_step`` tokens: one for every request that has only
    its last token left (decoding), then portions of the remaining prompts, each cut to the
    budget, to ``prefill_chunk`` and to the pages that are free; no more requests run at once
    than a step has tokens for, so a decoding request is never left out for want of budget;
  * a request whose next tokens find no free pages is left out of the step; if nothing at all
    fits and more than one request is running, the youngest running request that holds pages is
    preempted: its pages go back, it returns to the head of the waiting queue and later
    recomputes prompt + output from the start;
  * a request that could never fit the pool (or max_position_embeddings) is refused when added;
  * after sampling, a request ends on its end-of-sequence token (which is kept in the output)
    or at ``max_tokens``; its pages and slot go back at once.

Running ahead: while the samples of a launched step are still on their way to the host,
``lookahead`` names the step that follows it, if that does not depend on them: every running
request decodes, none can reach ``max_tokens`` with the pending sample, nobody waits to be
admitted and every request finds a page for one more token.  The engine launches that step with
the token ids taken from the device.  A request that turns out to have ended on its
end-of-sequence token has then run one token too far; that token is dropped, and what it wrote
lies beyond the request's end in pages that go back with the rest.
"""

from __future__ import annotations

import enum
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional

from ..cache.manager import CacheManager, RequestCache
from ..sampling.params import SamplingParams


class SeqStatus(enum.Enum):
    """include/engine/engine.hpp: Waiting, Running, Finished."""

    Waiting = 0
    Running = 1
    Finished = 2


@dataclass
class Request:
    """include/engine/engine.hpp:16-24."""

    prompt: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    max_tokens: int = 16
    eos_id: int = -1


@dataclass
class Sequence:
    id: int
    request: Request
    output: List[int] = field(default_factory=list)
    status: SeqStatus = SeqStatus.Waiting
    cache: Optional[RequestCache] = None

    @property
    def context(self) -> List[int]:
        return self.request.prompt + self.output

    def tokens(self, start: int, n: int) -> List[int]:
        """``context[start:start + n]`` without putting the whole context together (a decode step
        asks every request for one token of a context of thousands)."""
        prompt = self.request.prompt
        if start >= len(prompt):
            return self.output[start - len(prompt):start - len(prompt) + n]
        if start + n <= len(prompt):
            return prompt[start:start + n]
        return prompt[start:] + self.output[:start + n - len(prompt)]

    @property
    def computed(self) -> int:
        return self.cache.length if self.cache is not None else 0

    @property
    def remaining(self) -> int:
        return len(self.request.prompt) + len(self.output) - self.computed


@dataclass
class ScheduledItem:
    seq: Sequence
    tokens: List[int]
    wants_logits: bool
    ahead: bool = False  # launched before the sample that gives its token was read (ids from the device)


class Scheduler:
    def __init__(self, manager: CacheManager, max_batch: int = 256, max_tokens_per_step: int = 2048,
                 prefill_chunk: Optional[int] = None, max_position: int = 0):
        if max_batch < 1 or max_tokens_per_step < 1:
            raise ValueError("Scheduler: max_batch and max_tokens_per_step must be positive")
        self.manager = manager
        # never more running requests than a step has tokens for: every request that decodes
        # gets its token in every step, nobody starves behind the budget
        self.max_batch = min(max_batch, manager.max_requests, max_tokens_per_step)
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk or max_tokens_per_step
        self.max_position = max_position
        self.waiting: Deque[int] = deque()
        self.running: List[int] = []
        self.sequences: Dict[int, Sequence] = {}
        self.preemptions = 0
        self._next_id = 0

    # ------------------------------------------------------------------ requests
    def add_request(self, request: Request) -> int:
        if not request.prompt:
            raise ValueError("Engine: empty prompt")
        if request.max_tokens < 1:
            raise ValueError("Engine: max_tokens must be at least 1")
        total = len(request.prompt) + request.max_tokens - 1  # the last sampled token is never fed
        if self.max_position and total > self.max_position:
            raise ValueError(f"Engine: prompt of {len(request.prompt)} tokens + max_tokens {request.max_tokens} "
                             f"exceeds max_position_embeddings {self.max_position}")
        need = self.manager.max_pages_held(total, self.prefill_chunk)
        for g, pages in enumerate(need):
            if pages > self.manager.allocators[g].num_pages:
                raise ValueError(f"Engine: the request needs {pages} pages of {self.manager.tokens_per_page(g)} tokens, "
                                 f"the pool has {self.manager.allocators[g].num_pages}: it can never run")
        sid = self._next_id
        self._next_id += 1
        self.sequences[sid] = Sequence(id=sid, request=request)
        self.waiting.append(sid)
        return sid

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ one step
    def _admit(self) -> None:
        n_groups = len(self.manager.groups)
        # pages that running requests still need for the context they already own
        promised = [0] * n_groups
        for sid in self.running:
            seq = self.sequences[sid]
            for g, k in enumerate(self.manager.new_pages_needed(seq.cache, seq.remaining)):
                promised[g] += k
        while self.waiting and len(self.running) < self.max_batch and self.manager.free_slots > 0:
            seq = self.sequences[self.waiting[0]]
            need = self.manager.max_pages_held(seq.remaining, self.prefill_chunk)
            if any(need[g] > self.manager.free_pages(g) - promised[g] for g in range(n_groups)):
                break  # first come, first served: the head of the queue blocks those behind it
            for g in range(n_groups):
                promised[g] += need[g]
            seq.cache = self.manager.open(seq.id)
            seq.status = SeqStatus.Running
            self.running.append(seq.id)
            self.waiting.popleft()

    def _fit_tokens(self, taken: List[int], seq: Sequence, n: int) -> int:
        """Largest n' <= n such that the step can still reserve n' tokens for ``seq`` beside the
        pages per group that its other items have ``taken``."""
        manager = self.manager

        def fits(k: int) -> bool:
            need = manager.new_pages_needed(seq.cache, k)
            return all(need[g] + taken[g] <= manager.free_pages(g) for g in range(len(taken)))

        while n > 0 and not fits(n):
            # cut back to the last page boundary below n (what is free in the last held page
            # always fits), then page by page
            filled = seq.computed + n
            step = self.manager.smallest_page_tokens
            n = ((filled - 1) // step) * step - seq.computed
        return max(n, 0)

    def _build(self) -> List[ScheduledItem]:
        items: List[ScheduledItem] = []
        taken = [0] * len(self.manager.groups)
        budget = self.max_tokens_per_step
        seqs = [self.sequences[i] for i in self.running]
        for decode_pass in (True, False):
            for seq in seqs:
                decoding = seq.remaining == 1 and seq.computed > 0
                if decoding != decode_pass or budget <= 0:
                    continue
                n = min(seq.remaining, budget) if decode_pass else min(seq.remaining, self.prefill_chunk, budget)
                n = self._fit_tokens(taken, seq, n)
                if n <= 0:
                    continue
                tokens = seq.tokens(seq.computed, n)
                items.append(ScheduledItem(seq, tokens, n == seq.remaining))
                for g, k in enumerate(self.manager.new_pages_needed(seq.cache, n)):
                    taken[g] += k
                budget -= n
        return items

    def _preempt_youngest(self) -> bool:
        for sid in reversed(self.running):
            seq = self.sequences[sid]
            if seq.cache is None or not any(seq.cache.pages_held(g) for g in range(len(self.manager.groups))):
                continue  # holds no pages: preempting it would free nothing
            self.manager.close(seq.cache)
            seq.cache = None
            seq.status = SeqStatus.Waiting
            self.running.remove(sid)
            self.waiting.appendleft(sid)
            self.preemptions += 1
            return True
        return False

    def schedule(self) -> List[ScheduledItem]:
        """Admit, then choose the tokens of the next step (possibly none)."""
        self._admit()
        while True:
            items = self._build()
            if items or len(self.running) <= 1 or not self._preempt_youngest():
                return items

    def lookahead(self, items: List[ScheduledItem]) -> Optional[List[ScheduledItem]]:
        """The step after ``items`` (launched, samples not read yet), or None if it cannot be
        told without them.  Its tokens are stand-ins: the ids come from the device."""
        if self.waiting or not items or len(items) != len(self.running) or len(items) > self.max_tokens_per_step:
            return None
        taken = [0] * len(self.manager.groups)
        for item, sid in zip(items, self.running):
            seq = item.seq
            if seq.id != sid or not item.wants_logits or seq.status != SeqStatus.Running or seq.cache is None:
                return None
            if seq.remaining != 0:
                return None  # not everything it has is computed: it is still in its prompt
            if len(seq.output) + 1 >= seq.request.max_tokens:
                return None  # the pending sample is its last token
            for g, k in enumerate(self.manager.new_pages_needed(seq.cache, 1)):
                taken[g] += k
        if any(taken[g] > self.manager.free_pages(g) for g in range(len(taken))):
            return None
        return [ScheduledItem(item.seq, [0], True, ahead=True) for item in items]

    def finish_step(self, items: List[ScheduledItem], sampled: List[Optional[int]]) -> List[int]:
        """Record the tokens sampled for the items that wanted logits (``None`` for the others);
        returns the ids of the requests that finished.  The sample of a request that has ended
        meanwhile (it had run ahead) is dropped."""
        done = []
        for item, token in zip(items, sampled):
            if not item.wants_logits or item.seq.status != SeqStatus.Running:
                continue
            seq = item.seq
            seq.output.append(int(token))
            req = seq.request
            if (req.eos_id >= 0 and token == req.eos_id) or len(seq.output) >= req.max_tokens:
                seq.status = SeqStatus.Finished
                self.manager.close(seq.cache)
                seq.cache = None
                self.running.remove(seq.id)
                done.append(seq.id)
        return done
