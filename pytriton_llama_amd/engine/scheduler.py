"""The continuous-batching scheduler.

The reference has none: its generate loop runs one static batch, reserves the
cache for batch x (prompt + max_gen) tokens up front and keeps computing finished
rows until all are done (lite_llama/generate_stream.py:116-188; README.md lists
continuous batching as future work). This one is host-side logic only. Every
step it decides which requests run how many tokens:

* requests that are decoding come first, one token each;
* what is left of the token budget goes to prompts, in order of arrival, in
  portions of at most ``prefill_chunk`` tokens, so a long prompt spans several
  steps and shares them with decodes;
* waiting requests are admitted in order of arrival while a state slot, a place
  in the batch and the pages of their first portion are there;
* when a running request cannot get the page it needs, the most recently
  admitted running request is preempted: its pages and slot are given back, it
  returns to the front of the waiting queue and is computed again from its
  prompt plus the tokens it had generated (which are kept). If the request in
  need is itself the most recent one, it is the one that waits;
* a request that could never fit (prompt + max_new_tokens beyond the pool or
  beyond max_model_len) is refused when it is added.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from .request import FINISHED, RUNNING, WAITING, Request, StepOutput


@dataclass
class PlannedEntry:
    request: Request
    start: int              # position of the first token of the portion
    num_tokens: int
    samples: bool           # the portion ends the known tokens: its last logits are sampled


@dataclass
class StepPlan:
    entries: List[PlannedEntry] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(e.num_tokens for e in self.entries)


class Scheduler:
    def __init__(self, manager, max_num_seqs: int, max_num_batched_tokens: int,
                 prefill_chunk: Optional[int] = None, max_model_len: Optional[int] = None,
                 eos_token_ids: Sequence[int] = ()):
        self.manager = manager
        self.max_num_seqs = min(int(max_num_seqs), manager.max_num_seqs)
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.prefill_chunk = int(prefill_chunk) if prefill_chunk else self.max_num_batched_tokens
        self.max_model_len = max_model_len
        self.eos_token_ids = tuple(eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []          # in order of admission
        self.num_preemptions = 0

    # ---- submitting -----------------------------------------------------------
    def add(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError(f"request {req.id!r} has an empty prompt")
        total = len(req.prompt) + req.params.max_new_tokens
        if self.max_model_len is not None and total > self.max_model_len:
            raise ValueError(f"request {req.id!r}: prompt ({len(req.prompt)}) + max_new_tokens "
                             f"({req.params.max_new_tokens}) exceeds max_model_len {self.max_model_len}")
        P = self.manager.page_size
        for g in self.manager.paged:
            if -(-total // P) > g.pool.num_pages and g.spec.window is None:
                raise ValueError(f"request {req.id!r} needs {-(-total // P)} pages, the pool has "
                                 f"{g.pool.num_pages}: it can never fit")
        req.status = WAITING
        self.waiting.append(req)

    @property
    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning one step -------------------------------------------------------
    def _preempt(self, victim: Request, plan: StepPlan, reserve: List[int]) -> None:
        for e in list(plan.entries):
            if e.request is victim:
                plan.entries.remove(e)
                for g, n in enumerate(self.manager.pages_needed(victim.id, e.num_tokens)):
                    reserve[g] -= n
        if self.manager.is_live(victim.id):
            self.manager.free(victim.id)
        self.running.remove(victim)
        victim.num_computed = 0
        victim.status = WAITING
        victim.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        plan.preempted.append(victim)

    def _try_plan(self, req: Request, n: int, plan: StepPlan, reserve: List[int]) -> bool:
        """Plan n tokens of a running request, preempting later arrivals while
        pages are short. False when the request itself had to give way."""
        while not self.manager.can_append(req.id, n, reserve):
            victim = self.running[-1]
            self._preempt(victim, plan, reserve)
            if victim is req:
                return False
        for g, k in enumerate(self.manager.pages_needed(req.id, n)):
            reserve[g] += k
        plan.entries.append(PlannedEntry(req, req.num_computed, n, req.num_computed + n == req.num_tokens))
        return True

    def schedule(self) -> StepPlan:
        plan = StepPlan()
        reserve = [0] * len(self.manager.paged)
        budget = self.max_num_batched_tokens
        # 1. decodes, in order of admission
        for req in list(self.running):
            if req.status != RUNNING or req.remaining != 1 or budget <= 0:
                continue
            if self._try_plan(req, 1, plan, reserve):
                budget -= 1
        # 2. portions of prompts that are already running
        for req in list(self.running):
            if req.status != RUNNING or req.remaining <= 1 or budget <= 0:
                continue
            n = min(req.remaining, self.prefill_chunk, budget)
            if self._try_plan(req, n, plan, reserve):
                budget -= n
        # 3. admissions, in order of arrival, never past a request that does not fit
        slots_left = self.manager.num_free_slots
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and slots_left > 0:
            req = self.waiting[0]
            if req in plan.preempted:
                break                           # just preempted: it waits at least one step
            n = min(req.remaining, self.prefill_chunk, budget)
            if not self.manager.can_append(req.id, n, reserve):
                break
            self.waiting.popleft()
            req.status = RUNNING
            self.running.append(req)
            slots_left -= 1
            for g, k in enumerate(self.manager.pages_needed(req.id, n)):
                reserve[g] += k
            plan.entries.append(PlannedEntry(req, req.num_computed, n, req.num_computed + n == req.num_tokens))
            budget -= n
        if not plan.entries and self.has_work:
            raise RuntimeError("the scheduler can make no progress: no request fits the free pages")
        return plan

    def plan_ahead(self, plan: StepPlan) -> Optional[StepPlan]:
        """The step after ``plan``, decided before ``plan``'s tokens are known (its step is
        running and has taken its pages, ``update`` has not been called for it): possible when
        ``plan`` decodes every running request, nobody waits, none of them reaches a length
        limit with the token on its way, and each can get the page it may need. Whether a
        request stops at an end-of-sequence token is not known yet: it is planned, and
        ``update`` drops what was computed for it. None when the step has to be planned the
        ordinary way."""
        if self.waiting or plan.preempted or len(plan.entries) != len(self.running) or not plan.entries:
            return None
        nxt = StepPlan()
        reserve = [0] * len(self.manager.paged)
        for e in plan.entries:
            req = e.request
            if e.num_tokens != 1 or not e.samples or req.status != RUNNING:
                return None
            if len(req.output) + 2 > req.params.max_new_tokens:
                return None                     # the token on its way is its last
            if self.max_model_len is not None and req.num_tokens + 2 > self.max_model_len:
                return None
            if not self.manager.can_append(req.id, 1, reserve):
                return None
            for g, k in enumerate(self.manager.pages_needed(req.id, 1)):
                reserve[g] += k
            nxt.entries.append(PlannedEntry(req, e.start + 1, 1, True))
        return nxt

    # ---- after the step ------------------------------------------------------------
    def update(self, plan: StepPlan, sampled: Dict[Hashable, int]) -> List[StepOutput]:
        """Record what the step computed; ``sampled`` maps the id of every entry
        that samples to its new token. Finished requests give back what they hold."""
        outs: List[StepOutput] = []
        for e in plan.entries:
            req = e.request
            if req.status == FINISHED:
                continue            # planned ahead of the token that ended it: nothing to record
            req.num_computed += e.num_tokens
            if not e.samples:
                continue
            tok = int(sampled[req.id])
            req.output.append(tok)
            reason = None
            if not req.params.ignore_eos and tok in self.eos_token_ids:
                reason = "eos"
            elif len(req.output) >= req.params.max_new_tokens:
                reason = "length"
            elif self.max_model_len is not None and req.num_tokens >= self.max_model_len:
                reason = "max_model_len"
            if reason is not None:
                req.status = FINISHED
                req.finish_reason = reason
                self.running.remove(req)
                if self.manager.is_live(req.id):
                    self.manager.free(req.id)
            outs.append(StepOutput(req.id, tok, reason is not None, reason))
        return outs

    def abort(self, req: Request) -> None:
        if req in self.running:
            self.running.remove(req)
            if self.manager.is_live(req.id):
                self.manager.free(req.id)
        elif req in self.waiting:
            self.waiting.remove(req)
        req.status = FINISHED
        req.finish_reason = "aborted"
