"""Continuous batching: who runs in the next step, with how many tokens.

Every step is mixed by construction: each decoding request brings one token,
requests that are still reading their prompt bring a portion of it, and new
requests are admitted while the budget lasts.  The reference alternates
prefill turns and decode turns by a ratio and runs a "mixed" step as separate
calls (zstreamer/scheduler.py:199-223, zstreamer/batch_runner.py:96-102); its
names are kept where it has them: ``max_batch_tokens`` (4096),
``prefill_chunk_size`` (512), ``max_batch_seqs`` (64) (zstreamer/scheduler.py:83-104).

Order within a step: (1) running requests, oldest first: one token for a
decoding request, min(remaining, chunk, budget left) for one inside its
prompt; (2) waiting requests, preempted ones first, then by arrival, each with
its first portion, while requests, slots, budget and pages allow.

When pages run out (the reference raises inside ``extend_sequence`` and fails
the whole batch, cache/cache_manager.py:256-261, zstreamer/batch_runner.py:305-309):
a running request that cannot get pages for its step makes the most recently
admitted running request give up everything it holds; that request goes to
the front of the queue and is computed again from its prompt and the tokens
it has produced.  If the request itself is the last one left and still does
not fit, it ends with an error.  Admission never preempts.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

from ..cache.manager import CacheManager
from ..cache.slots import OutOfSlots
from .request import FinishReason, Request, RequestState


UNKNOWN_TOKEN = -1      # stands in an output for a token that has not reached the host yet


@dataclass
class SchedulerConfig:
    max_batch_tokens: int = 4096
    prefill_chunk_size: int = 512
    max_batch_seqs: int = 64


@dataclass
class Scheduled:
    request: Request
    start: int            # position of the first token of the portion
    count: int            # tokens in the portion
    sample: bool          # the portion ends the known tokens: its last logits give the next token


@dataclass
class StepPlan:
    items: List[Scheduled] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    failed: List[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(s.count for s in self.items)

    def __bool__(self):
        return bool(self.items)


class Scheduler:
    def __init__(self, config: SchedulerConfig, manager: CacheManager):
        if config.max_batch_tokens <= 0 or config.prefill_chunk_size <= 0 or config.max_batch_seqs <= 0:
            raise ValueError("scheduler limits must be positive")
        self.config = config
        self.manager = manager
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []         # in order of admission
        self.finished: Dict[object, Request] = {}
        self._arrivals = 0
        self.num_preemptions = 0
        self.steps = 0

    # ---- intake
    def add_request(self, req: Request) -> None:
        if not req.prompt_tokens:
            raise ValueError(f"request {req.request_id!r} has an empty prompt")
        if len(req.prompt_tokens) > self.manager.max_model_len:
            raise ValueError(f"request {req.request_id!r}: prompt of {len(req.prompt_tokens)} tokens "
                             f"exceeds the longest context, {self.manager.max_model_len}")
        req.arrival = self._arrivals
        req.arrival_time = time.monotonic()
        self._arrivals += 1
        req.state = RequestState.WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step
    def _portion(self, req: Request, budget: int) -> int:
        if req.state == RequestState.DECODING and req.remaining == 1:
            return 1 if budget >= 1 else 0
        return max(0, min(req.remaining, self.config.prefill_chunk_size, budget))

    def _preempt(self, victim: Request, plan: StepPlan) -> None:
        self.manager.release(victim.request_id)
        self.running.remove(victim)
        plan.items = [s for s in plan.items if s.request is not victim]
        victim.state = RequestState.PREEMPTED
        victim.num_computed = 0
        victim.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        plan.preempted.append(victim)

    def _fail(self, req: Request, why: str, plan: StepPlan) -> None:
        self.manager.release(req.request_id)
        if req in self.running:
            self.running.remove(req)
        req.state = RequestState.FINISHED
        req.finish_reason = FinishReason.ERROR
        req.finish_time = time.monotonic()
        req.error = why
        self.finished[req.request_id] = req
        plan.failed.append(req)

    def schedule(self) -> StepPlan:
        cfg, m = self.config, self.manager
        plan = StepPlan()
        budget = cfg.max_batch_tokens
        # (1) running requests, oldest first
        for req in list(self.running):
            if req not in self.running:        # preempted while an older request was served
                continue
            n = self._portion(req, budget)
            if n == 0:
                continue
            while not m.reserve(req.request_id, req.num_computed + n):
                victim = self.running[-1]
                if victim is req:
                    if len(self.running) == 1:
                        self._fail(req, f"needs pages for {req.num_computed + n} tokens; the cache "
                                        f"cannot hold them even alone", plan)
                    else:
                        self._preempt(req, plan)
                    n = 0
                    break
                self._preempt(victim, plan)
                budget = cfg.max_batch_tokens - plan.num_tokens
            if n == 0:
                continue
            plan.items.append(Scheduled(req, req.num_computed, n, req.num_computed + n == req.num_tokens))
            budget -= n
        # (2) admissions
        while self.waiting and budget > 0 and len(self.running) < cfg.max_batch_seqs:
            req = self.waiting[0]
            if m.slots.free_slots == 0 or req in plan.preempted:
                break       # a request that just gave up its pages does not take them back at once
            n = max(0, min(req.remaining, cfg.prefill_chunk_size, budget))
            if n == 0:
                break
            m.add(req.request_id)
            if not m.reserve(req.request_id, n):
                m.release(req.request_id)
                if not self.running:
                    self.waiting.popleft()
                    self._fail(req, f"needs pages for {n} tokens; the cache cannot hold them even "
                                    f"alone", plan)
                    continue
                break
            self.waiting.popleft()
            req.state = RequestState.PREFILLING
            req.num_computed = 0
            self.running.append(req)
            plan.items.append(Scheduled(req, 0, n, n == req.num_tokens))
            budget -= n
        self.steps += 1
        return plan

    # ---- after the step ran
    def on_step_done(self, plan: StepPlan, sampled: Dict[object, int]) -> List[Request]:
        """Advance every scheduled request; ``sampled`` maps the ids of requests whose
        portion ended their known tokens to the token drawn.  Returns those that finished."""
        done = []
        for s in plan.items:
            req = s.request
            req.num_computed += s.count
            self.manager.commit(req.request_id, req.num_computed)
            if not s.sample:
                continue
            known = sampled[req.request_id] is not None
            tok = int(sampled[req.request_id]) if known else UNKNOWN_TOKEN     # still on the device: set later
            req.output_tokens.append(tok)
            if req.first_token_time is None:
                req.first_token_time = time.monotonic()
            req.state = RequestState.DECODING
            reason = None
            if known and req.params.stop_tokens and tok in req.params.stop_tokens:
                reason = FinishReason.STOP
            elif len(req.output_tokens) >= req.params.max_tokens:
                reason = FinishReason.LENGTH
            elif req.num_tokens >= self.manager.max_model_len:
                reason = FinishReason.LENGTH
            if reason is not None:
                req.state = RequestState.FINISHED
                req.finish_reason = reason
                req.finish_time = time.monotonic()
                self.manager.release(req.request_id)
                self.running.remove(req)
                self.finished[req.request_id] = req
                done.append(req)
        return done

    def finish_at(self, req: Request, length: int, reason: FinishReason) -> bool:
        """A token that was still unknown when the request was stepped on turned out to end
        it: cut its output to ``length`` tokens and finish it now.  Returns True if the request
        was still running or waiting to run again (it is then reported as done by the caller),
        False if it had already finished for another reason."""
        del req.output_tokens[length:]
        was_live = False
        if req in self.running:
            self.running.remove(req)
            was_live = True
        elif req in self.waiting:
            # preempted after the step that drew the token, before the token was known: it
            # must not be admitted and computed again
            self.waiting.remove(req)
            was_live = True
        if was_live:
            self.manager.release(req.request_id)      # a request in the queue holds nothing: a no-op
            self.finished[req.request_id] = req
        req.state = RequestState.FINISHED
        req.finish_reason = reason
        req.finish_time = req.finish_time or time.monotonic()
        return was_live

    def stats(self) -> dict:
        return {"waiting": len(self.waiting), "running": len(self.running),
                "finished": len(self.finished), "preemptions": self.num_preemptions,
                "steps": self.steps}
