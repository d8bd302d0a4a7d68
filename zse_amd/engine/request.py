"""A request's record through its life.

States and finish reasons follow the reference (zstreamer/request.py:18-35):
WAITING -> PREFILLING -> DECODING -> FINISHED, with PREEMPTED for a request
whose pages were taken and which waits to be computed again.  ``num_computed``
stands where the reference has ``prefill_offset`` and also covers that
recomputation: it counts the tokens of ``prompt + output`` whose keys are in
the cache.
"""
from __future__ import annotations

import enum
import time
from dataclasses import dataclass, field
from typing import List, Optional

from ..sampling.sampler import SamplingParams


class RequestState(enum.Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    DECODING = "decoding"
    PREEMPTED = "preempted"
    FINISHED = "finished"


class FinishReason(enum.Enum):
    LENGTH = "length"     # max_tokens, or the model's longest context, reached
    STOP = "stop"         # a stop token was produced
    ERROR = "error"       # the request cannot be served (it does not fit the cache alone)


@dataclass(eq=False)      # a request is itself: lists of requests are searched by identity, not by comparing every field
class Request:
    request_id: object
    prompt_tokens: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    seed: int = 0
    state: RequestState = RequestState.WAITING
    output_tokens: List[int] = field(default_factory=list)
    num_computed: int = 0
    finish_reason: Optional[FinishReason] = None
    error: Optional[str] = None
    arrival: int = 0
    num_preemptions: int = 0
    # clock readings (time.monotonic) for the timing figures below
    arrival_time: float = 0.0
    first_token_time: Optional[float] = None
    finish_time: Optional[float] = None

    @property
    def all_tokens(self) -> List[int]:
        return self.prompt_tokens + self.output_tokens

    def tokens_at(self, start: int, count: int) -> List[int]:
        """``all_tokens[start:start + count]`` without putting the two lists together."""
        np_ = len(self.prompt_tokens)
        if start + count <= np_:
            return self.prompt_tokens[start:start + count]
        if start >= np_:
            return self.output_tokens[start - np_:start - np_ + count]
        return self.prompt_tokens[start:] + self.output_tokens[:start + count - np_]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_tokens) + len(self.output_tokens)

    @property
    def remaining(self) -> int:
        """Tokens known but not yet in the cache."""
        return self.num_tokens - self.num_computed

    def penalty_counts(self) -> dict:
        """Token id -> count for the repetition penalty, as the reference's continuous-batching
        engine keeps it: every token of the prompt counts once however often it occurs
        (zstreamer/engine.py:441), every produced token adds one (zstreamer/request.py:164).
        The sampler scales the penalty by these counts (orchestrator/sampler.py:64-74)."""
        counts = {int(t): 1 for t in self.prompt_tokens}
        for t in self.output_tokens:
            counts[int(t)] = counts.get(int(t), 0) + 1
        return counts

    # ---- timing, with the reference's names and meanings (zstreamer/request.py:206-228)
    @property
    def total_time_ms(self) -> float:
        return ((self.finish_time or time.monotonic()) - self.arrival_time) * 1000.0

    @property
    def ttft_ms(self) -> float:
        """Time to the first token; the whole time for a request that never produced one."""
        if self.first_token_time is None:
            return self.total_time_ms
        return (self.first_token_time - self.arrival_time) * 1000.0

    @property
    def tpot_ms(self) -> float:
        """Mean time per output token after the first."""
        if self.first_token_time is None:
            return self.total_time_ms
        end = self.finish_time or time.monotonic()
        return (end - self.first_token_time) * 1000.0 / max(len(self.output_tokens), 1)

    @property
    def tokens_per_sec(self) -> float:
        total = self.total_time_ms
        return max(len(self.output_tokens), 1) / (total / 1000.0) if total > 0 else 0.0

    @property
    def finished(self) -> bool:
        return self.state == RequestState.FINISHED
