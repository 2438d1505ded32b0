"""Host-side state of one request and the records the engine hands out
(reference: ullm/core/common.py:22-43,57-179)."""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import List, Optional

from ..cache.manager import RequestCache
from ..sampling.params import SamplingParams


class FinishReason(enum.Enum):
    STOP = enum.auto()       # the end-of-sequence token was produced
    LENGTH = enum.auto()     # a length cap (or the cache's capacity) was reached


class RequestStatus(enum.Enum):
    WAITING = enum.auto()
    RUNNING = enum.auto()
    FINISHED = enum.auto()


@dataclass
class Request:
    request_id: str
    token_ids: List[int]                      # prompt followed by generated tokens
    num_prompt_tokens: int
    params: SamplingParams
    seed: int
    order: int                                # arrival number: first come, first served
    status: RequestStatus = RequestStatus.WAITING
    cache: Optional[RequestCache] = None      # held while RUNNING
    finish_reason: Optional[FinishReason] = None
    num_preemptions: int = 0

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def num_generated_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def num_computed(self) -> int:
        return self.cache.num_computed if self.cache is not None else 0

    @property
    def generated_token_ids(self) -> List[int]:
        return self.token_ids[self.num_prompt_tokens:]


@dataclass
class Scheduled:
    """One request's share of a step: ``num_tokens`` tokens from position ``start``; the step
    samples for it only if the share reaches the end of what is known of the request."""
    request: Request
    start: int
    num_tokens: int
    samples: bool = False

    def __post_init__(self):
        self.samples = self.start + self.num_tokens == self.request.num_tokens


@dataclass
class EngineStepResult:
    """As the reference's record of the same name (ullm/core/common.py:36-43)."""
    seq_id: str
    new_token_id: int
    is_finished: bool
    finish_reason: Optional[FinishReason]
    num_prompt_tokens: int
    num_generated_tokens: int
