"""A generation request and its progress (reference: src/dli/engine/request.py:13-66)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, IntEnum
from typing import Optional

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"    # queued, or preempted and waiting to be recomputed
    RUNNING = "running"    # holds cache and is scheduled every step
    FINISHED = "finished"


class FinishReason(str, Enum):
    STOP = "stop"          # emitted an end-of-sequence or stop token
    LENGTH = "length"      # reached max_tokens
    ABORTED = "aborted"    # cancelled by the caller
    CAPACITY = "capacity"  # can never fit the cache pool: rejected, never runs

    def __str__(self) -> str:
        return self.value


class Priority(IntEnum):
    """Scheduling class; the lower value is served first."""

    INTERACTIVE = 0
    BATCH = 1


@dataclass(eq=False)
class Request:
    """``num_computed_tokens`` counts tokens whose keys are in the cache; after a preemption it
    drops to 0 and the request recomputes ``prompt + outputs`` when it is admitted again.
    ``seed`` keys the request's random stream; draw ``n`` of it samples output token ``n``."""

    request_id: str
    prompt_ids: list[int]
    params: SamplingParams
    arrival_seq: int
    priority: Priority = Priority.INTERACTIVE
    tenant: str = "default"
    seed: Optional[int] = None
    output_ids: list[int] = field(default_factory=list)
    status: RequestStatus = RequestStatus.WAITING
    finish_reason: Optional[FinishReason] = None
    num_computed_tokens: int = 0
    num_preemptions: int = 0
    arrival_step: int = 0

    @property
    def all_token_ids(self) -> list[int]:
        return self.prompt_ids + self.output_ids

    def token_slice(self, begin: int, end: int) -> list[int]:
        """Tokens ``[begin, end)`` of prompt followed by output, without joining the two lists."""
        n_prompt = len(self.prompt_ids)
        if end <= n_prompt:
            return self.prompt_ids[begin:end]
        if begin >= n_prompt:
            return self.output_ids[begin - n_prompt:end - n_prompt]
        return self.prompt_ids[begin:] + self.output_ids[:end - n_prompt]

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_ids) + len(self.output_ids)

    @property
    def is_finished(self) -> bool:
        return self.status is RequestStatus.FINISHED
