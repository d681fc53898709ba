"""A generation request and its progress (reference: src/dli/engine/request.py:13-66)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum, IntEnum
from typing import Optional

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    """Where a request is: in the waiting queue (new, or put back there after it lost its pages),
    among the running ones (it owns pages and a state slot and gets tokens every step), or done."""

    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class FinishReason(str, Enum):
    """Why a request is done: its last token was a stop or end-of-sequence id (``stop``), it has
    ``max_tokens`` outputs (``length``), the caller cancelled it (``aborted``), or its prompt plus
    ``max_tokens`` exceeds the whole pool, so it was turned away on arrival (``capacity``)."""

    STOP = "stop"
    LENGTH = "length"
    ABORTED = "aborted"
    CAPACITY = "capacity"

    def __str__(self) -> str:
        return self.value


class Priority(IntEnum):
    """Class of service: a smaller number goes first, in admission and when victims are chosen."""

    INTERACTIVE = 0
    BATCH = 1


@dataclass(eq=False)
class Request:
    """What the caller gave (id, prompt, sampling parameters, class, tenant, seed) and how far the
    engine has come. ``num_computed_tokens`` of ``prompt + outputs`` are in the cache; a request
    that loses its pages starts again from 0 and runs its outputs so far as part of the prompt.
    Draw ``n`` of the random stream keyed by ``seed`` chooses output token ``n``, whatever else
    runs. ``arrival_seq`` orders requests of one class; ``arrival_step`` is the scheduler's step
    count when the request came, for aging."""

    request_id: str
    prompt_ids: list[int]
    params: SamplingParams
    arrival_seq: int
    priority: Priority = Priority.INTERACTIVE
    tenant: str = "default"
    seed: Optional[int] = None
    # progress
    status: RequestStatus = RequestStatus.WAITING
    output_ids: list[int] = field(default_factory=list)
    num_computed_tokens: int = 0
    finish_reason: Optional[FinishReason] = None
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
