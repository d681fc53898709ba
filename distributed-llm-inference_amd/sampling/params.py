"""Per-request sampling settings; names, defaults and limits are the reference's
(src/dli/sampling.py:22-56)."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class SamplingParams:
    """
    Attributes:
        max_tokens: most tokens to generate.
        temperature: 0 selects greedy decoding (argmax, lowest id on ties); at most 2.
        top_k: keep the k most likely tokens; -1 switches it off.
        top_p: nucleus sampling: a token is dropped iff strictly more likely tokens already hold
            this much probability.
        seed: seed of this request's random draws; ``None``: the engine draws one.
        stop_token_ids: generation stops after emitting any of these (the token stays in the output).
        ignore_eos: do not stop at the engine's end-of-sequence ids.
    """

    max_tokens: int = 16
    temperature: float = 0.0
    top_k: int = -1
    top_p: float = 1.0
    seed: Optional[int] = None
    stop_token_ids: tuple[int, ...] = ()
    ignore_eos: bool = False

    def __post_init__(self) -> None:
        if self.max_tokens < 1:
            raise ValueError("max_tokens must be >= 1")
        if math.isnan(self.temperature) or not 0.0 <= self.temperature <= 2.0:
            raise ValueError("temperature must be in [0, 2]")
        if self.top_k == 0 or self.top_k < -1:
            raise ValueError("top_k must be -1 (disabled) or >= 1")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1]")
        object.__setattr__(self, "stop_token_ids", tuple(self.stop_token_ids))

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0 or self.top_k == 1
