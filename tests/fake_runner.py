"""A deterministic stand-in for the model, for scheduler and engine tests on the CPU.

The next token is a hash of the *whole* history, so a scheduling fault that drops, repeats or
reorders tokens, or loses progress across a preemption, changes the output (the idea of the
reference's tests/unit/engine/fake.py). "Logits" are just the chosen token ids here; the matching
sampler below passes them through.
"""

from __future__ import annotations

import hashlib
from typing import Collection, Sequence

VOCAB = 50


def next_token(history: Sequence[int]) -> int:
    digest = hashlib.blake2b(repr(list(history)).encode("ascii"), digest_size=8).digest()
    return int.from_bytes(digest, "little") % VOCAB


def alone(prompt: Sequence[int], max_tokens: int, stop: Collection[int] = ()) -> list[int]:
    """What one request generates by itself."""
    toks, out = list(prompt), []
    for _ in range(max_tokens):
        t = next_token(toks)
        out.append(t)
        toks.append(t)
        if t in stop:
            break
    return out


class FakeRunner:
    def __init__(self, manager) -> None:
        self.manager = manager
        self.calls = []

    def execute(self, sched):
        self.calls.append(sched)
        picks = []
        for ch in sched.chunks:
            rid = ch.request.request_id
            assert self.manager.num_computed_tokens(rid) == ch.start, "chunk does not continue the cache"
            assert ch.num_tokens >= 1
            self.manager.slot_mapping(rid, ch.start, ch.start + ch.num_tokens)  # slots must be reserved
            self.manager.mark_computed(rid, ch.start + ch.num_tokens)
            if ch.needs_logits:
                picks.append(next_token(ch.request.all_token_ids[:ch.start + ch.num_tokens]))
        return picks

    # the interface of a runner that also samples, with several decoded tokens per step
    max_decode_steps = 8

    def execute_and_sample(self, sched):
        k = sched.decode_steps
        if k == 1:
            return self.execute(sched)
        self.calls.append(sched)
        rounds = [[] for _ in range(k)]
        for ch in sched.chunks:
            rid = ch.request.request_id
            assert ch.num_tokens == 1 and ch.needs_logits, "only decoding requests take several tokens a step"
            assert self.manager.num_computed_tokens(rid) == ch.start == self.manager.num_tokens(rid) - 1
            ps = self.manager.page_size
            assert len(self.manager.table_ref(rid)) * ps >= ch.start + k, "no room reserved ahead"
            history = ch.request.token_slice(0, ch.start + 1)
            for j in range(k):
                tok = next_token(history)
                rounds[j].append(tok)
                history.append(tok)
                if j < k - 1:
                    assert self.manager.append_slots(rid, [tok]) == []
            self.manager.mark_computed(rid, ch.start + k)
        return rounds


def passthrough_sampler(logits, params, seeds, draws):
    assert len(logits) == len(params) == len(seeds) == len(draws)
    return list(logits)
