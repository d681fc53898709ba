"""Continuous batching with chunked prefill: which tokens of which requests run next.

Every step gets a token budget (``max_num_batched_tokens``) and a cap on live requests
(``max_num_seqs``). Running requests are served first, each with its next decoded token or the
next portion of its unfinished prompt; then waiting requests are admitted while budget, cap and
cache allow, a prompt longer than the budget left being cut into portions that continue in later
steps (reference: src/dli/engine/scheduler.py:1-21,151-214).

**When pages run out** a running request that needs a page makes the newest-admitted running
request that is not yet in this step's batch give up its cache (preemption by recompute: its pages
are freed, its outputs kept, it goes to the front of the waiting queue and later recomputes
``prompt + outputs`` as a prompt, reusing what the content index still holds); if no other request
can yield, the requester preempts itself. No request is admitted in a step that preempted. A
request whose prompt plus ``max_tokens`` can never fit the pool is rejected on arrival
(``CAPACITY``), which guarantees that the oldest running request can always finish: the engine
cannot livelock (:102-120, :244-267).

The scheduler sees requests, pages and slots, never tensors.
"""

from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Mapping, Optional

from ..cache.manager import CacheManager, CopyOp, NoFreePagesError
from .request import FinishReason, Priority, Request, RequestStatus


@dataclass(frozen=True)
class SchedulerConfig:
    """Limits of a step (reference: src/dli/engine/scheduler.py:32-58).

    ``namespace`` scopes content reuse of cache pages (model and weights identity);
    ``tenant_weights`` gives tenants a weighted fair share of admissions; after ``aging_steps``
    steps of waiting a request counts as INTERACTIVE. ``decode_steps`` > 1 lets a step in which
    every request decodes, nobody waits and the cache has room run up to that many tokens of each
    request on the device before the host sees them (the reference has no counterpart; 1 keeps
    its behaviour).
    """

    max_num_seqs: int = 64
    max_num_batched_tokens: int = 512
    namespace: bytes = b""
    tenant_weights: Mapping[str, float] = field(default_factory=dict)
    aging_steps: int = 200
    decode_steps: int = 1

    def __post_init__(self) -> None:
        if self.max_num_seqs < 1 or self.max_num_batched_tokens < 1:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be >= 1")
        if self.decode_steps < 1:
            raise ValueError("decode_steps must be >= 1")
        if self.aging_steps < 1:
            raise ValueError("aging_steps must be >= 1")
        if any(w <= 0 for w in self.tenant_weights.values()):
            raise ValueError("tenant weights must be positive")


@dataclass(frozen=True)
class ScheduledChunk:
    """Run ``num_tokens`` tokens of ``request`` from absolute position ``start``. ``needs_logits``:
    the chunk reaches the request's last known token, so a new token is sampled after it."""

    request: Request
    start: int
    num_tokens: int
    needs_logits: bool


@dataclass
class SchedulerOutput:
    chunks: list[ScheduledChunk] = field(default_factory=list)
    copy_ops: list[CopyOp] = field(default_factory=list)
    preempted: list[Request] = field(default_factory=list)
    decode_steps: int = 1  # tokens that each chunk's request decodes in this step (all chunks decode if > 1)

    @property
    def num_batched_tokens(self) -> int:
        return sum(c.num_tokens for c in self.chunks)


class Scheduler:
    def __init__(self, config: SchedulerConfig, manager: CacheManager) -> None:
        if config.max_num_seqs > manager.slots.num_slots:
            raise ValueError(
                f"max_num_seqs={config.max_num_seqs} exceeds the cache's {manager.slots.num_slots} state slots")
        self.config = config
        self.manager = manager
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self._by_id: dict[str, Request] = {}
        self._step = 0
        self._vtime: dict[str, float] = {}  # tokens served / weight, per tenant

    # ------------------------------------------------------------------ lifecycle

    def add(self, req: Request) -> bool:
        """Queue a request; False (finished with CAPACITY) if it could never fit the pool alone."""
        if req.request_id in self._by_id:
            raise ValueError(f"duplicate request id {req.request_id!r}")
        worst_case = len(req.prompt_ids) + req.params.max_tokens
        if -(-worst_case // self.manager.page_size) > self.manager.num_pages:
            req.status = RequestStatus.FINISHED
            req.finish_reason = FinishReason.CAPACITY
            return False
        self._by_id[req.request_id] = req
        req.arrival_step = self._step
        self._activate_tenant(req.tenant)
        self.waiting.append(req)
        return True

    def finish(self, req: Request, reason: FinishReason) -> None:
        """Give back the request's cache and take it out of scheduling."""
        if req.status is RequestStatus.RUNNING:
            self.manager.free(req.request_id)
            self.running.remove(req)
        elif req.status is RequestStatus.WAITING:
            self.waiting.remove(req)
        req.status = RequestStatus.FINISHED
        req.finish_reason = reason
        self._by_id.pop(req.request_id, None)

    def abort(self, request_id: str) -> Optional[Request]:
        """Cancel a queued or running request (None for unknown or finished ids)."""
        req = self._by_id.get(request_id)
        if req is None:
            return None
        self.finish(req, FinishReason.ABORTED)
        return req

    @property
    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ one step's decision

    def schedule(self) -> SchedulerOutput:
        """Decide the next step: running requests first, then admissions."""
        plan = SchedulerOutput()
        left = self._serve_running(plan, self.config.max_num_batched_tokens)
        if not plan.preempted:  # memory that was just freed serves running requests first
            self._admit_waiting(plan, left)
        plan.decode_steps = self._decode_steps(plan)
        self._step += 1
        return plan

    def _decode_steps(self, plan: SchedulerOutput) -> int:
        """How many tokens each request of the step may decode before the host looks again: more
        than one only if the step is all decoding, nobody waits for admission, nothing was
        preempted or has to be copied, and the pages for the extra tokens can be reserved now.
        Never more than the request with the fewest tokens left may still produce."""
        k = self.config.decode_steps
        if k <= 1 or not plan.chunks or self.waiting or plan.preempted or plan.copy_ops:
            return 1
        for ch in plan.chunks:
            if ch.num_tokens != 1 or not ch.needs_logits:
                return 1
            k = min(k, ch.request.params.max_tokens - len(ch.request.output_ids))
        if k <= 1:
            return 1
        try:
            for ch in plan.chunks:
                self.manager.reserve_ahead(ch.request.request_id, k - 1)
        except NoFreePagesError:
            return 1  # what was reserved so far stays with its requests and is used later
        return k

    def _serve_running(self, plan: SchedulerOutput, budget: int) -> int:
        """Give each running request its next token or portion; returns the budget left."""
        # Victims are taken from the end of this order, so its front always progresses.
        self.running.sort(key=lambda r: (self._effective_priority(r), r.arrival_seq))
        placed: set[str] = set()
        for req in tuple(self.running):
            if budget <= 0:
                break
            if req.status is not RequestStatus.RUNNING:
                continue  # lost its cache to an earlier request of this loop
            take = min(req.num_tokens - req.num_computed_tokens, budget)
            if take <= 0:
                continue
            copies = self._reserve(req)
            while copies is None:
                victim = self._newest_outside(placed | {req.request_id})
                if victim is None:
                    victim = req  # nobody else can yield: the requester gives up its own cache
                self._preempt(victim)
                plan.preempted.append(victim)
                if victim is req:
                    break
                copies = self._reserve(req)
            if copies is None:
                continue
            plan.copy_ops.extend(copies)
            self._place(plan, req, take)
            placed.add(req.request_id)
            budget -= take
        return budget

    def _admit_waiting(self, plan: SchedulerOutput, budget: int) -> int:
        """Admit waiting requests in order of merit while budget, cap and cache allow."""
        cfg = self.config
        while self.waiting and budget > 0 and len(self.running) < cfg.max_num_seqs:
            req = min(self.waiting, key=self._admission_key)
            tokens = req.all_token_ids
            if not self.manager.can_allocate(tokens, cfg.namespace):
                break  # the most deserving request waits for memory; nobody overtakes it
            grant = self.manager.allocate(req.request_id, tokens, namespace=cfg.namespace)
            self.waiting.remove(req)
            self.running.append(req)
            req.status = RequestStatus.RUNNING
            req.num_computed_tokens = grant.num_cached_tokens
            take = min(len(tokens) - grant.num_cached_tokens, budget)
            self._place(plan, req, take)
            budget -= take
        return budget

    def _place(self, plan: SchedulerOutput, req: Request, take: int) -> None:
        begin = req.num_computed_tokens
        plan.chunks.append(ScheduledChunk(req, begin, take, needs_logits=begin + take == req.num_tokens))
        self._vtime[req.tenant] += take / self.config.tenant_weights.get(req.tenant, 1.0)

    # ------------------------------------------------------------------ fairness

    def _effective_priority(self, req: Request) -> int:
        if self._step - req.arrival_step >= self.config.aging_steps:
            return int(Priority.INTERACTIVE)
        return int(req.priority)

    def _admission_key(self, req: Request) -> tuple[int, int, float, int]:
        resumed = 0 if req.num_preemptions else 1  # preempted requests held a place already
        return (self._effective_priority(req), resumed, self._vtime[req.tenant], req.arrival_seq)

    def _activate_tenant(self, tenant: str) -> None:
        """A tenant that was idle starts at the current virtual clock: no credit is banked."""
        active = {r.tenant for r in self.waiting} | {r.tenant for r in self.running}
        active.discard(tenant)
        clock = min((self._vtime[t] for t in active), default=0.0)
        self._vtime[tenant] = max(self._vtime.get(tenant, 0.0), clock)

    # ------------------------------------------------------------------ memory pressure

    def _newest_outside(self, exclude: set[str]) -> Optional[Request]:
        """The running request admitted last among those not in ``exclude``."""
        return next((r for r in reversed(self.running) if r.request_id not in exclude), None)

    def _preempt(self, req: Request) -> None:
        self.manager.free(req.request_id)
        self.running.remove(req)
        req.status = RequestStatus.WAITING
        req.num_computed_tokens = 0
        req.num_preemptions += 1
        self.waiting.appendleft(req)

    def _reserve(self, req: Request) -> Optional[list[CopyOp]]:
        """Reserve cache slots for tokens the manager has not seen (the newly sampled one)."""
        missing = req.num_tokens - self.manager.num_tokens(req.request_id)
        if missing <= 0:
            return []
        try:
            total = req.num_tokens
            return self.manager.append_slots(req.request_id, req.token_slice(total - missing, total))
        except NoFreePagesError:
            return None
