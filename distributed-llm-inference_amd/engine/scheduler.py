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
from typing import Iterable, Mapping, Optional

from ..cache.manager import CacheManager, CopyOp, NoFreePagesError
from .request import FinishReason, Priority, Request, RequestStatus


@dataclass(frozen=True)
class SchedulerConfig:
    """Limits of a step; names and defaults as in src/dli/engine/scheduler.py:32-58.

    ``namespace`` keeps the cache pages of different models or weights apart in the content
    index. ``tenant_weights``: share of admitted work per tenant (absent tenants weigh 1).
    A request that has waited ``aging_steps`` steps is treated as INTERACTIVE whatever its class.
    ``decode_steps`` > 1 lets a step in which every request decodes, nobody waits and the cache
    has room run up to that many tokens of each request on the device before the host sees them
    (the reference has no counterpart; 1 keeps its behaviour).
    """

    max_num_seqs: int = 64
    max_num_batched_tokens: int = 512
    namespace: bytes = b""
    tenant_weights: Mapping[str, float] = field(default_factory=dict)
    aging_steps: int = 200
    decode_steps: int = 1

    def __post_init__(self) -> None:
        for name in ("max_num_seqs", "max_num_batched_tokens", "aging_steps", "decode_steps"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be at least 1, got {getattr(self, name)}")
        bad = {t: w for t, w in self.tenant_weights.items() if not w > 0}
        if bad:
            raise ValueError(f"a tenant's weight must be positive: {bad}")


class TenantLedger:
    """Who is owed the next admission among tenants.

    Every token placed into a step is charged to its request's tenant, divided by the tenant's
    weight; the tenant with the smallest charge is served first, so over time tokens are
    admitted in proportion to the weights. A tenant that had nothing in the system and comes
    back is lifted to the smallest charge among the tenants present: idle time earns nothing.
    """

    def __init__(self, weights: Mapping[str, float]) -> None:
        self._weights = dict(weights)
        self._charge: dict[str, float] = {}

    def enter(self, tenant: str, present: Iterable[str]) -> None:
        """``tenant`` brings a request while the tenants in ``present`` have requests queued or
        running. One that is present itself keeps its figure."""
        present = set(present)
        if tenant in present:
            return
        floor = min((self._charge[t] for t in present if t in self._charge), default=0.0)
        self._charge[tenant] = max(self._charge.get(tenant, 0.0), floor)

    def charge(self, tenant: str, tokens: int) -> None:
        self._charge[tenant] = self._charge.get(tenant, 0.0) + tokens / self._weights.get(tenant, 1.0)

    def owed(self, tenant: str) -> float:
        """Smaller is served sooner."""
        return self._charge.get(tenant, 0.0)


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
        self.ledger = TenantLedger(config.tenant_weights)

    # ------------------------------------------------------------------ lifecycle

    def add(self, req: Request) -> bool:
        """Queue a request. One whose prompt plus ``max_tokens`` needs more pages than the pool
        has is finished at once with CAPACITY and False comes back: admitted later it could
        block the queue for ever."""
        if req.request_id in self._by_id:
            raise ValueError(f"duplicate request id {req.request_id!r}")
        pages_at_most = -(-(len(req.prompt_ids) + req.params.max_tokens) // self.manager.page_size)
        if pages_at_most > self.manager.num_pages:
            req.status, req.finish_reason = RequestStatus.FINISHED, FinishReason.CAPACITY
            return False
        self.ledger.enter(req.tenant, [r.tenant for r in self._by_id.values()])
        req.arrival_step = self._step
        self._by_id[req.request_id] = req
        self.waiting.append(req)
        return True

    def _release(self, req: Request, becomes: RequestStatus, reason: Optional[FinishReason] = None) -> None:
        """Take ``req`` out of the queue it is in, returning its pages and state slot if it has
        any, and leave it ``becomes``: FINISHED (with ``reason``) or WAITING (preempted: it keeps
        its outputs, forgets what was computed and goes to the head of the waiting queue)."""
        if req.status is RequestStatus.RUNNING:
            self.manager.free(req.request_id)
            self.running.remove(req)
        elif req.status is RequestStatus.WAITING:
            self.waiting.remove(req)
        req.status = becomes
        if becomes is RequestStatus.FINISHED:
            req.finish_reason = reason
            self._by_id.pop(req.request_id, None)
        else:
            req.num_computed_tokens = 0
            req.num_preemptions += 1
            self.waiting.appendleft(req)

    def finish(self, req: Request, reason: FinishReason) -> None:
        self._release(req, RequestStatus.FINISHED, reason)

    def abort(self, request_id: str) -> Optional[Request]:
        """Cancel a request wherever it is; None if the id is unknown or already finished."""
        req = self._by_id.get(request_id)
        if req is not None:
            self._release(req, RequestStatus.FINISHED, FinishReason.ABORTED)
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
        # The step runs its chunks in this order: single tokens first (as the step function lays
        # them out anyway), those with the most keys first. The decode attention's workgroups start
        # in row order, and with rows of 128 to 2,300 keys as they come the launch ended with a few
        # long rows alone on the device (64 such rows at the 3B sizes: 69 us a layer, 59 sorted).
        plan.chunks.sort(key=lambda c: (0, -c.start) if c.num_tokens == 1 else (1, 0))
        self._step += 1
        return plan

    def _decode_steps(self, plan: SchedulerOutput) -> int:
        """How many tokens each request of the step may decode before the host looks again: more
        than one only if the step is all decoding, nobody waits for admission, nothing was
        preempted or has to be copied, and the pages for the extra tokens can be reserved now.
        Never more than the request with the fewest tokens left may still produce, and a power of two."""
        k = self.config.decode_steps
        if k <= 1 or not plan.chunks or self.waiting or plan.preempted or plan.copy_ops:
            return 1
        for ch in plan.chunks:
            if ch.num_tokens != 1 or not ch.needs_logits:
                return 1
            k = min(k, ch.request.params.max_tokens - len(ch.request.output_ids))
        if k <= 1:
            return 1
        k = 1 << (k.bit_length() - 1)  # a power of two: a runner that records a graph for each count records few
        try:
            for ch in plan.chunks:
                self.manager.reserve_ahead(ch.request.request_id, k - 1)
        except NoFreePagesError:
            return 1  # what was reserved so far stays with its requests and is used later
        return k

    def _serve_running(self, plan: SchedulerOutput, budget: int) -> int:
        """Give each running request its next token or portion; returns the budget left."""
        # Victims are taken from the end of this order, so its front always progresses.
        self.running.sort(key=lambda r: (self._class_of(r), r.arrival_seq))
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
        self.ledger.charge(req.tenant, take)

    # ------------------------------------------------------------------ order of service

    def _class_of(self, req: Request) -> int:
        """The request's priority class now (lower first); long waiting lifts any request to
        the first class so that a stream of urgent requests cannot starve it."""
        waited = self._step - req.arrival_step
        return int(Priority.INTERACTIVE) if waited >= self.config.aging_steps else int(req.priority)

    def _admission_key(self, req: Request) -> tuple[int, bool, float, int]:
        """Order of admission: class, then requests that lost their cache to a preemption (they
        were running once) before new ones, then the tenant owed most, then arrival."""
        return (self._class_of(req), req.num_preemptions == 0, self.ledger.owed(req.tenant), req.arrival_seq)

    # ------------------------------------------------------------------ memory pressure

    def _newest_outside(self, exclude: set[str]) -> Optional[Request]:
        """The running request admitted last among those not in ``exclude``."""
        return next((r for r in reversed(self.running) if r.request_id not in exclude), None)

    def _preempt(self, req: Request) -> None:
        self._release(req, RequestStatus.WAITING)

    def _reserve(self, req: Request) -> Optional[list[CopyOp]]:
        """Cache slots for the tokens of ``req`` that the manager has not been told of yet (the
        token sampled last step). The page copies this asks for, or None if no page is free."""
        known, total = self.manager.num_tokens(req.request_id), req.num_tokens
        if known >= total:
            return []
        try:
            return self.manager.append_slots(req.request_id, req.token_slice(known, total))
        except NoFreePagesError:
            return None
