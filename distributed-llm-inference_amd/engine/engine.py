"""The engine's step loop and Python entry point.

One ``step()``: schedule, run the scheduled tokens as one batch through the step function, sample
a token for every request whose chunk reached its last known token, append it, finish what is done
(reference: src/dli/engine/engine.py:183-246). Each phase is timed (``StepStats``).
"""

from __future__ import annotations

import dataclasses

import itertools
import random
import time
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Callable, Collection, Iterable, Optional, Protocol, Sequence

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams
from .request import FinishReason, Priority, Request
from .scheduler import Scheduler, SchedulerConfig, SchedulerOutput


class Runner(Protocol):
    """Runs a scheduler decision. Afterwards every scheduled chunk's keys are written and marked
    computed in the cache manager. Returns logits, one row per chunk with ``needs_logits``, in
    schedule order (reference: src/dli/engine/runner.py:18-25)."""

    def execute(self, sched: SchedulerOutput) -> Any: ...


TokenSampler = Callable[[Any, Sequence[SamplingParams], Sequence[Optional[int]], Sequence[int]], list[int]]


class ModelRunner:
    """The runner for a real model: turns chunks into step entries for the step function."""

    def __init__(self, core: Any) -> None:
        self.core = core

    def execute(self, sched: SchedulerOutput) -> Any:
        return self.core.step.run(self._entries(sched), sched.copy_ops)

    def execute_and_sample(self, sched: SchedulerOutput) -> list[int]:
        """Run the step and choose a token for every chunk that needs one, on the GPU (inside
        the replayed graph for decode steps); token ids in schedule order."""
        from ..sampling.sampler import sampling_tuple

        sampling = [sampling_tuple(c.request.params, c.request.seed, len(c.request.output_ids))
                    for c in sched.chunks if c.needs_logits]
        return self.core.step.run(self._entries(sched), sched.copy_ops, sampling=sampling, steps=sched.decode_steps)

    @property
    def max_decode_steps(self) -> int:
        """Tokens per request that one step can decode on the device (1 without decode graphs)."""
        return self.core.step.max_decode_steps

    def _entries(self, sched: SchedulerOutput) -> list:
        from .batch import StepEntry

        entries = []
        for ch in sched.chunks:
            req = ch.request
            n_prompt = len(req.prompt_ids)
            lo, hi = ch.start, ch.start + ch.num_tokens
            if hi <= n_prompt:
                tokens = req.prompt_ids[lo:hi]
            else:
                tokens = (req.prompt_ids[lo:] if lo < n_prompt else []) + req.output_ids[max(0, lo - n_prompt):hi - n_prompt]
            entries.append(StepEntry(req.request_id, tokens, ch.start,
                                     (ch.num_tokens - 1,) if ch.needs_logits else ()))
        return entries


@dataclass(frozen=True)
class RequestOutput:
    request_id: str
    new_token_ids: list[int]
    finished: bool
    finish_reason: Optional[FinishReason]


@dataclass(frozen=True)
class StepStats:
    """Shape and timing (seconds) of one step (the fields of src/dli/engine/engine.py:39-54, and
    ``decode_steps``: how many tokens each request of the step decoded, 1 unless the step ran
    several on the device)."""

    num_seqs: int
    num_batched_tokens: int
    num_prefill_tokens: int
    num_decode_tokens: int
    num_preempted: int
    schedule_s: float
    forward_s: float
    postprocess_s: float
    decode_steps: int = 1

    @property
    def total_s(self) -> float:
        return self.schedule_s + self.forward_s + self.postprocess_s

    @classmethod
    def of(cls, plan: SchedulerOutput, marks: Sequence[float]) -> "StepStats":
        """The record of a step that ran ``plan``; ``marks``: the clock before scheduling, after
        it, after the forward pass, and at the end. A chunk counts as decoding if it is the one
        token whose successor is sampled; everything else is prompt work."""
        decoding = sum(1 for c in plan.chunks if c.num_tokens == 1 and c.needs_logits)
        tokens = plan.num_batched_tokens
        spans = [later - earlier for earlier, later in zip(marks, marks[1:])]
        return cls(num_seqs=len(plan.chunks), num_batched_tokens=tokens, num_prefill_tokens=tokens - decoding,
                   num_decode_tokens=decoding, num_preempted=len(plan.preempted), schedule_s=spans[0],
                   forward_s=spans[1], postprocess_s=spans[2], decode_steps=plan.decode_steps)


@dataclass
class EngineStats:
    steps: list[StepStats] = field(default_factory=list)


class LLMEngine:
    """Continuous-batching engine over the paged cache; single-threaded.

    Build with :meth:`for_model`. Tests may inject any :class:`Runner` and token sampler together
    with the cache manager they work on.
    """

    def __init__(self, runner: Runner, manager: CacheManager, config: Optional[SchedulerConfig] = None, *,
                 eos_token_ids: Collection[int] = (), seed: int = 0,
                 sampler: Optional[TokenSampler] = None) -> None:
        self.runner = runner
        self.manager = manager
        config = config or SchedulerConfig()
        # several tokens per step need a runner that decodes and samples them on the device
        can = getattr(runner, "max_decode_steps", 1) if sampler is None else 1
        if config.decode_steps > can:
            config = dataclasses.replace(config, decode_steps=max(1, can))
        self.scheduler = Scheduler(config, manager)
        self.eos = frozenset(eos_token_ids)
        self._rng = random.Random(seed)
        self._arrivals = itertools.count()
        self._step_no = 0
        self._sample_is_default = sampler is None
        if sampler is None:
            from ..sampling.sampler import sample as sampler  # the GPU sampler
        self._sample = sampler
        self.stats = EngineStats()

    @classmethod
    def for_model(cls, model: Any, *, num_blocks: Optional[int] = None, kv_cache_gb: Optional[float] = None,
                  block_size: int = 16, config: Optional[SchedulerConfig] = None,
                  eviction_policy: str = "lru", enable_prefix_caching: bool = True,
                  eos_token_ids: Collection[int] = (), seed: int = 0, dtype: str = "bfloat16",
                  device: str = "cuda", cuda_graphs: bool = True,
                  max_model_len: Optional[int] = None, decode_weight_copy: bool = True) -> "LLMEngine":
        """Engine for a loaded model or a model folder.

        ``num_blocks`` pages of ``block_size`` tokens, or as many as ``kv_cache_gb`` GiB hold
        (default 1 GiB), as the reference's server takes them (src/dli/server/__main__.py:150-156).
        ``cuda_graphs``: replay decode-only steps through HIP graphs (the reference's option of
        this name replays CUDA graphs; here it is on by default and falls back to eager steps for
        shapes whose decode path is not captured). ``decode_weight_copy`` (when ``model`` is a
        folder): see :func:`load_model`.
        """
        from ..weights.loader import load_model
        from .core import build_core, pages_for_budget

        if num_blocks is not None and kv_cache_gb is not None:
            raise ValueError("give num_blocks or kv_cache_gb, not both")
        if isinstance(model, (str, Path)):
            model = load_model(model, dtype=dtype, device=device, decode_weight_copy=decode_weight_copy)
        if num_blocks is None:
            gib = 1.0 if kv_cache_gb is None else kv_cache_gb
            num_blocks = pages_for_budget(model, block_size, int(gib * 2 ** 30))
        config = config or SchedulerConfig()
        core = build_core(model, num_pages=num_blocks, page_size=block_size, max_seqs=config.max_num_seqs,
                          enable_prefix_caching=enable_prefix_caching, eviction_policy=eviction_policy)
        if cuda_graphs:
            longest = num_blocks * block_size
            core.step.enable_decode_graphs(config.max_num_seqs, min(max_model_len or longest, longest))
        engine = cls(ModelRunner(core), core.manager, config, eos_token_ids=eos_token_ids, seed=seed)
        engine.core = core
        return engine

    # ------------------------------------------------------------------ API

    def warm_up(self, batches: Sequence[int], max_len: int) -> int:
        """Capture the decode graphs that steps of ``batches`` running requests with contexts up to
        ``max_len`` tokens will replay (for every number of tokens per step that the scheduler may
        choose), before the first request arrives. Returns how many graphs were captured; 0 for an
        engine without graph replay."""
        graphs = getattr(getattr(getattr(self, "core", None), "step", None), "graphs", None)
        if graphs is None:
            return 0
        k = self.scheduler.config.decode_steps
        return graphs.warm_up(batches, max_len, sampled=True, steps=tuple(range(1, k + 1)))

    def add_request(self, request_id: str, prompt_ids: Sequence[int], params: Optional[SamplingParams] = None, *,
                    priority: Priority = Priority.INTERACTIVE, tenant: str = "default") -> Request:
        """Queue a request. One that can never fit finishes at once with CAPACITY."""
        if not prompt_ids:
            raise ValueError("prompt must be non-empty")
        params = params or SamplingParams()
        seed = params.seed if params.seed is not None else self._rng.getrandbits(63)
        req = Request(request_id=request_id, prompt_ids=[int(t) for t in prompt_ids], params=params,
                      arrival_seq=next(self._arrivals), priority=priority, tenant=tenant,
                      seed=None if params.greedy else seed, arrival_step=self._step_no)
        self.scheduler.add(req)
        return req

    def abort(self, request_id: str) -> bool:
        return self.scheduler.abort(request_id) is not None

    def has_unfinished(self) -> bool:
        return self.scheduler.has_unfinished

    def step(self) -> list[RequestOutput]:
        """Schedule, run, sample, append; one :class:`StepStats` per call, also for a step in
        which nothing could be scheduled."""
        marks = [time.perf_counter()]
        plan = self.scheduler.schedule()
        marks.append(time.perf_counter())
        outputs: list[RequestOutput] = []
        if plan.chunks:
            rounds = self._run(plan, marks)
            wanted = [c for c in plan.chunks if c.needs_logits]
            if len(rounds) != plan.decode_steps or any(len(r) != len(wanted) for r in rounds):
                raise RuntimeError("the sampler returned a wrong number of tokens")
            outputs = [self._append_tokens(c.request, [int(r[i]) for r in rounds]) for i, c in enumerate(wanted)]
        else:
            marks.append(marks[-1])
        marks.append(time.perf_counter())
        self.stats.steps.append(StepStats.of(plan, marks))
        self._step_no += 1
        return outputs

    def _run(self, plan: SchedulerOutput, marks: list[float]) -> list[Sequence[int]]:
        """Run the plan's chunks and choose the tokens: one sequence of token ids (in the order
        of the chunks that need logits) per decoded position. Notes the time after the forward
        pass in ``marks`` and moves every request's count of computed tokens on."""
        fused = getattr(self.runner, "execute_and_sample", None) if self._sample_is_default else None
        result = fused(plan) if fused is not None else self.runner.execute(plan)
        marks.append(time.perf_counter())
        for c in plan.chunks:
            c.request.num_computed_tokens += c.num_tokens + plan.decode_steps - 1
        if fused is None:
            wanted = [c.request for c in plan.chunks if c.needs_logits]
            result = self._sample(result, [r.params for r in wanted], [r.seed for r in wanted],
                                  [len(r.output_ids) for r in wanted])
        return result if plan.decode_steps > 1 else [result]

    def generate(self, prompts: Iterable[Sequence[int]],
                 params: SamplingParams | Sequence[SamplingParams] | None = None) -> list[list[int]]:
        """Run prompts (token ids) to completion; generated ids in input order."""
        prompts = list(prompts)
        if params is None or isinstance(params, SamplingParams):
            per = [params or SamplingParams()] * len(prompts)
        else:
            per = list(params)
            if len(per) != len(prompts):
                raise ValueError("one SamplingParams per prompt, or one for all")
        tag = next(self._arrivals)
        reqs = [self.add_request(f"gen-{tag}-{i}", p, per[i]) for i, p in enumerate(prompts)]
        while self.has_unfinished():
            self.step()
        return [r.output_ids for r in reqs]

    # ------------------------------------------------------------------ internals

    def _append_tokens(self, req: Request, toks: Sequence[int]) -> RequestOutput:
        """Take the tokens that a step decoded for the request, in order, up to the one that ends
        it; what was decoded beyond that one is dropped."""
        reason: Optional[FinishReason] = None
        taken: list[int] = []
        for tok in toks:
            req.output_ids.append(tok)
            taken.append(tok)
            if tok in req.params.stop_token_ids or (not req.params.ignore_eos and tok in self.eos):
                reason = FinishReason.STOP
            elif len(req.output_ids) >= req.params.max_tokens:
                reason = FinishReason.LENGTH
            if reason is not None:
                self.scheduler.finish(req, reason)
                break
        return RequestOutput(req.request_id, taken, reason is not None, reason)
