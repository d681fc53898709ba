"""The scheduler's decisions with a fake model: budget, portions, admission, preemption, fairness.

Vectors from the reference's tests/unit/engine/test_continuous_batching.py, test_preemption.py and
test_scheduler_properties.py.
"""

from __future__ import annotations

import random

import pytest

from dli_amd.cache import CacheManager
from dli_amd.engine import FinishReason, LLMEngine, Priority, SchedulerConfig
from dli_amd.sampling import SamplingParams
from fake_runner import FakeRunner, alone, passthrough_sampler


def make(num_pages=256, page_size=4, max_seqs=8, budget=32, eos=(), **sched):
    m = CacheManager(num_pages=num_pages, page_size=page_size, max_seqs=max(max_seqs, 8), watermark=0.0)
    runner = FakeRunner(m)
    eng = LLMEngine(runner, m, SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=budget, **sched),
                    eos_token_ids=eos, sampler=passthrough_sampler)
    return eng, runner, m


def run(eng, limit=10000):
    for _ in range(limit):
        if not eng.has_unfinished():
            return
        eng.step()
    raise AssertionError("the engine did not finish (livelock?)")


def test_concurrent_requests_equal_each_alone_and_nothing_leaks():
    eng, _, m = make()
    rng = random.Random(1)
    prompts = [[rng.randrange(50) for _ in range(rng.randrange(1, 40))] for _ in range(20)]
    reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=rng.randrange(1, 25))) for i, p in enumerate(prompts)]
    run(eng)
    for r, p in zip(reqs, prompts):
        assert r.output_ids == alone(p, r.params.max_tokens), r.request_id
        assert r.finish_reason is FinishReason.LENGTH
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == m.stats().num_pages and m.slots.num_free == m.slots.num_slots


def test_budget_and_cap_hold_every_step():
    eng, runner, _ = make(max_seqs=3, budget=10)
    for i in range(10):
        eng.add_request(f"r{i}", list(range(i, i + 17)), SamplingParams(max_tokens=5))
    run(eng)
    for sched in runner.calls:
        assert sched.num_batched_tokens <= 10 and len(sched.chunks) <= 3
        assert len({c.request.request_id for c in sched.chunks}) == len(sched.chunks)
    assert all(s.num_batched_tokens == s.num_prefill_tokens + s.num_decode_tokens for s in eng.stats.steps)


def test_long_prompt_is_cut_into_portions_while_decoding_goes_on():
    eng, runner, _ = make(budget=8)
    short = eng.add_request("short", [1, 2, 3], SamplingParams(max_tokens=20))
    eng.step()
    long = eng.add_request("long", list(range(40)), SamplingParams(max_tokens=2))
    for _ in range(5):
        eng.step()
    assert len(short.output_ids) == 6  # one token every step, never stalled
    portions = [c for s in runner.calls for c in s.chunks if c.request is long]
    assert portions and all(c.num_tokens <= 7 for c in portions) and not long.output_ids
    assert all(not c.needs_logits for c in portions)
    run(eng)
    assert long.output_ids == alone(list(range(40)), 2)


def test_a_step_lists_decoding_requests_first_and_the_longest_of_them_first():
    """The plan's order is the order of the step's rows: single tokens before portions, the rows with
    the most keys first (the decode attention's workgroups start in row order)."""
    eng, runner, _ = make(budget=64)
    lens = [5, 23, 11, 17]
    for i, n in enumerate(lens):
        eng.add_request(f"r{i}", list(range(n)), SamplingParams(max_tokens=6))
    eng.step()                       # all four prompts whole
    eng.add_request("late", list(range(100, 130)), SamplingParams(max_tokens=2))
    eng.step()
    chunks = runner.calls[-1].chunks
    assert [c.request.request_id for c in chunks] == ["r1", "r3", "r2", "r0", "late"]
    assert [c.num_tokens for c in chunks] == [1, 1, 1, 1, 30]
    starts = [c.start for c in chunks[:4]]
    assert starts == sorted(starts, reverse=True) == [23, 17, 11, 5]
    run(eng)


def test_content_reuse_starts_the_portion_after_the_cached_pages():
    eng, runner, _ = make(budget=64)
    p = list(range(30))
    eng.add_request("a", p, SamplingParams(max_tokens=1))
    run(eng)
    b = eng.add_request("b", p + [7], SamplingParams(max_tokens=3))
    run(eng)
    first = next(c for s in runner.calls for c in s.chunks if c.request is b)
    assert first.start == 28  # seven full pages of four reused
    assert b.output_ids == alone(p + [7], 3)


def test_stop_reasons():
    eng, _, _ = make(eos=(alone([5, 6], 3)[1],))
    r_eos = eng.add_request("eos", [5, 6], SamplingParams(max_tokens=10))
    r_stop = eng.add_request("stop", [9], SamplingParams(max_tokens=10, stop_token_ids=(alone([9], 4)[2],)))
    r_ign = eng.add_request("ign", [5, 6], SamplingParams(max_tokens=4, ignore_eos=True))
    run(eng)
    assert (r_eos.finish_reason, len(r_eos.output_ids)) == (FinishReason.STOP, 2)
    assert (r_stop.finish_reason, len(r_stop.output_ids)) == (FinishReason.STOP, 3)
    assert (r_ign.finish_reason, len(r_ign.output_ids)) == (FinishReason.LENGTH, 4)


def test_request_that_can_never_fit_is_rejected():
    eng, _, _ = make(num_pages=4, page_size=4)
    r = eng.add_request("big", list(range(10)), SamplingParams(max_tokens=10))
    assert r.finish_reason is FinishReason.CAPACITY and r.is_finished and not eng.has_unfinished()


def test_abort_frees_everything_and_is_idempotent():
    eng, _, m = make(max_seqs=1)
    running = eng.add_request("run", list(range(9)), SamplingParams(max_tokens=50))
    waiting = eng.add_request("wait", [1, 2], SamplingParams(max_tokens=5))
    eng.step()
    eng.step()
    assert eng.abort("run") and eng.abort("wait") and not eng.abort("run")
    assert running.finish_reason is FinishReason.ABORTED and waiting.finish_reason is FinishReason.ABORTED
    assert not eng.has_unfinished()
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == m.stats().num_pages


def test_duplicate_ids_and_empty_prompts():
    eng, _, _ = make()
    eng.add_request("x", [1])
    with pytest.raises(ValueError, match="duplicate"):
        eng.add_request("x", [2])
    with pytest.raises(ValueError, match="non-empty"):
        eng.add_request("y", [])


# ------------------------------------------------------------------ when pages run out

@pytest.mark.parametrize("pages", [12, 20, 40])
def test_outputs_do_not_change_under_preemption(pages):
    eng, runner, m = make(num_pages=pages, budget=16)
    rng = random.Random(pages)
    prompts = [[rng.randrange(50) for _ in range(rng.randrange(3, 14))] for _ in range(8)]
    reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=20)) for i, p in enumerate(prompts)]
    run(eng)
    assert sum(len(s.preempted) for s in runner.calls) > 0 or pages == 40
    for r, p in zip(reqs, prompts):
        assert r.output_ids == alone(p, 20)
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == pages


def test_no_admission_in_a_step_that_preempted_and_oldest_is_never_preempted():
    eng, runner, _ = make(num_pages=12, budget=64)
    reqs = [eng.add_request(f"r{i}", [i, i + 1, i + 2, i + 3, i + 4], SamplingParams(max_tokens=30)) for i in range(5)]
    run(eng)
    assert sum(len(s.preempted) for s in runner.calls) > 0
    for sched in runner.calls:
        if sched.preempted:
            starts_fresh = [c for c in sched.chunks if c.start == 0 and c.request.num_preemptions == 0
                            and c.num_tokens == len(c.request.prompt_ids)]
            assert all(c.request in sched.preempted or c.request.output_ids for c in starts_fresh) or not starts_fresh
    assert reqs[0].num_preemptions == 0
    for i, r in enumerate(reqs):
        assert r.output_ids == alone(r.prompt_ids, 30)


def test_resumed_request_reuses_what_the_index_still_holds():
    eng, runner, m = make(num_pages=14, budget=64)
    a = eng.add_request("a", list(range(20)), SamplingParams(max_tokens=24))
    b = eng.add_request("b", list(range(100, 120)), SamplingParams(max_tokens=24))
    run(eng)
    assert b.num_preemptions > 0
    resumed = [c for s in runner.calls for c in s.chunks if c.request is b and c.start > 0 and c.num_tokens > 1]
    assert resumed and all(c.start % 4 == 0 for c in resumed)
    assert a.output_ids == alone(list(range(20)), 24) and b.output_ids == alone(list(range(100, 120)), 24)


# ------------------------------------------------------------------ fairness

def test_priority_aging_and_tenant_shares():
    eng, runner, _ = make(max_seqs=1, budget=64)
    first = eng.add_request("first", [1], SamplingParams(max_tokens=2))
    batch = eng.add_request("batch", [2], SamplingParams(max_tokens=1), priority=Priority.BATCH)
    inter = eng.add_request("inter", [3], SamplingParams(max_tokens=1))
    run(eng)
    order = [c.request.request_id for s in runner.calls for c in s.chunks if c.start == 0]
    assert order == ["first", "inter", "batch"]
    # after aging_steps a BATCH request counts as INTERACTIVE and its earlier arrival wins
    eng2, runner2, _ = make(max_seqs=1, budget=64, aging_steps=3)
    eng2.add_request("hog", [1], SamplingParams(max_tokens=6))
    eng2.add_request("old-batch", [2], SamplingParams(max_tokens=1), priority=Priority.BATCH)
    for _ in range(4):
        eng2.step()
    eng2.add_request("new-inter", [3], SamplingParams(max_tokens=1))
    run(eng2)
    order2 = [c.request.request_id for s in runner2.calls for c in s.chunks if c.start == 0]
    assert order2.index("old-batch") < order2.index("new-inter")
    # weighted tenants: tenant "big" (weight 3) gets about three admissions for each of "small"
    eng3, runner3, _ = make(max_seqs=1, budget=64, tenant_weights={"big": 3.0, "small": 1.0})
    for i in range(12):
        eng3.add_request(f"b{i}", [1, 2, 3, 4], SamplingParams(max_tokens=1), tenant="big")
        eng3.add_request(f"s{i}", [1, 2, 3, 4], SamplingParams(max_tokens=1), tenant="small")
    for _ in range(12):
        eng3.step()
    served = [c.request.tenant for s in runner3.calls for c in s.chunks]
    assert 8 <= served.count("big") <= 10 and 2 <= served.count("small") <= 4


def test_tenant_ledger_banks_no_credit_and_preempted_requests_come_back_first():
    from dli_amd.engine.scheduler import TenantLedger

    led = TenantLedger({"heavy": 4.0})
    led.enter("a", [])
    led.charge("a", 100)
    led.enter("heavy", ["a"])                 # arrives late: starts level with those present
    assert led.owed("heavy") == led.owed("a") == 100.0
    led.charge("heavy", 100)
    assert led.owed("heavy") == 125.0         # a quarter of the charge for the same tokens
    led.enter("a", ["heavy", "a"])            # present all along: keeps its own figure
    assert led.owed("a") == 100.0
    led.enter("idle", [])                     # nobody present: nothing to be lifted to
    assert led.owed("idle") == 0.0
    # a request that lost its cache is admitted before a new one of the same class
    eng, runner, _ = make(num_pages=6, page_size=4, max_seqs=4, budget=64)
    old = eng.add_request("old", list(range(9)), SamplingParams(max_tokens=12))
    young = eng.add_request("young", list(range(20, 29)), SamplingParams(max_tokens=12))
    while not young.num_preemptions:
        eng.step()
    late = eng.add_request("late", [5], SamplingParams(max_tokens=1))
    run(eng)
    firsts = [c.request.request_id for s in runner.calls for c in s.chunks if c.start == 0]
    assert firsts.index("late") > len(firsts) - 1 - firsts[::-1].index("young")
    assert old.num_preemptions == 0 and young.output_ids == alone(list(range(20, 29)), 12)


# ------------------------------------------------------------------ random scenarios

@pytest.mark.parametrize("seed", range(12))
def test_random_scenarios_keep_invariants_and_outputs(seed):
    rng = random.Random(seed)
    pages, ps = rng.randrange(6, 40), rng.choice([1, 2, 4, 8])
    budget, seqs = rng.choice([1, 2, 3, 8, 32, 128]), rng.randrange(1, 7)
    eng, runner, m = make(num_pages=pages, page_size=ps, max_seqs=seqs, budget=budget)
    expected = {}
    n = 0
    steps = 0
    while steps < 20000:
        if n < 25 and rng.random() < 0.3:
            prompt = [rng.randrange(4) for _ in range(rng.randrange(1, 20))]
            mt = rng.randrange(1, 12)
            r = eng.add_request(f"q{n}", prompt, SamplingParams(max_tokens=mt))
            if r.finish_reason is FinishReason.CAPACITY:
                assert -(-(len(prompt) + mt) // ps) > pages
            else:
                expected[r] = alone(prompt, mt)
            n += 1
        if rng.random() < 0.03 and expected:
            victim = rng.choice(list(expected))
            if not victim.is_finished:
                eng.abort(victim.request_id)
                del expected[victim]
        if not eng.has_unfinished():
            if n >= 25:
                break
            continue
        before = len(runner.calls)
        eng.step()
        steps += 1
        m.check_invariants()
        if len(runner.calls) > before:
            sched = runner.calls[-1]
            assert sched.num_batched_tokens <= budget and len(sched.chunks) <= seqs
            assert len({c.request.request_id for c in sched.chunks}) == len(sched.chunks)
    assert steps < 20000, "liveness"
    for r, out in expected.items():
        assert r.output_ids == out
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == pages


def test_scheduler_config_is_validated():
    with pytest.raises(ValueError):
        SchedulerConfig(max_num_seqs=0)
    with pytest.raises(ValueError):
        SchedulerConfig(tenant_weights={"a": 0.0})
    m = CacheManager(num_pages=4, page_size=4, max_seqs=2)
    with pytest.raises(ValueError, match="state slots"):
        LLMEngine(FakeRunner(m), m, SchedulerConfig(max_num_seqs=3), sampler=passthrough_sampler)


# ------------------------------------------------------------------ several tokens per step

def make_multi(decode_steps, num_pages=256, page_size=4, max_seqs=8, budget=32, eos=()):
    """An engine whose runner decodes and samples by itself (the fake's hash of the history)."""
    m = CacheManager(num_pages=num_pages, page_size=page_size, max_seqs=max(max_seqs, 8), watermark=0.0)
    runner = FakeRunner(m)
    eng = LLMEngine(runner, m, SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=budget,
                                               decode_steps=decode_steps), eos_token_ids=eos)
    return eng, runner, m


@pytest.mark.parametrize("k", [2, 3, 8])
def test_several_tokens_per_step_give_the_same_outputs(k):
    eng, runner, m = make_multi(k)
    rng = random.Random(k)
    prompts = [[rng.randrange(50) for _ in range(rng.randrange(1, 40))] for _ in range(6)]
    limits = [1, 2, 5, 16, 17, 23]
    reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=mt)) for i, (p, mt) in enumerate(zip(prompts, limits))]
    run(eng)
    for r, p in zip(reqs, prompts):
        assert r.output_ids == alone(p, r.params.max_tokens), r.request_id
        assert r.finish_reason is FinishReason.LENGTH
    assert any(s.decode_steps > 1 for s in runner.calls), "no step took several tokens"
    for s in runner.calls:  # never past a request's limit, never while somebody waits or a prompt runs
        if s.decode_steps > 1:
            assert all(c.num_tokens == 1 and c.needs_logits for c in s.chunks)
            assert s.decode_steps & (s.decode_steps - 1) == 0   # powers of two only
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == m.stats().num_pages and m.slots.num_free == m.slots.num_slots


def test_stop_token_inside_a_run_of_tokens_ends_the_request_there():
    prompt = [3, 1, 4, 1, 5]
    full = alone(prompt, 30)
    stop = full[6]
    cut = full.index(stop) + 1
    eng, _, m = make_multi(4)
    r = eng.add_request("a", prompt, SamplingParams(max_tokens=30, stop_token_ids=(stop,)))
    outs = []
    while eng.has_unfinished():
        outs.extend(eng.step())
    assert r.output_ids == full[:cut] and r.finish_reason is FinishReason.STOP
    assert [t for o in outs for t in o.new_token_ids] == full[:cut]
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == m.stats().num_pages


def test_one_token_per_step_while_somebody_waits_or_pages_are_short():
    eng, runner, m = make_multi(4, max_seqs=1)
    eng.add_request("a", [1, 2, 3], SamplingParams(max_tokens=6))
    eng.add_request("b", [4, 5], SamplingParams(max_tokens=6))  # waits: the cap is one request
    while not eng.scheduler.running or eng.scheduler.waiting:
        eng.step()
        if eng.scheduler.waiting:
            assert runner.calls[-1].decode_steps == 1
    run(eng)
    # pages: prompt of 6 and 9 tokens to come need 4 pages of 4; with exactly 4 there is no room to
    # reserve ahead at first, and the outputs stay right
    eng, runner, m = make_multi(8, num_pages=4, page_size=4)
    r = eng.add_request("c", [1, 2, 3, 4, 5, 6], SamplingParams(max_tokens=9))
    run(eng)
    assert r.output_ids == alone([1, 2, 3, 4, 5, 6], 9)
    m.check_invariants()


@pytest.mark.parametrize("seed", range(8))
def test_random_scenarios_with_several_tokens_per_step(seed):
    rng = random.Random(100 + seed)
    pages, ps = rng.randrange(6, 40), rng.choice([1, 2, 4, 8])
    budget, seqs = rng.choice([1, 2, 3, 8, 32, 128]), rng.randrange(1, 7)
    eng, runner, m = make_multi(rng.choice([2, 4, 8]), num_pages=pages, page_size=ps, max_seqs=seqs, budget=budget)
    expected, n, steps = {}, 0, 0
    while steps < 20000:
        if n < 25 and rng.random() < 0.3:
            prompt = [rng.randrange(4) for _ in range(rng.randrange(1, 20))]
            mt = rng.randrange(1, 12)
            r = eng.add_request(f"q{n}", prompt, SamplingParams(max_tokens=mt))
            if r.finish_reason is not FinishReason.CAPACITY:
                expected[r] = alone(prompt, mt)
            n += 1
        if rng.random() < 0.03 and expected:
            victim = rng.choice(list(expected))
            if not victim.is_finished:
                eng.abort(victim.request_id)
                del expected[victim]
        if not eng.has_unfinished():
            if n >= 25:
                break
            continue
        eng.step()
        steps += 1
        m.check_invariants()
    assert steps < 20000, "liveness"
    for r, out in expected.items():
        assert r.output_ids == out
    m.reset_prefix_cache()
    m.check_invariants()
    assert m.stats().free_pages == pages
