"""The engine's entry points on the GPU: greedy generation against the plain implementation,
regimes of the scheduler on real kernels, graph replay against eager steps, sampling."""

from __future__ import annotations

import random

import pytest
import torch

import plain_llama as P
from tiny_configs import model_folder

pytestmark = pytest.mark.gpu


def prompts(name, lengths, seed):
    cfg, _ = P.load_folder(model_folder(name))
    rng = random.Random(seed)
    return [[rng.randrange(cfg["vocab_size"]) for _ in range(n)] for n in lengths]


def plain_greedy(name, prompt, n):
    cfg, w = P.load_folder(model_folder(name))
    return P.greedy_generate(w, cfg, prompt, n)


def assert_same_or_near_tie(name, prompt, got, want, margin):
    """Greedy tokens of the engine against the plain implementation, the whole run: ``got`` equals
    ``want`` (the plain implementation's own greedy run), or else every token of ``got`` is checked
    against the plain logits of the engine's own tokens before it (teacher forcing: one plain
    evaluation of ``prompt + got``): the token must be the plain model's best there, or lie within
    ``margin`` of it, where rounding decides. A run that parts from the plain one at a near-tie
    is thus still checked to its end."""
    assert len(got) == len(want), (len(got), len(want))
    if list(got) == list(want):
        return
    cfg, w = P.load_folder(model_folder(name))
    logits = P.forward_logits(w, cfg, list(prompt) + list(got[:-1]))
    for j, g in enumerate(got):
        row = logits[len(prompt) - 1 + j]
        gap = (row.max() - row[g]).item()
        assert gap < margin, f"token {j} is {g}: the plain logits prefer {int(row.argmax())} by {gap}"


def assert_draws_follow_the_plain_distribution(name, prompt, got, params, seed, tol):
    """Seeded tokens of the engine against the plain implementation, the whole run: at every
    position the request's uniform draw (host Philox, keyed by seed and position) must lie in the
    token's cell of the plain cumulative distribution over the engine's own tokens before it, or
    within ``tol`` of that cell, where rounding decides."""
    from test_sampling_gpu import philox_uniform

    cfg, w = P.load_folder(model_folder(name))
    logits = P.forward_logits(w, cfg, list(prompt) + list(got[:-1]))
    for j, tok in enumerate(got):
        probs = P.sampling_probabilities(logits[len(prompt) - 1 + j], params.temperature, params.top_k, params.top_p)
        hi = float(torch.cumsum(probs, 0)[tok])
        lo, u = hi - float(probs[tok]), philox_uniform(seed, j)
        assert lo - tol <= u <= hi + tol, f"draw {j}: token {tok} has the cell [{lo}, {hi}], the draw is {u}"


@pytest.mark.parametrize("name,dtype,block", [("A", "float32", 16), ("B", "float32", 8), ("A", "bfloat16", 16),
                                              ("B", "bfloat16", 16), ("C", "bfloat16", 32), ("D", "bfloat16", 16)])
def test_greedy_generation_through_the_entry_point(name, dtype, block):
    from dli_amd.engine.generate import greedy_generate

    for prompt in prompts(name, [7, 33], seed=21):
        want = plain_greedy(name, prompt, 24)
        got = greedy_generate(str(model_folder(name)), prompt, 24, dtype=dtype, block_size=block)
        assert len(got) == 24
        assert_same_or_near_tie(name, prompt, got, want, 1e-3 if dtype == "float32" else 0.25)


@pytest.mark.parametrize("regime", ["roomy", "small budget", "tight pool"])
def test_engine_equals_single_requests_in_three_regimes(regime):
    """32-bit path: continuous batching must give each request what it gets alone (the reference's
    tests/unit/model/test_engine_tiny.py:26-57)."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    name = "A"
    ps = prompts(name, [7, 16, 33, 50, 5, 21], seed=22)
    kw = {"roomy": dict(num_blocks=256, block_size=16, config=SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=512)),
          "small budget": dict(num_blocks=256, block_size=16, config=SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=16)),
          "tight pool": dict(num_blocks=36, block_size=4, config=SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=64)),
          }[regime]
    eng = LLMEngine.for_model(str(model_folder(name)), dtype="float32", **kw)
    outs = eng.generate(ps, SamplingParams(max_tokens=24))
    if regime == "tight pool":
        assert sum(s.num_preempted for s in eng.stats.steps) > 0
    for p, got in zip(ps, outs):
        assert_same_or_near_tie(name, p, got, plain_greedy(name, p, 24), 1e-3)
    eng.manager.reset_prefix_cache()
    eng.manager.check_invariants()
    assert eng.manager.stats().used_pages == 0


@pytest.mark.parametrize("name,block", [("A", 16), ("C", 32), ("D", 16)])
def test_graph_replay_equals_eager_steps(name, block):
    """Decode steps through HIP graphs against the same steps run eagerly: logits of every step
    must agree, with other work and synchronisations between the replays, batch sizes that
    change (padding rows), and pages that are handed on."""
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    def run(graphs: bool):
        core = build_core(model_folder(name), num_pages=40, page_size=block, max_seqs=8, dtype="bfloat16",
                          enable_prefix_caching=False, watermark=0.0)
        if graphs:
            core.step.enable_decode_graphs(8, 40 * block)
            assert core.step.graphs is not None
        s = TraceSession(core)
        rng = random.Random(4)
        toks = prompts(name, [40, 9, 70, 23, 55], seed=23)
        fed = {}
        outs = []
        live = [0, 1, 2]
        for r in live:
            outs.append(s.step([{"id": r, "tokens": toks[r][:5], "want": [4]}]).float().cpu())
            fed[r] = 5
        pending = [3, 4]
        for it in range(60):
            entries, end = [], []
            for r in list(live):
                if rng.random() < 0.15 and len(live) > 1:
                    continue
                entries.append({"id": r, "tokens": [toks[r][fed[r]]], "want": [0]})
                fed[r] += 1
                if fed[r] == len(toks[r]):
                    end.append(r)
            if entries:
                outs.append(s.step(entries, end).float().cpu())
                torch.cuda.synchronize()
            for r in end:
                live.remove(r)
                if pending:
                    nxt = pending.pop(0)
                    outs.append(s.step([{"id": nxt, "tokens": toks[nxt][:6], "want": [5]}]).float().cpu())
                    fed[nxt] = 6
                    live.append(nxt)
            if not live:
                break
        return outs, core

    eager, _ = run(False)
    graphed, core = run(True)
    assert core.step.graphs.replays > 20 and len(core.step.graphs.captured) >= 2
    assert len(eager) == len(graphed)
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert a.shape == b.shape
        assert torch.equal(a, b), f"step {i}: graph replay differs from the eager step by {(a - b).abs().max()}"


@pytest.mark.parametrize("name,block,k,graph_len", [("A", 16, 4, None), ("C", 32, 3, None), ("B", 16, 8, None),
                                                   ("A", 16, 4, 40), ("D", 16, 8, None)])
def test_several_decode_tokens_per_step_equal_one_per_step(name, block, k, graph_len):
    """Steps that decode `k` tokens of every request on the device (sampled tokens fed back there,
    positions, slots and draw counters advanced by a kernel) against one token per step: greedy
    and seeded sampling give the same tokens; limits that are no multiple of k, a stop token
    inside a run, prompts that end at a page's edge, and pages reserved ahead that are returned.
    `graph_len`: the graphs are sized for shorter requests than some that come, whose tokens then
    run one step at a time."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    ps = prompts(name, [block - 1, block, 5, 2 * block + 3], seed=31)
    limits = [7, 2 * block + 5, 1, 13]

    def run(steps, stop=()):
        eng = LLMEngine.for_model(str(model_folder(name)), dtype="bfloat16", num_blocks=64, block_size=block,
                                  max_model_len=graph_len,
                                  config=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=256, decode_steps=steps))
        params = [SamplingParams(max_tokens=limits[0], stop_token_ids=tuple(stop)),
                  SamplingParams(max_tokens=limits[1], temperature=0.8, top_k=12, seed=5),
                  SamplingParams(max_tokens=limits[2]),
                  SamplingParams(max_tokens=limits[3], temperature=1.1, top_p=0.9, seed=9)]
        reqs = [eng.add_request(f"r{i}", p, q) for i, (p, q) in enumerate(zip(ps, params))]
        many = 0
        while eng.has_unfinished():
            eng.step()
            eng.core.manager.check_invariants()
        many = sum(1 for s in eng.stats.steps if s.num_decode_tokens and s.num_seqs)
        eng.core.manager.reset_prefix_cache()
        st = eng.core.manager.stats()
        assert st.free_pages == st.num_pages
        return [r.output_ids for r in reqs], [r.finish_reason for r in reqs], len(eng.stats.steps)

    one, why1, n1 = run(1)
    some, whyk, nk = run(k)
    assert one == some and why1 == whyk
    assert nk < n1, "no step decoded several tokens"
    stop = one[0][3]  # ends request 0 inside a run of k
    one, why1, _ = run(1, [stop])
    some, whyk, _ = run(k, [stop])
    assert one == some and why1 == whyk and one[0][-1] == stop and len(one[0]) <= 4


def test_shared_prefix_sampling_preemption_config_b():
    """Six prompts that share a 40-token prefix, sampled at temperature 0.8 with per-request seeds
    in a pool so small that requests are preempted: with and without content reuse of cache pages,
    and each request alone, the tokens are the same (32-bit path)."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    name = "B"
    rng = random.Random(31)
    vocab = 384
    prefix = [rng.randrange(vocab) for _ in range(40)]
    ps = [prefix + [rng.randrange(vocab) for _ in range(n)] for n in (5, 22, 90, 37, 61, 12)]
    params = [SamplingParams(max_tokens=32, temperature=0.8, seed=1000 + i) for i in range(len(ps))]

    def run(prompts, pars, **kw):
        eng = LLMEngine.for_model(str(model_folder(name)), dtype="float32", block_size=8, **kw)
        outs = eng.generate(prompts, pars)
        eng.manager.check_invariants()
        return outs, eng

    alone = [run([p], [q], num_blocks=64, config=SchedulerConfig(max_num_seqs=2, max_num_batched_tokens=256))[0][0]
             for p, q in zip(ps, params)]
    tight = dict(num_blocks=44, config=SchedulerConfig(max_num_seqs=6, max_num_batched_tokens=48))
    with_reuse, eng = run(ps, params, enable_prefix_caching=True, **tight)
    assert sum(s.num_preempted for s in eng.stats.steps) > 0
    assert eng.manager.stats().prompt_tokens_hit > 0
    without, _ = run(ps, params, enable_prefix_caching=False, **tight)
    assert with_reuse == alone and without == alone
    assert all(len(o) == 32 for o in alone) and len({tuple(o) for o in alone}) > 1
    # and what they agree on is what the plain implementation's distributions and the requests' own draws give
    for p, q, out in zip(ps, params, alone):
        assert_draws_follow_the_plain_distribution(name, p, out, q, q.seed, 1e-3)


def assert_same_or_near_cell_edge(name, prompt, a, b, params, seed, tol):
    """Two runs of one seeded request: the same tokens, or at the first difference the request's
    uniform draw (host Philox) lies within ``tol`` of the edge between the two tokens' cells of the
    plain cumulative distribution (then rounding decides and the runs part there)."""
    from test_sampling_gpu import philox_uniform

    cfg, w = P.load_folder(model_folder(name))
    for j, (x, y) in enumerate(zip(a, b)):
        if x == y:
            continue
        logits = P.forward_logits(w, cfg, list(prompt) + list(a[:j]))[-1]
        probs = P.sampling_probabilities(logits, params.temperature, params.top_k, params.top_p)
        cdf = torch.cumsum(probs, 0)
        u = philox_uniform(seed, j)
        for tok in (x, y):
            lo, hi = float(cdf[tok] - probs[tok]), float(cdf[tok])
            assert lo - tol <= u <= hi + tol, f"draw {j}: token {tok} has cell [{lo}, {hi}], the draw is {u}"
        return
    assert len(a) == len(b)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seeded_request_is_the_same_alone_and_in_a_busy_batch(dtype):
    """The reference's tests/unit/model/test_engine_tiny.py:89-107, in both precisions. bfloat16
    runs the matrix-core kernels, graph replay and the sampler inside the graph; there the kernels
    chosen depend on the batch, so logits agree to rounding and a draw at the very edge of a
    token's cell may fall to the neighbour."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    name = "A"
    ps = prompts(name, [9, 30, 14, 21, 6], seed=33)
    sp = SamplingParams(max_tokens=20, temperature=0.9, top_k=40, top_p=0.95, seed=7)

    def run(which):
        eng = LLMEngine.for_model(str(model_folder(name)), dtype=dtype, num_blocks=64, block_size=16,
                                  config=SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=64))
        pars = [sp if i == 2 else SamplingParams(max_tokens=25, temperature=1.0, seed=50 + i) for i in which]
        out = eng.generate([ps[i] for i in which], pars)[which.index(2)]
        if dtype == "bfloat16":
            assert eng.core.step.graphs is not None and eng.core.step.graphs.replays > 0
        return out

    alone, busy, pair = run([2]), run([0, 1, 2, 3, 4]), run([2, 4])
    assert_draws_follow_the_plain_distribution(name, ps[2], alone, sp, 7, 1e-3 if dtype == "float32" else 0.05)
    if dtype == "float32":
        assert alone == busy == pair
    else:
        assert len(alone) == 20
        assert_same_or_near_cell_edge(name, ps[2], alone, busy, sp, 7, 0.02)
        assert_same_or_near_cell_edge(name, ps[2], alone, pair, sp, 7, 0.02)


@pytest.mark.parametrize("name", ["A", "D"])
def test_graph_row_of_a_request_that_lost_its_pages_and_came_back(name):
    """The schedule in which a captured graph's block-table row goes stale if it is keyed by the
    request's id: B decodes in row 1 of the two-request graph and gives back its pages; C takes
    them and writes its own keys there; A decodes alone meanwhile (the one-request graph, so the
    other graph's row 1 is not touched); B comes back under its id with other pages and decodes
    beside A in the two-request graph again. Every logit row is the plain implementation's."""
    from test_model_gpu import check, plain_logits
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    page = 16
    a, b, c, d = prompts(name, [120, 100, 80, 96], seed=43)
    core = build_core(model_folder(name), num_pages=15, page_size=page, max_seqs=4, dtype="bfloat16",
                      enable_prefix_caching=False, watermark=0.0)
    core.step.enable_decode_graphs(4, 15 * page)
    s = TraceSession(core)
    ref_a, ref_b = plain_logits(name, a), plain_logits(name, b)
    fed_a, fed_b = 50, 70
    s.step([{"id": "A", "tokens": a[:fed_a], "want": []}])
    s.step([{"id": "B", "tokens": b[:fed_b], "want": []}])

    def decode_both(steps):
        nonlocal fed_a, fed_b
        for _ in range(steps):
            got = s.step([{"id": "A", "tokens": [a[fed_a]], "want": [0]}, {"id": "B", "tokens": [b[fed_b]], "want": [0]}])
            check(got, torch.stack([ref_a[fed_a], ref_b[fed_b]]), "bfloat16", f"{name} A at {fed_a}, B at {fed_b}")
            fed_a, fed_b = fed_a + 1, fed_b + 1

    decode_both(4)
    replays = core.step.graphs.replays
    assert replays == 4
    old_pages = core.manager.block_table("B")
    s.step([{"id": "D", "tokens": d, "want": []}], end=["B"])  # D fills the pool; B gives back its pages
    s.step([{"id": "C", "tokens": c, "want": []}], end=["D"])  # C's keys now lie in the pages that were B's
    assert set(core.manager.block_table("C")) == set(old_pages)
    for _ in range(3):                                        # A alone: the one-request graph
        got = s.step([{"id": "A", "tokens": [a[fed_a]], "want": [0]}])
        check(got, ref_a[fed_a:fed_a + 1], "bfloat16", f"{name} A alone at {fed_a}")
        fed_a += 1
    s.step([{"id": "B", "tokens": b[:fed_b], "want": []}])   # B again, recomputed, in other pages
    assert core.manager.block_table("B")[:4] != old_pages[:4]
    decode_both(6)
    assert core.step.graphs.replays == replays + 3 + 6
    core.manager.check_invariants()


@pytest.mark.parametrize("name", ["A", "D"])
@pytest.mark.parametrize("reuse", [False, True])
def test_graph_replay_under_preemption_bf16(name, reuse):
    """bfloat16 with graph replay in a pool so small that requests lose their pages and recompute:
    a request that comes back under its id holds other pages, and the block-table row that the
    captured graph kept for it must show them (the reference's
    tests/unit/engine/test_preemption.py:32-45 with tests/unit/model/test_cuda_graph_gpu.py:129-150).
    With content reuse on, the pool is small enough for idle cached pages to be reclaimed. Each
    request's tokens are the plain implementation's, up to near-ties."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    ps = prompts(name, [40, 23, 55, 31, 47, 18, 60, 12], seed=37)
    eng = LLMEngine.for_model(str(model_folder(name)), dtype="bfloat16", num_blocks=14, block_size=16,
                              enable_prefix_caching=reuse,
                              config=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64))
    assert eng.core.step.graphs is not None
    reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=44)) for i, p in enumerate(ps)]
    while eng.has_unfinished():
        eng.step()
        eng.manager.check_invariants()
    assert eng.core.step.graphs.replays > 0
    assert sum(s.num_preempted for s in eng.stats.steps) > 0
    assert max(r.num_preemptions for r in reqs) > 0
    if reuse:
        assert eng.manager.stats().evictions > 0
    for p, r in zip(ps, reqs):
        assert len(r.output_ids) == 44
        assert_same_or_near_tie(name, p, r.output_ids, plain_greedy(name, p, 44), margin=0.25)
    eng.manager.reset_prefix_cache()
    assert eng.manager.stats().used_pages == 0


@pytest.mark.parametrize("name", ["A", "D"])
@pytest.mark.parametrize("reuse", [False, True])
def test_eight_tokens_a_step_in_a_pool_that_runs_out_bf16(name, reuse):
    """What ``generate()`` and the command line do by default (bfloat16, decode graphs, up to
    eight tokens of every request per engine step), in a pool so small that requests lose their
    pages and recompute and that reserving pages ahead fails half-way in some steps (what was
    reserved so far then stays with its request and a single token is decoded): the reference's
    tests/unit/engine/test_preemption.py:32-61 with tests/unit/model/test_cuda_graph_gpu.py:129-150,
    on the real block tables, the kernel that moves positions and slots on between the tokens of
    a step, and the graphs' rows. Greedy and seeded requests side by side; every token of every
    request is checked against the plain implementation on the request's own tokens before it."""
    from dli_amd.cache.manager import NoFreePagesError
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    ps = prompts(name, [40, 23, 55, 31, 47, 18, 60, 12, 35, 50], seed=71)
    eng = LLMEngine.for_model(str(model_folder(name)), dtype="bfloat16", num_blocks=16, block_size=16,
                              enable_prefix_caching=reuse,
                              config=SchedulerConfig(max_num_seqs=6, max_num_batched_tokens=64, decode_steps=8))
    graphs = eng.core.step.graphs
    assert graphs is not None and eng.scheduler.config.decode_steps == 8
    refused = []
    reserve = eng.manager.reserve_ahead

    def counting(*a, **k):
        try:
            return reserve(*a, **k)
        except NoFreePagesError:
            refused.append(a)
            raise

    eng.manager.reserve_ahead = counting
    seeded = {1: SamplingParams(max_tokens=44, temperature=0.8, top_k=40, seed=11),
              4: SamplingParams(max_tokens=44, temperature=1.0, seed=12),
              7: SamplingParams(max_tokens=44, temperature=0.9, top_p=0.95, seed=13)}
    reqs = [eng.add_request(f"r{i}", p, seeded.get(i, SamplingParams(max_tokens=44))) for i, p in enumerate(ps)]
    while eng.has_unfinished():
        eng.step()
        eng.manager.check_invariants()
    steps = eng.stats.steps
    assert sum(s.num_preempted for s in steps) > 0 and max(r.num_preemptions for r in reqs) > 0
    assert sum(1 for s in steps if s.decode_steps > 1) >= 3 and max(s.decode_steps for s in steps) == 8
    assert refused, "reserving ahead never failed: the pool was meant to be too small for that"
    assert graphs.replays > 0
    if reuse:
        assert eng.manager.stats().evictions > 0
    for i, (p, r) in enumerate(zip(ps, reqs)):
        assert len(r.output_ids) == 44
        if i in seeded:
            assert_draws_follow_the_plain_distribution(name, p, r.output_ids, seeded[i], seeded[i].seed, 0.05)
        else:
            assert_same_or_near_tie(name, p, r.output_ids, plain_greedy(name, p, 44), margin=0.25)
    eng.manager.reset_prefix_cache()
    assert eng.manager.stats().used_pages == 0


def test_a_graph_of_more_than_64_rows_cuts_the_keys_as_its_mixer_planned(monkeypatch):
    """Decode steps of more than 64 requests are recorded through the loop in C that issues all
    layers' launches. While a graph is recorded the context's host arrays say nothing about the
    steps that it will replay, so the number of runs into which the keys are cut must be the one
    that the mixer planned for the graph's shape (two kv heads: 80 rows leave compute units idle
    unless long requests' keys are cut), not one computed from those arrays; and the logits are
    the plain implementation's."""
    from test_model_gpu import check, plain_logits
    from dli_amd.engine.core import build_core
    from dli_amd.kernels import ops
    from dli_amd.trace import TraceSession

    name, count = "B", 70
    lens = [600 if r % 20 == 0 else 20 + r % 7 for r in range(count)]
    toks = [prompts(name, [n + 3], seed=200 + r)[0] for r, n in enumerate(lens)]
    core = build_core(model_folder(name), num_pages=sum(-(-(n + 3) // 16) for n in lens) + 4, page_size=16,
                      max_seqs=count, dtype="bfloat16", enable_prefix_caching=False, watermark=0.0)
    core.step.enable_decode_graphs(count, 640)
    seen = []
    real = ops.prenorm_blocks

    def recording(x, blocks, n_blocks, step):
        seen.append((step.rows, step.num_decode, step.shapes[0].decode_splits))
        return real(x, blocks, n_blocks, step)

    monkeypatch.setattr(ops, "prenorm_blocks", recording)
    s = TraceSession(core)
    for r in range(count):
        s.step([{"id": r, "tokens": toks[r][:lens[r]], "want": []}])
    del seen[:]
    for i in range(3):
        out = s.step([{"id": r, "tokens": [toks[r][lens[r] + i]], "want": [0]} for r in range(count)])
        if i == 0 or i == 2:
            rows = torch.stack([plain_logits(name, toks[r])[lens[r] + i] for r in range(count)])
            check(out, rows, "bfloat16", f"decode step {i} of {count} requests")
    assert core.step.graphs.replays == 3
    (key,) = core.step.graphs.captured
    planned = set(key[1])
    assert len(planned) == 1 and min(planned) > 1, key
    assert seen and all(rows == 80 and nd == 80 and splits == min(planned) for rows, nd, splits in seen), seen


def test_a_recorded_step_is_planned_for_its_requests_and_not_for_the_padded_rows():
    """17 requests decode on a graph of 32 rows. What the mixers plan for the recording (into how
    many runs the attention cuts a request's keys) is asked for 17 requests: the padded rows bring
    no work, and a plan for 32 would leave compute units idle."""
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    name, count, n = "B", 17, 4100
    toks = prompts(name, [n + 2] * count, seed=300)
    core = build_core(model_folder(name), num_pages=count * (-(-(n + 2) // 16)) + 4, page_size=16, max_seqs=32,
                      dtype="bfloat16", enable_prefix_caching=False, watermark=0.0)
    core.step.enable_decode_graphs(32, n + 4)
    s = TraceSession(core)
    for r in range(count):
        s.step([{"id": r, "tokens": toks[r][:n], "want": []}])
    out = s.step([{"id": r, "tokens": [toks[r][n]], "want": [0]} for r in range(count)])
    assert out.shape[0] == count and torch.isfinite(out).all()
    (key,) = core.step.graphs.captured
    owners = core.step.plan_owners
    assert key[0] == 32 and owners
    assert key[1] == tuple(part.decode_plan(count, n + 1) for part in owners)
    assert key[1] != tuple(part.decode_plan(32, n + 1) for part in owners), "the test's sizes no longer tell the two apart"


def test_a_shape_that_is_asked_for_rarely_is_served_by_a_recorded_shape_of_more_rows(monkeypatch):
    """Eight requests decode on a graph of eight rows; five of them end, and the three that go on
    are served by that graph until they have asked for as many steps as a recording is taken to
    be worth (three here; a recording costs as much as many steps, and the tail of a batch changes
    its shape every few steps), then by a recording of their own. A graph of more than four times
    the rows does not stand in. The logits are the plain implementation's all along."""
    from test_model_gpu import check, plain_logits
    from dli_amd.engine import decode_graph
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    monkeypatch.setattr(decode_graph, "RECORD_AFTER_STEPS", 3)

    name, count, n = "B", 8, 40
    toks = prompts(name, [n + 8] * count, seed=310)
    core = build_core(model_folder(name), num_pages=count * 4 + 4, page_size=16, max_seqs=8, dtype="bfloat16",
                      enable_prefix_caching=False, watermark=0.0)
    core.step.enable_decode_graphs(8, 64)
    graphs = core.step.graphs
    s = TraceSession(core)
    s.step([{"id": r, "tokens": toks[r][:n], "want": []} for r in range(count)])

    def decode(rows, i, end=()):
        out = s.step([{"id": r, "tokens": [toks[r][n + i]], "want": [0]} for r in rows], end=end)
        check(out, torch.stack([plain_logits(name, toks[r])[n + i] for r in rows]), "bfloat16", f"step {i}, rows {rows}")

    decode(range(8), 0, end=range(3, 8))
    assert len(graphs.captured) == 1 and graphs.replays == 1
    decode(range(3), 1)
    decode(range(3), 2)
    assert len(graphs.captured) == 1 and graphs.replays == 3, "the graph of eight rows stands in twice"
    decode(range(3), 3)
    assert len(graphs.captured) == 2 and graphs.replays == 4
    assert sorted(k[0] for k in graphs.captured) == [4, 8]
    decode(range(3), 4, end=range(1, 3))
    assert len(graphs.captured) == 2 and graphs.replays == 5
    decode(range(1), 5)
    assert len(graphs.captured) == 2 and graphs.replays == 6, "the graph of four rows stands in for one request"
    monkeypatch.setattr(decode_graph, "STAND_IN_ROWS", 2)
    graphs._asked.clear()
    decode(range(1), 6)
    assert sorted(k[0] for k in graphs.captured) == [1, 4, 8], "four rows are more than twice one row"


def test_trace_run_program(tmp_path):
    """bin/trace_run as a user runs it: steps on standard input, `done` lines, <step>.f32 files."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    name = "A"
    cfg, w = P.load_folder(model_folder(name))
    a, b = prompts(name, [70, 19], seed=41)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:37], "want": [0, 36]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[37:39], "want": []}, {"id": "b", "tokens": b[:17], "want": [16]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[17:18], "want": [0]}], "end": []},
        {"step": 3, "entries": [{"id": "a", "tokens": a[39:70], "want": [30]}, {"id": "b", "tokens": b[18:19], "want": [0]}], "end": ["b"]},
        {"step": 7, "entries": [{"id": "c", "tokens": b, "want": [18]}], "end": ["a", "c"]},
    ]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        proc = subprocess.run(
            [sys.executable, str(root / "bin" / "trace_run"), "--model", str(model_folder(name)), "--dtype", dtype,
             "--out", str(out), "--max-tokens", "192"],
            input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        ref_a, ref_b = P.forward_logits(w, cfg, a), P.forward_logits(w, cfg, b)
        want = {0: ref_a[[0, 36]], 1: ref_b[[16]], 2: ref_b[[17]], 3: torch.stack([ref_a[69], ref_b[18]]), 7: ref_b[[18]]}
        assert sorted(p.name for p in out.iterdir()) == sorted(f"{k}.f32" for k in want)
        for k, ref in want.items():
            got = np.fromfile(out / f"{k}.f32", dtype="<f4").reshape(-1, cfg["vocab_size"])
            err = np.abs(got - ref.numpy()).max()
            assert err < (1e-4 if dtype == "float32" else 0.08 * float(ref.abs().max())), (dtype, k, err)
    # a trace that asks for more than the pool holds fails with one clear line
    proc = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", str(model_folder(name)), "--dtype", "float32",
         "--out", str(tmp_path / "x"), "--max-tokens", "64"],
        input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": a, "want": [0]}], "end": []}) + "\n",
        capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0 and "NoFreePagesError" in proc.stderr


@pytest.mark.parametrize("name,count", [("D", 20), ("D", 40), ("A", 20)])
def test_many_requests_decode_together_through_the_engine(name, count):
    """More than sixteen requests at once: configuration D's sizes tile, so its decode steps take
    the product kernel for 17 to 64 rows inside the graphs (A's do not and take the plain path);
    tokens are the plain implementation's either way."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    eng = LLMEngine.for_model(str(model_folder(name)), dtype="bfloat16", num_blocks=4 * count + 8, block_size=16,
                              enable_prefix_caching=False,
                              config=SchedulerConfig(max_num_seqs=count, max_num_batched_tokens=1024))
    ps = prompts(name, [5 + (7 * i) % 23 for i in range(count)], seed=67)
    reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=12)) for i, p in enumerate(ps)]
    while eng.has_unfinished():
        eng.step()
    assert eng.core.step.graphs.replays >= 10
    assert max(s.num_seqs for s in eng.stats.steps) == count
    for r, p in zip(reqs, ps):
        assert len(r.output_ids) == 12
        assert_same_or_near_tie(name, p, r.output_ids, plain_greedy(name, p, 12), margin=0.25)


def test_warm_up_captures_every_graph_that_serving_then_replays():
    """After ``warm_up`` no decode step captures a graph: requests of several lengths and batch
    sizes, one and several tokens per step, only replay what exists, and the tokens are the plain
    implementation's."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams

    name = "D"
    for k in (1, 4):
        eng = LLMEngine.for_model(str(model_folder(name)), dtype="bfloat16", num_blocks=96, block_size=16,
                                  enable_prefix_caching=False,
                                  config=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=256, decode_steps=k))
        graphs = eng.core.step.graphs
        made = eng.warm_up([1, 2, 3, 4], 420)
        assert made == len(graphs.captured) > 0 and eng.warm_up([1, 2, 3, 4], 420) == 0
        before = set(graphs.captured)
        ps = prompts(name, [5, 250, 300, 130], seed=61)
        reqs = [eng.add_request(f"r{i}", p, SamplingParams(max_tokens=70 + 9 * i)) for i, p in enumerate(ps)]
        while eng.has_unfinished():
            eng.step()
        assert set(graphs.captured) == before, set(graphs.captured) - before
        assert graphs.replays > 20
        for r, p in zip(reqs, ps):
            assert_same_or_near_tie(name, p, r.output_ids, plain_greedy(name, p, len(r.output_ids)), margin=0.25)


def test_generate_command_line(tmp_path):
    """``python -m dli_amd random-weights`` then ``... generate`` as a user runs them (the reference's
    flag names, src/dli/server/__main__.py:65-124): the printed ids are the plain implementation's."""
    import json
    import os
    import subprocess
    import sys
    from pathlib import Path

    from tiny_configs import TINY_B

    root = Path(__file__).resolve().parent.parent
    env = dict(os.environ, PYTHONPATH=str(root) + os.pathsep + os.environ.get("PYTHONPATH", ""))
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(TINY_B))
    folder = tmp_path / "model"
    proc = subprocess.run([sys.executable, "-m", "dli_amd", "random-weights", "--config", str(cfg_file), "--out",
                           str(folder), "--seed", "9", "--std", "0.085", "--norm-jitter", "0.1"],
                          capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0, proc.stderr
    assert Path(proc.stdout.strip().splitlines()[-1]) == folder and (folder / "model.safetensors").exists()
    cfg, w = P.load_folder(folder)
    ps = [[11, 5, 300, 42, 7, 7, 129], list(range(3, 3 + 41))]
    (tmp_path / "prompts.txt").write_text(json.dumps(ps[1]) + "\n")
    for dtype, block, extra in (("float32", 8, ["--no-prefix-caching"]), ("bfloat16", 16, ["--max-num-batched-tokens", "24", "--cuda-graphs"]),
                                ("auto", 16, ["--no-cuda-graphs", "--num-blocks", "12"])):
        proc = subprocess.run(
            [sys.executable, "-m", "dli_amd", "generate", "--model", str(folder), "--dtype", dtype, "--block-size",
             str(block), "--max-tokens", "12", "--prompt-ids", " ".join(map(str, ps[0])), "--prompt-file",
             str(tmp_path / "prompts.txt"), *extra],
            capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
        assert proc.returncode == 0, proc.stderr
        got = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("[")]
        assert len(got) == 2 and all(len(g) == 12 for g in got), proc.stdout
        for g, prompt in zip(got, ps):
            want = P.greedy_generate(w, cfg, prompt, 12)
            if dtype == "float32":
                assert g == want
            else:
                toks = list(prompt)
                for a, b in zip(g, want):
                    if a != b:
                        logits = P.forward_logits(w, cfg, toks)[-1]
                        assert 0 <= (logits[b] - logits[a]).item() < 0.25
                        break
                    toks.append(b)
    # a stop token ends a request early; the option's name is the reference's
    stop = P.greedy_generate(w, cfg, ps[0], 12)[4]
    proc = subprocess.run(
        [sys.executable, "-m", "dli_amd", "generate", "--model", str(folder), "--dtype", "float32", "--block-size", "8",
         "--max-tokens", "12", "--prompt-ids", ",".join(map(str, ps[0])), "--stop-token-ids", str(stop)],
        capture_output=True, text=True, timeout=300, env=env, cwd=tmp_path)
    assert proc.returncode == 0, proc.stderr
    out = json.loads([l for l in proc.stdout.splitlines() if l.startswith("[")][0])
    assert out[-1] == stop and len(out) <= 5


def test_generation_without_the_decode_copy_of_the_weights():
    """The second, tile-ordered copy of the matrices is an option: without it the decode steps
    read the row-major matrices (and run the rotation kernel), and greedy generation gives the
    plain implementation's tokens either way."""
    from dli_amd.engine.generate import generate
    from dli_amd.sampling import SamplingParams

    name = "D"
    ps = prompts(name, [9, 40], seed=23)
    want = [plain_greedy(name, p, 20) for p in ps]
    for copy in (True, False):
        got = generate(str(model_folder(name)), ps, SamplingParams(max_tokens=20), dtype="bfloat16", num_blocks=32, cuda_graphs=True,
                       enable_prefix_caching=False, decode_weight_copy=copy)
        for g, w, p in zip(got, want, ps):
            assert len(g) == 20
            assert_same_or_near_tie(name, p, g, w, margin=0.25)


def test_generate_sizes_its_pool_from_the_requests():
    """``generate`` with no pool size: as many pages as its live requests can fill (here the 8 longest
    of 30; the others wait), and every request's tokens are the plain implementation's; the same
    through a pool that holds all 30 at once."""
    from dli_amd.engine.generate import generate, pages_for_requests
    from dli_amd.sampling import SamplingParams

    name = "B"
    lengths = [3 + (7 * i) % 45 for i in range(30)]
    ps = prompts(name, lengths, seed=31)
    news = [4 + i % 9 for i in range(30)]
    want = [plain_greedy(name, p, n) for p, n in zip(ps, news)]
    for seqs in (8, 256):
        got = generate(str(model_folder(name)), ps, [SamplingParams(max_tokens=n) for n in news], dtype="float32",
                       max_num_seqs=seqs, max_num_batched_tokens=64)
        assert got == want, seqs
    few = pages_for_requests([a + b for a, b in zip(lengths, news)], 16, 8, 10 ** 9)
    assert few < pages_for_requests([a + b for a, b in zip(lengths, news)], 16, 256, 10 ** 9)
