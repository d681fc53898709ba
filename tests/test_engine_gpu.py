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
    """Tokens must be the plain implementation's; a difference is allowed only where the plain
    logits of the two candidates are within ``margin`` of each other (then the run is cut there)."""
    cfg, w = P.load_folder(model_folder(name))
    toks = list(prompt)
    for g, x in zip(got, want):
        if g != x:
            logits = P.forward_logits(w, cfg, toks)[-1]
            gap = (logits[x] - logits[g]).item()
            assert 0 <= gap < margin, f"token {g} instead of {x}: plain logits differ by {gap}"
            return
        toks.append(x)


@pytest.mark.parametrize("name,dtype,block", [("A", "float32", 16), ("B", "float32", 8), ("A", "bfloat16", 16),
                                              ("B", "bfloat16", 16), ("C", "bfloat16", 32)])
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


@pytest.mark.parametrize("name,block", [("A", 16), ("C", 32)])
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
