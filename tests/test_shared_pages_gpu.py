"""Requests whose block tables name the same physical pages, replayed against the plain logits:
a fork that writes into a shared, partly filled page (copy-on-write before the write), and live
requests on a shared prefix that content reuse handed to them (the reference's
tests/unit/model/test_paged_generation.py:53-96), in 32-bit and in bfloat16."""

from __future__ import annotations

import pytest
import torch

from test_model_gpu import check, plain_logits, prompts_for
from tiny_configs import model_folder

pytestmark = pytest.mark.gpu

CASES = [("A", 16, "float32"), ("A", 16, "bfloat16"), ("B", 8, "float32"), ("B", 16, "bfloat16"),
         ("D", 16, "bfloat16")]


def make(name, dtype, pages, page, reuse):
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    core = build_core(model_folder(name), num_pages=pages, page_size=page, max_seqs=8, dtype=dtype,
                      enable_prefix_caching=reuse, watermark=0.0)
    core.step.enable_decode_graphs(8, pages * page)  # as serving does (bfloat16 only)
    return core, TraceSession(core)


def page_rows(core, page_id, filled):
    """Keys and values of the first ``filled`` slots of a page, every layer."""
    out = []
    for cache in core.store.layers:
        out.append(cache.k_pages[page_id, :, :filled, :].clone())
        out.append(cache.v_pages[page_id, :, :, :filled].clone())
    return out


@pytest.mark.parametrize("name,page,dtype", CASES)
def test_fork_writes_into_a_shared_partial_page_after_a_copy(name, page, dtype):
    core, s = make(name, dtype, pages=24, page=page, reuse=False)
    mgr = core.manager
    n0 = 2 * page + page // 2 + 1                     # the third page is partly filled and shared
    prompt, cont_p, cont_c = prompts_for(name, [n0, 40, 40], seed=71)
    got = s.step([{"id": "p", "tokens": prompt, "want": [n0 - 1]}])
    check(got, plain_logits(name, prompt)[n0 - 1:], dtype, f"{name} prompt")
    s.fork("p", "c")
    shared = mgr.block_table("p")[2]
    assert mgr.block_table("c") == mgr.block_table("p")
    filled = n0 - 2 * page
    before = page_rows(core, shared, filled)
    replays = core.step.graphs.replays if core.step.graphs else 0
    seq = {"p": list(prompt), "c": list(prompt)}
    # both write position n0 in the same step: the first asks for a copy, the second then owns the page alone
    sizes_p = [1, 1, 1, 3, 1, 2, 1, 1, 5, 1]
    sizes_c = [1, 1, 4, 1, 1, 1, 2, 1, 1, 7]
    at = {"p": 0, "c": 0}
    for step, (np_, nc) in enumerate(zip(sizes_p, sizes_c)):
        entries = []
        for rid, cont, n in (("p", cont_p, np_), ("c", cont_c, nc)):
            toks = cont[at[rid]:at[rid] + n]
            at[rid] += n
            seq[rid] += toks
            entries.append({"id": rid, "tokens": toks, "want": list(range(n))})
        got = s.step(entries)
        want = torch.cat([plain_logits(name, seq["p"])[-np_:], plain_logits(name, seq["c"])[-nc:]])
        check(got, want, dtype, f"{name} fork step {step}")
        if step == 0:
            assert mgr.stats().cow_copies == 1
            tp, tc = mgr.block_table("p"), mgr.block_table("c")
            assert tp[:2] == tc[:2] and tp[2] != tc[2] and shared in (tp[2], tc[2])
            if core.step.graphs:
                assert core.step.graphs.replays == replays, "a step with page copies runs eagerly"
        if step == 1 and core.step.graphs:
            assert core.step.graphs.replays == replays + 1, "the next decode-only step replays a graph"
    assert mgr.stats().cow_copies == 1
    # what the prompt wrote into the shared page is in both pages, untouched by either's tokens
    for rid in ("p", "c"):
        after = page_rows(core, mgr.block_table(rid)[2], filled)
        assert all(torch.equal(a, b) for a, b in zip(after, before)), rid
    mgr.check_invariants()
    s.step([], end=["p", "c"])
    assert mgr.stats().used_pages == 0


@pytest.mark.parametrize("name,page,dtype", CASES)
def test_live_requests_on_the_same_prefix_pages(name, page, dtype):
    core, s = make(name, dtype, pages=40, page=page, reuse=True)
    mgr = core.manager
    prefix, sa, sb, sc = prompts_for(name, [3 * page + 5, 30, 41, 22], seed=72)
    s.step([{"id": "warm", "tokens": prefix, "want": []}], end=["warm"])  # leaves three full pages in the index
    a, b = prefix[:3 * page] + sa, prefix[:3 * page] + sb
    c = prefix[:2 * page] + sc                         # shares two of them
    ref = {"a": plain_logits(name, a), "b": plain_logits(name, b), "c": plain_logits(name, c)}
    toks = {"a": a, "b": b, "c": c}
    fed = {}

    def run(parts):
        entries, want = [], []
        for rid, n in parts:
            first = rid not in fed
            lo = 0 if first else fed[rid]
            hi = min(len(toks[rid]), (shared_tokens[rid] if first else lo) + n)
            start = shared_tokens[rid] if first else lo
            entries.append({"id": rid, "tokens": toks[rid][lo:hi], "want": list(range(start - lo, hi - lo))})
            want.append(ref[rid][start:hi])
            fed[rid] = hi
        got = s.step(entries)
        check(got, torch.cat(want), dtype, f"{name} shared prefix {parts}")

    shared_tokens = {"a": 3 * page, "b": 3 * page, "c": 2 * page}
    run([("a", 7)])
    run([("a", 2), ("b", 9)])
    assert mgr.block_table("a")[:3] == mgr.block_table("b")[:3]
    assert mgr.stats().prompt_tokens_hit == 6 * page
    run([("b", 3), ("c", 5), ("a", 1)])
    assert mgr.block_table("c")[:2] == mgr.block_table("a")[:2] and mgr.block_table("c")[2] != mgr.block_table("a")[2]
    replays = core.step.graphs.replays if core.step.graphs else 0
    while any(fed[r] < len(toks[r]) for r in toks):
        live = [r for r in ("c", "a", "b") if fed[r] < len(toks[r])]
        run([(r, 1) for r in live])                    # decoded tokens of all three, on shared pages
        if fed["c"] < len(toks["c"]) - 6:
            run([("c", 4), ("a", 1)] if fed["a"] < len(toks["a"]) else [("c", 4)])
    if core.step.graphs:
        assert core.step.graphs.replays > replays + 10
    mgr.check_invariants()
    assert mgr.stats().cow_copies == 0
    s.step([], end=["a", "b", "c"])
    mgr.reset_prefix_cache()
    assert mgr.stats().used_pages == 0 and mgr.stats().free_pages == mgr.stats().num_pages
