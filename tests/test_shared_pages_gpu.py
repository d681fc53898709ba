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


import contextlib


@contextlib.contextmanager
def three_groups_toy(window):
    """A toy architecture whose three attention layers form three cache groups: every key, a
    window of keys, every key with other head sizes. Yields ``(model folder, plain, vocab)``;
    ``plain(tokens)`` is a 64-bit model of the toy, written here with the plain implementation's
    parts and a band mask of its own."""
    import math
    import tempfile

    import plain_llama as P
    from dli_amd.config import register_architecture, unregister_architecture
    from dli_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from dli_amd.weights import write_random_model

    h, inter, vocab, eps, theta = 48, 80, 53, 1e-5, 1000.0
    shapes = [dict(num_heads=3, num_kv_heads=1, head_dim=16, window=0),
              dict(num_heads=3, num_kv_heads=1, head_dim=16, window=window),
              dict(num_heads=2, num_kv_heads=2, head_dim=32, window=0)]

    def build(cfg):
        norm = dict(width=h, eps=eps)
        layers = []
        for i, shape in enumerate(shapes):
            p = f"layers.{i}."
            pos = PartSpec("rotary", dict(dim=shape["head_dim"], theta=theta))
            layers.append(LayerSpec(PartSpec("pre_norm"), {
                "mixer_norm": ("norm", PartSpec("rms_norm", norm, p + "n1.")),
                "mixer": ("mixer", PartSpec("gqa_attention", dict(shape, hidden_size=h, position=pos), p + "attn.")),
                "feed_forward_norm": ("norm", PartSpec("rms_norm", norm, p + "n2.")),
                "feed_forward": ("feed_forward", PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=inter),
                                                          p + "mlp."))}))
        return ModelSpec(
            architecture="ToyThreeGroupsForCausalLM", vocab_size=vocab, hidden_size=h,
            embedding=PartSpec("token_embedding", dict(vocab_size=vocab, hidden_size=h), "embed."),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in range(3)),
            final_norm=PartSpec("rms_norm", norm, "norm."),
            head=PartSpec("linear_head", dict(vocab_size=vocab, hidden_size=h, tied=True), "head."))

    def banded_attention(x, w, prefix, shape):
        """Projections, rotation, softmax over the keys j with i - window < j <= i, output projection."""
        n, nh, nkv, d = x.shape[0], shape["num_heads"], shape["num_kv_heads"], shape["head_dim"]
        cos, sin = P.rope_cos_sin(P.inverse_frequencies({"rope_type": "default", "theta": theta}, d),
                                  torch.arange(n), torch.float64)
        q = P.apply_rope(P.linear(x, w[prefix + "q_proj.weight"]).view(n, nh, d).transpose(0, 1), cos, sin)
        k = P.apply_rope(P.linear(x, w[prefix + "k_proj.weight"]).view(n, nkv, d).transpose(0, 1), cos, sin)
        v = P.linear(x, w[prefix + "v_proj.weight"]).view(n, nkv, d).transpose(0, 1)
        i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
        seen = (j <= i) & ((j > i - shape["window"]) if shape["window"] else (j >= 0))
        out = torch.empty_like(q)
        for head in range(nh):
            scores = (q[head] @ k[head // (nh // nkv)].T) / math.sqrt(d)
            out[head] = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1) @ v[head // (nh // nkv)]
        return P.linear(out.transpose(0, 1).reshape(n, nh * d), w[prefix + "o_proj.weight"])

    register_architecture("ToyThreeGroupsForCausalLM", dict, build)
    try:
        with tempfile.TemporaryDirectory() as tmp:
            folder = write_random_model(tmp, {"architectures": ["ToyThreeGroupsForCausalLM"]}, seed=21, std=0.15,
                                        norm_jitter=0.1)
            w = {k: v.double() for k, v in P.load_folder(folder)[1].items()}

            def plain(tokens):
                x = w["embed.weight"][torch.tensor(tokens)]
                for i, shape in enumerate(shapes):
                    p = f"layers.{i}."
                    x = x + banded_attention(P.rms_norm(x, w[p + "n1.weight"], eps), w, p + "attn.", shape)
                    x = x + P.swiglu_mlp(P.rms_norm(x, w[p + "n2.weight"], eps), w, p + "mlp.")
                return P.linear(P.rms_norm(x, w["norm.weight"], eps), w["embed.weight"])

            yield folder, plain, vocab
    finally:
        unregister_architecture("ToyThreeGroupsForCausalLM")


@pytest.mark.parametrize("dtype,page,window", [("float32", 4, 10), ("bfloat16", 16, 24)])
def test_a_toy_model_of_three_cache_groups_is_served_a_prefix_from_all_of_them(dtype, page, window):
    """The requests of a model with three cache groups (every key, a window of keys, every key with
    other head sizes) are served a prefix that an earlier request left behind, from all three
    groups at once (the window group gives only the pages that the first computed token still
    reaches; the table starts with released entries); they step in portions and token by token
    beside each other against the plain model of the toy. The pool has no page to spare while the
    two run, so the groups that keep every key lose the rest of the prefix, and a later request is
    served the shorter run that all three can still give."""
    from dli_amd.cache import RELEASED
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession
    from dli_amd.weights import load_model

    with three_groups_toy(window) as (folder, plain, vocab):
        rng = torch.Generator().manual_seed(5)
        rand = lambda n: torch.randint(0, vocab, (n,), generator=rng).tolist()
        prefix = rand(5 * page + 3)
        toks = {"a": prefix[:4 * page] + rand(21), "b": prefix[:3 * page] + rand(14), "c": prefix + rand(9)}
        ref = {rid: plain(t) for rid, t in toks.items()}
        # as many pages as the two live requests need together, three of them shared: whatever
        # else the index holds has to go while they run
        pages = -(-len(toks["a"]) // page) + -(-len(toks["b"]) // page) - 3
        core = build_core(load_model(folder, dtype=dtype), num_pages=pages, page_size=page, max_seqs=4, watermark=0.0)
        mgr = core.manager
        assert mgr.prefix_caching and [g.kind for g in mgr.groups] == ["full", "window", "full"]
        core.step.enable_decode_graphs(4, pages * page)
        s = TraceSession(core)
        got = s.step([{"id": "w", "tokens": prefix, "want": [len(prefix) - 1]}], end=["w"])
        check(got, plain(prefix)[-1:], dtype, "three groups, the prefix")
        fed = {}

        def run(plan):
            entries, want = [], []
            for rid, n in plan:
                lo = fed.get(rid, 0)
                start = shared[rid] if rid not in fed else lo      # a new request is fed from its first token
                hi = min(len(toks[rid]), start + n)
                entries.append({"id": rid, "tokens": toks[rid][lo:hi], "want": list(range(start - lo, hi - lo))})
                want.append(ref[rid][start:hi])
                fed[rid] = hi
            check(s.step(entries), torch.cat(want), dtype, f"three groups, {plan} up to {fed}")
            mgr.check_invariants()

        shared = {"a": 4 * page, "b": 3 * page}
        run([("a", 6)])
        first = max(0, 4 * page - window + 1) // page       # the window at a's first computed token
        assert first > 0
        assert mgr.block_table("a", 1)[:first] == (RELEASED,) * first and RELEASED not in mgr.block_table("a", 0)
        run([("a", 3), ("b", 5)])
        assert mgr.stats().prompt_tokens_hit == 7 * page
        for g in (0, 2):
            assert mgr.block_table("a", g)[:3] == mgr.block_table("b", g)[:3]
        run([("b", 2), ("a", 5)])
        while fed["a"] < len(toks["a"]) or fed["b"] < len(toks["b"]):
            run([(rid, 1) for rid in ("a", "b") if fed[rid] < len(toks[rid])])
        if dtype == "bfloat16":
            assert core.step.graphs.replays > 0
        assert mgr.stats().window_pages_released > 0
        s.step([], end=["a", "b"])
        # the whole prefix again: what the pools still hold of it decides how much is served
        served = -(-len(toks["c"]) // page) - mgr.pages_needed_for_prompt(toks["c"])
        assert mgr.pools[0].evictions > 0 and served == 4
        shared["c"] = served * page
        run([("c", 4)])
        run([("c", 100)])
        s.step([], end=["c"])
        mgr.reset_prefix_cache()
        assert mgr.stats().used_pages == 0 and mgr.stats().free_pages == mgr.stats().num_pages


def test_an_engine_for_the_toy_of_three_cache_groups_generates_the_same_with_and_without_reuse():
    """Through the engine's own loop (scheduler, eight tokens a step where it may, too few pages
    for all requests at once, so that some are preempted and computed again): greedy tokens of
    requests on a common prefix are those of the plain model of the toy, with content reuse in all
    three groups and without it; with it, prompt tokens are served from the indexes."""
    from dli_amd.engine import LLMEngine, SchedulerConfig
    from dli_amd.sampling import SamplingParams
    from dli_amd.weights import load_model

    page, window, new = 4, 10, 14
    with three_groups_toy(window) as (folder, plain, vocab):
        rng = torch.Generator().manual_seed(9)
        rand = lambda n: torch.randint(0, vocab, (n,), generator=rng).tolist()
        prefix = rand(6 * page + 1)
        prompts = {"w": prefix, "a": prefix[:5 * page] + rand(7), "b": prefix[:4 * page] + rand(11),
                   "c": prefix[:5 * page + 2] + rand(3), "d": rand(9)}

        def plain_greedy(prompt):
            seq = list(prompt)
            for _ in range(new):
                logits = plain(seq)[-1]
                top = torch.topk(logits, 2).values
                assert top[0] - top[1] > 1e-3, "a near tie: the comparison would prove little"
                seq.append(int(logits.argmax()))
            return seq[len(prompt):]

        want = {rid: plain_greedy(p) for rid, p in prompts.items()}
        model = load_model(folder, dtype="float32")
        hits = {}
        for reuse in (True, False):
            need = max(-(-(len(p) + new) // page) for p in prompts.values())
            engine = LLMEngine.for_model(model, num_blocks=need + 6, block_size=page, enable_prefix_caching=reuse,
                                         config=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=16, decode_steps=8))
            got = {rid: [] for rid in prompts}
            engine.add_request("w", prompts["w"], SamplingParams(max_tokens=new, ignore_eos=True))
            steps = 0
            while engine.has_unfinished():
                for out in engine.step():
                    got[out.request_id] += out.new_token_ids
                steps += 1
                if steps == 3:    # the others arrive while the first still runs
                    for rid in ("a", "b", "c", "d"):
                        engine.add_request(rid, prompts[rid], SamplingParams(max_tokens=new, ignore_eos=True))
                engine.manager.check_invariants()
                assert steps < 400
            assert got == want, f"reuse {reuse}"
            stats = engine.manager.stats()
            hits[reuse] = stats.prompt_tokens_hit
            assert sum(st.num_preempted for st in engine.stats.steps) > 0, "the pool was meant to be too small for all of them"
            engine.manager.reset_prefix_cache()
            assert engine.manager.stats().used_pages == 0
        assert hits[True] >= 4 * page and hits[False] == 0
