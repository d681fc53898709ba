"""The engine at the layer sizes it serves (Llama-3.2-1B's widths, two layers) against the plain
implementation: the kernels that the tiny configurations reach only through their kernel tests
(head size 64 in groups of four, products of depth 2048 and 8192, decode graphs at batch 1 and 8)
run here inside the whole model."""

from __future__ import annotations

import random

import pytest
import torch

import plain_llama as P
from test_model_gpu import check
from tiny_configs import model_folder

pytestmark = pytest.mark.gpu

_plain: dict = {}


_weights: list = []


def plain(tokens):
    key = tuple(tokens)
    if key not in _plain:
        if not _weights:  # converted to 64-bit once, not in every call
            cfg, w = P.load_folder(model_folder("W"))
            _weights.extend([cfg, {k: t.double() for k, t in w.items()}])
        _plain[key] = P.forward_logits(_weights[1], _weights[0], tokens)
    return _plain[key]


def make_core(dtype, pages, page=16, graphs=0):
    from dli_amd.engine.core import build_core

    core = build_core(model_folder("W"), num_pages=pages, page_size=page, max_seqs=max(8, graphs), dtype=dtype,
                      enable_prefix_caching=False, watermark=0.0)
    if graphs:
        core.step.enable_decode_graphs(graphs, pages * page)
    return core


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_whole_prompt_then_decoding_at_serving_widths(dtype):
    from dli_amd.trace import TraceSession

    rng = random.Random(3)
    toks = [rng.randrange(32003) for _ in range(150 if dtype == "bfloat16" else 70)]
    ref = plain(toks)
    core = make_core(dtype, pages=12, graphs=1)
    s = TraceSession(core)
    got = s.step([{"id": "w", "tokens": toks, "want": list(range(len(toks)))}], end=["w"])
    check(got, ref, dtype, "wide whole")
    head = len(toks) - 24
    got = s.step([{"id": "d", "tokens": toks[:head], "want": [head - 1]}])
    check(got, ref[head - 1:head], dtype, "wide prefix")
    for i in range(head, len(toks)):  # one row: the 4x4-block products, through the decode graph in bfloat16
        got = s.step([{"id": "d", "tokens": [toks[i]], "want": [0]}])
        check(got, ref[i:i + 1], dtype, f"wide decode at {i}")
    if dtype == "bfloat16":
        assert core.step.graphs is not None and core.step.graphs.replays >= 24


@pytest.mark.parametrize("count", [8, 24, 40, 64, 130])
def test_requests_decode_together_at_serving_widths(count):
    """Prompts of different lengths go in as mixed batches of portions, then all decode side by
    side: eight through the 16x16-tile products with their fused norm, SwiGLU and residual
    epilogues, 24, 40 and 64 through the product kernel that shares the activations through LDS and
    its finishing kernels (two, three and four row tiles: graphs of 32, 48 and 64 rows), 130
    through the library's products with separate norm, rotation and SwiGLU kernels (a graph of
    144 rows)."""
    from dli_amd.trace import TraceSession

    rng = random.Random(4 + count)
    lens = [rng.randrange(18, 44) for _ in range(count)]
    steps = 10 if count == 8 else 4
    toks = [[rng.randrange(32003) for _ in range(n + steps)] for n in lens]
    core = make_core("bfloat16", pages=4 * count + 8, graphs=count)
    s = TraceSession(core)
    fed = [0] * count
    # prompts in two mixed steps of portions
    for part in (0, 1):
        entries = []
        for r in range(count):
            n = lens[r] // 2 if part == 0 else lens[r] - lens[r] // 2
            entries.append({"id": r, "tokens": toks[r][fed[r]:fed[r] + n], "want": [n - 1] if part else []})
            fed[r] += n
        out = s.step(entries)
    rows = torch.stack([plain(toks[r])[lens[r] - 1] for r in range(count)])
    check(out, rows, "bfloat16", "wide mixed prompts")
    for stepno in range(steps):
        entries = [{"id": r, "tokens": [toks[r][fed[r]]], "want": [0]} for r in range(count)]
        out = s.step(entries)
        rows = torch.stack([plain(toks[r])[fed[r]] for r in range(count)])
        check(out, rows, "bfloat16", f"wide decode step {stepno} of {count}")
        for r in range(count):
            fed[r] += 1
    assert core.step.graphs.replays >= steps


@pytest.mark.parametrize("count", [1, 2])
def test_one_and_two_requests_decode_without_a_merge_kernel(count, monkeypatch):
    """With one or two rows (two: where the limit is set so) and keys enough for two runs, the o
    projection merges the runs of keys itself: the path is taken (counted), agrees with the plain implementation, and gives the
    bits of the path with the merge kernel. The steps' logits are copied on the stream and looked
    at only after the last step: a replay must not refill its staging buffer while the copy of the
    step before is still queued."""
    from dli_amd.kernels import ops
    from dli_amd.parts import attention
    from dli_amd.trace import TraceSession

    rng = random.Random(11 + count)
    lens = [600, 540][:count]
    steps = 6
    toks = [[rng.randrange(32003) for _ in range(n + steps)] for n in lens]
    calls = []
    real = ops.skinny_gemm_merged
    monkeypatch.setattr(ops, "skinny_gemm_merged", lambda *a, **k: (calls.append(a[2]), real(*a, **k))[1])

    def run(limit):
        monkeypatch.setattr(attention, "MERGE_IN_PRODUCT_ROWS", limit)
        core = make_core("bfloat16", pages=80, graphs=count)
        s = TraceSession(core)
        s.step([{"id": r, "tokens": toks[r][:lens[r]], "want": []} for r in range(count)])
        outs = []
        for i in range(steps):
            outs.append(s.step([{"id": r, "tokens": [toks[r][lens[r] + i]], "want": [0]} for r in range(count)]).clone())
        return outs

    merged = run(2)
    assert calls and all(splits >= 2 for splits in calls)
    for i, out in enumerate(merged):
        rows = torch.stack([plain(toks[r])[lens[r] + i] for r in range(count)])
        check(out, rows, "bfloat16", f"decode step {i} of {count} without a merge kernel")
    seen = len(calls)
    separate = run(0)
    assert len(calls) == seen
    for a, b in zip(merged, separate):
        assert torch.equal(a, b)


def test_decode_attention_merges_its_runs_of_keys_in_the_launch(monkeypatch):
    """Four requests with keys enough for several runs: the decode attention launches merge by
    themselves (counted: arrival counters are passed), also when replayed from graphs, step after
    step on the same counters; the result agrees with the plain implementation and has the bits of
    the path with the merge kernel."""
    from dli_amd.kernels import ops
    from dli_amd.parts import attention
    from dli_amd.trace import TraceSession

    rng = random.Random(23)
    lens = [600, 540, 280, 17]
    steps = 6
    toks = [[rng.randrange(32003) for _ in range(n + steps)] for n in lens]
    seen = []
    real = ops.attention_decode

    def counted(*a, **k):
        seen.append((a[9] if len(a) > 9 else k.get("splits", 1), k.get("arrivals") is not None))
        return real(*a, **k)

    monkeypatch.setattr(ops, "attention_decode", counted)

    def run(self_merging):
        if not self_merging:
            monkeypatch.setattr(attention.GQAttention, "arrival_counters", lambda self, needed: None)
        core = make_core("bfloat16", pages=100, graphs=4)
        s = TraceSession(core)
        s.step([{"id": r, "tokens": toks[r][:lens[r]], "want": []} for r in range(4)])
        outs = []
        for i in range(steps):
            outs.append(s.step([{"id": r, "tokens": [toks[r][lens[r] + i]], "want": [0]} for r in range(4)]).clone())
        assert core.step.graphs.replays >= steps - 1
        return outs

    merged = run(True)
    assert seen and all(splits >= 2 and counters for splits, counters in seen)
    for i, out in enumerate(merged):
        rows = torch.stack([plain(toks[r])[lens[r] + i] for r in range(4)])
        check(out, rows, "bfloat16", f"decode step {i} that merges in the attention launch")
    del seen[:]
    separate = run(False)
    assert seen and not any(counters for _, counters in seen)
    for a, b in zip(merged, separate):
        assert torch.equal(a, b)


_one_b: dict = {}


def one_b():
    """Llama-3.2-1B with random weights, written to a folder once (a billion weights: drawn on the
    GPU) and loaded as the plain implementation reads a checkpoint; its weights in 64-bit are
    kept, so that every plain evaluation does not convert them again."""
    if not _one_b:
        folder = model_folder("1B", device="cuda")
        cfg, w = P.load_folder(folder)
        assert cfg["num_hidden_layers"] == 16 and w["model.embed_tokens.weight"].shape == (128256, 2048)
        _one_b.update(folder=folder, cfg=cfg, w=w, w64={k: t.double() for k, t in w.items()}, drift=None)
    return _one_b


def one_b_drift(toks, ref):
    """Rounding adds up over 16 layers: how far bfloat16 may drift on average is measured, not
    guessed, by evaluating the plain implementation itself in bfloat16 (once). The engine
    accumulates in 32-bit where that evaluation rounds, so it must not be further from the 64-bit
    logits."""
    m = one_b()
    if m["drift"] is None:
        rounded = P.forward_logits(m["w"], m["cfg"], toks, dtype=torch.bfloat16).double()
        m["drift"] = ((rounded - ref).abs().max(dim=-1).values / ref.abs().max(dim=-1).values).mean().item()
        assert 0.01 < m["drift"] < 0.08, m["drift"]
    return m["drift"]


def test_llama_3_2_1b_at_full_depth_and_vocabulary():
    """All 16 layers and all 128,256 vocabulary rows of Llama-3.2-1B (random weights written to a
    folder and loaded by name like a checkpoint), 32-bit and bfloat16 against the plain
    implementation in 64-bit: the prompt whole, then its last tokens one by one (the reference's
    parity bound is tests/unit/model/test_reference_parity.py:20; here the bounds are those of
    every other whole-model test)."""
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    m = one_b()
    folder = m["folder"]
    rng = random.Random(8)
    toks = [rng.randrange(128256) for _ in range(64)]
    ref = P.forward_logits(m["w64"], m["cfg"], toks)
    drift = one_b_drift(toks, ref)
    for dtype in ("float32", "bfloat16"):
        core = build_core(folder, num_pages=8, page_size=16, max_seqs=2, dtype=dtype,
                          enable_prefix_caching=False, watermark=0.0)
        core.step.enable_decode_graphs(1, 128)
        s = TraceSession(core)
        got = s.step([{"id": "p", "tokens": toks, "want": list(range(64))}], end=["p"])
        check(got, ref, dtype, f"1B whole {dtype}", mean_rtol=drift)
        got = s.step([{"id": "d", "tokens": toks[:56], "want": [55]}])
        check(got, ref[55:56], dtype, f"1B prefix {dtype}")
        for i in range(56, 64):
            got = s.step([{"id": "d", "tokens": [toks[i]], "want": [0]}])
            check(got, ref[i:i + 1], dtype, f"1B decode at {i} {dtype}")
        del core, s
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_llama_3_2_1b_in_portions_and_in_mixed_batches(dtype):
    """The same model cut the other two ways (the reference's
    tests/parity/test_engine_parity.py:7-12 names all of them for its real checkpoint): one request
    in portions of changing size down to two tokens, and five requests of 40 to 100 tokens mixed,
    up to four live, portions of some beside single tokens of others, in a pool that the four
    longest fill to the last page, so that the fifth runs in pages that another one wrote before;
    decode graphs on in bfloat16, as serving has them."""
    from test_model_gpu import mixed_trace
    from dli_amd.engine.core import build_core
    from dli_amd.trace import TraceSession

    m = one_b()
    rng = random.Random(18)
    lengths = [100, 92, 70, 50, 40]
    all_toks = [[rng.randrange(128256) for _ in range(n)] for n in lengths]
    refs = [P.forward_logits(m["w64"], m["cfg"], t) for t in all_toks]
    drift = one_b_drift(all_toks[2], refs[2])
    pages = sum(-(-n // 16) for n in lengths[:4])
    core = build_core(m["folder"], num_pages=pages, page_size=16, max_seqs=4, dtype=dtype,
                      enable_prefix_caching=False, watermark=0.0)
    core.step.enable_decode_graphs(4, pages * 16)
    s = TraceSession(core)
    toks, ref, pos = all_toks[0], refs[0], 0
    sizes = [16, 7, 5, 3, 2, 9, 2, 31, 4, 2, 17]
    for k in range(100):
        n = min(sizes[k % len(sizes)], len(toks) - pos)
        if len(toks) - pos - n == 1:  # never leave a single token: portions go down to two
            n += 1
        got = s.step([{"id": "r", "tokens": toks[pos:pos + n], "want": list(range(n))}])
        check(got, ref[pos:pos + n], dtype, f"1B portion [{pos},{pos + n}) {dtype}", mean_rtol=drift)
        pos += n
        if pos == len(toks):
            break
    s.step([], end=["r"])
    mixed_trace(core, all_toks, lambda r: refs[r], dtype, f"1B {dtype}", seed=19, mean_rtol=drift)
    if dtype == "bfloat16":
        assert core.step.graphs.replays > 0


def test_a_prompt_of_1700_tokens_whole_and_on_top_of_cached_keys(monkeypatch):
    """1,700 tokens at the 1B widths are 54 query tiles of eight kv heads each: between one and two
    workgroups a compute unit, so that units work on two tiles of different lengths at a time and
    the longest tiles have their keys cut into two runs that two workgroups share. The whole model
    through the prefill attention as the step lists its tiles, whole and as a portion on top of
    cached keys, against the plain implementation."""
    from dli_amd.kernels import ops
    from dli_amd.trace import TraceSession

    rng = random.Random(29)
    toks = [rng.randrange(32003) for _ in range(1700)]
    ref = plain(toks)
    seen = []
    real = ops.attention_prefill

    def counted(*a, **k):
        seen.append((a[7].shape[0], a[13]))  # entries of the tile list, and how many tiles are listed twice, with half their keys each
        return real(*a, **k)

    monkeypatch.setattr(ops, "attention_prefill", counted)
    core = make_core("bfloat16", pages=110)
    core.model.native_steps = False  # through the parts, so that the launches can be counted here
    s = TraceSession(core)
    want = [0, 17, 511, 512, 1023, 1699]
    got = s.step([{"id": "w", "tokens": toks, "want": want}], end=["w"])
    check(got, ref[want], "bfloat16", "1,700 tokens whole")
    assert seen and all(entries == 54 + cut and cut > 0 for entries, cut in seen)
    got = s.step([{"id": "p", "tokens": toks[:60], "want": [59]}])
    check(got, ref[59:60], "bfloat16", "first portion")
    got = s.step([{"id": "p", "tokens": toks[60:], "want": [w - 60 for w in want[2:]]}], end=["p"])
    check(got, ref[want[2:]], "bfloat16", "1,640 tokens on top of 60 cached keys")
