"""The sampling kernel against the plain distribution and a host Philox; vectors from the
reference's tests/unit/test_sampling.py."""

from __future__ import annotations

from collections import Counter

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

LOGITS = torch.log(torch.tensor([[0.5, 0.3, 0.15, 0.05]]))


def philox_uniform(seed: int, counter: int) -> float:
    """Philox4x32-10, first output word, top 24 bits as a float in [0, 1)."""
    m = 0xFFFFFFFF
    c = [counter & m, (counter >> 32) & m, 0, 0]
    k = [seed & m, (seed >> 32) & m]
    for _ in range(10):
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & m, p1 & m, ((p0 >> 32) ^ c[3] ^ k[1]) & m, p0 & m]
        k = [(k[0] + 0x9E3779B9) & m, (k[1] + 0xBB67AE85) & m]
    return (c[0] >> 8) / 16777216.0


def draw(logits, params, seeds, draws):
    from dli_amd.sampling.sampler import sample

    return sample(logits.cuda().float(), params, seeds, draws)


def test_greedy_is_argmax_lowest_id_on_ties():
    from dli_amd.sampling import SamplingParams

    assert draw(torch.tensor([[0.1, 2.0, 2.0, -1.0]]), [SamplingParams()], [None], [0]) == [1]
    big = torch.full((3, 128256), -5.0)
    big[0, 77777] = 1.0
    big[1, 128255] = 1.0
    big[2, 5] = big[2, 100000] = 3.0
    assert draw(big, [SamplingParams()] * 3, [None] * 3, [0] * 3) == [77777, 128255, 5]


def test_top_k_one_and_tiny_top_p_reduce_to_greedy():
    from dli_amd.sampling import SamplingParams

    assert draw(LOGITS, [SamplingParams(temperature=1.0, top_k=1)], [None], [0]) == [0]
    assert draw(LOGITS, [SamplingParams(temperature=1.0, top_p=1e-6)], [3], [0]) == [0]


def freqs(params, n=10000):
    rows = LOGITS.expand(n, 4).contiguous()
    out = draw(rows, [params] * n, [123] * n, list(range(n)))
    c = Counter(out)
    return {t: c[t] / n for t in c}


def test_frequencies_follow_the_distribution():
    from dli_amd.sampling import SamplingParams

    f = freqs(SamplingParams(temperature=1.0))
    for tok, p in enumerate([0.5, 0.3, 0.15, 0.05]):
        assert abs(f.get(tok, 0.0) - p) < 0.02  # 10k draws: about four sigma
    fk = freqs(SamplingParams(temperature=1.0, top_k=2))
    assert set(fk) == {0, 1} and abs(fk[0] - 0.625) < 0.02
    fp = freqs(SamplingParams(temperature=1.0, top_p=0.6))
    assert set(fp) == {0, 1}
    ft = freqs(SamplingParams(temperature=0.5))
    assert abs(ft[0] - 0.25 / 0.365) < 0.02


@pytest.mark.parametrize("vocab", [50, 384, 5000])
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.9, 20, 0.95), (1.3, -1, 0.7), (0.7, 5, 1.0), (2.0, -1, 1.0)])
def test_each_draw_is_the_inverse_cdf_of_the_plain_distribution(vocab, temperature, top_k, top_p):
    """The kernel's token for (seed, draw) must be where the host Philox uniform falls in the
    cumulative plain distribution (vocabulary order), up to rounding at the cell's edges."""
    from dli_amd.sampling import SamplingParams

    torch.manual_seed(vocab)
    logits = torch.randn(1, vocab) * 2
    probs = P.sampling_probabilities(logits[0], temperature, top_k, top_p)
    cdf = torch.cumsum(probs, 0)
    params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p)
    n = 200
    got = draw(logits.expand(n, vocab).contiguous(), [params] * n, [77] * n, list(range(n)))
    for i, tok in enumerate(got):
        u = philox_uniform(77, i)
        assert probs[tok] > 0, "a token outside the kept set was drawn"
        lo = cdf[tok] - probs[tok]
        assert lo - 1e-4 <= u <= cdf[tok] + 1e-4, (i, tok, u, float(lo), float(cdf[tok]))


def test_a_request_draws_the_same_alone_and_in_a_batch():
    from dli_amd.sampling import SamplingParams

    torch.manual_seed(0)
    rows = torch.randn(5, 50)
    p = SamplingParams(temperature=0.9, top_p=0.95, top_k=20)
    alone = [draw(rows[2:3], [p], [102], [step])[0] for step in range(10)]
    batched = [draw(rows, [p] * 5, [100, 101, 102, 103, 104], [step] * 5)[2] for step in range(10)]
    assert alone == batched
    mixed = draw(torch.tensor([[0.0, 5.0, 0.0], [5.0, 0.0, 0.0]]),
                 [SamplingParams(), SamplingParams(temperature=1.0, top_k=1)], [None, None], [0, 0])
    assert mixed == [1, 0]
    with pytest.raises(ValueError, match="generator"):
        draw(LOGITS, [SamplingParams(temperature=1.0)], [None], [0])


def test_invalid_params():
    from dli_amd.sampling import SamplingParams

    for kw in ({"max_tokens": 0}, {"temperature": -0.1}, {"temperature": float("nan")}, {"top_k": 0},
               {"top_p": 0.0}, {"top_p": 1.5}, {"temperature": 2.5}):
        with pytest.raises(ValueError, match="must"):
            SamplingParams(**kw)
    assert SamplingParams(top_k=1, temperature=1.0).greedy and SamplingParams().greedy


@pytest.mark.parametrize("rows,n,k,workgroups", [(1, 3088, 2048, 0), (8, 1008, 1024, 5), (16, 272, 4096, 1), (5, 128256, 2048, 0)])
def test_the_logits_kernel_leaves_the_first_stage_of_the_argmax(rows, n, k, workgroups):
    """The kernel that makes the logits of a few rows has each of them in a register once: asked
    to, every workgroup leaves each row's best logit and its lowest index, and the best of those
    parts is the row's argmax (ties to the lowest index: several logits are made equal and the
    largest on purpose, far apart, so that they fall to different workgroups)."""
    from dli_amd.kernels import ops

    torch.manual_seed(rows + n)
    x = torch.randn(rows, k, device="cuda").bfloat16()
    w = (torch.randn(n, k, device="cuda") / k ** 0.5).bfloat16()
    for r in range(rows):  # equal weight rows give equal logits: a tie between n//5 + r and 4n//5 + r, above the rest
        lo, hi = n // 5 + r, 4 * n // 5 + r
        w[lo] = w[hi] = (x[r].float() / x[r].float().norm() * 8).bfloat16()
    wt = ops.tile_weights(w)
    out = torch.empty(rows, n, device="cuda", dtype=torch.float32)
    scratch = ops.sample_scratch(rows, x.device)
    scratch[0].fill_(float("nan"))
    scratch[1].fill_(-7)
    parts = ops.head_gemm(x, wt, out, workgroups=workgroups, best=scratch)
    assert parts == min(workgroups or ops.compute_units(x.device), (n // 16 + 1) // 2)
    vals = scratch[0][:rows * parts].view(rows, parts).cpu()
    idxs = scratch[1][:rows * parts].view(rows, parts).cpu()
    logits = out.cpu()
    for r in range(rows):
        top = logits[r].max()
        first = int((logits[r] == top).nonzero()[0])
        assert first == n // 5 + r, "the tie was meant to hold the row's largest logit"
        assert vals[r].max() == top
        assert int(idxs[r][vals[r] == top].min()) == first
        for p in range(parts):  # every part is a logit of the row at the index it names
            assert logits[r, idxs[r, p]] == vals[r, p]
    assert ops.head_gemm(x, wt, out) == 0


@pytest.mark.parametrize("stage_one", ["own", "given"])
def test_sampling_and_handing_on_in_one_kernel_equals_the_two(stage_one):
    """`sample_and_advance` against `sample` followed by `decode_advance`: greedy and seeded rows,
    a padding row without keys, two groups of layers, with the first stage of the argmax done by
    its own kernel or given as parts (here: the best of every seven logits)."""
    from dli_amd.kernels import ops

    rows, vocab, ps, width = 6, 1000, 8, 5
    g = torch.Generator().manual_seed(5)
    logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
    temperature = torch.tensor([0.0, 0.8, 1.0, 0.0, 1.3, 0.7]).cuda()
    top_k = torch.tensor([-1, 20, -1, 1, 50, -1], dtype=torch.int32).cuda()
    top_p = torch.tensor([1.0, 1.0, 0.9, 1.0, 0.8, 1.0]).cuda()
    seeds = torch.arange(11, 11 + rows, dtype=torch.int64).cuda()

    def state():
        tables = [torch.randint(0, 40, (rows, width), generator=torch.Generator().manual_seed(9 + i), dtype=torch.int32).cuda()
                  for i in range(2)]
        return dict(counters=torch.tensor([0, 3, 7, 1, 2, 4], dtype=torch.int64).cuda(),
                    token_ids=torch.full((rows,), 5, dtype=torch.int32).cuda(),
                    positions=torch.tensor([6, 7, 15, 22, 31, 0], dtype=torch.int32).cuda(),
                    kv_len=torch.tensor([7, 8, 16, 23, 32, 0], dtype=torch.int32).cuda(),  # the last row is padding
                    slots=[torch.full((rows,), -1, dtype=torch.int32).cuda() for _ in range(2)], tables=tables,
                    tokens_out=torch.full((rows,), -3, dtype=torch.int32).cuda())

    for advance in (True, False):
        a, b = state(), state()
        out_a = torch.empty(rows, dtype=torch.int32, device="cuda")
        ops.sample(logits, temperature, top_k, top_p, seeds, a["counters"], out_a)
        ops.decode_advance(out_a, a["tokens_out"], a["token_ids"], a["positions"], a["kv_len"], a["counters"],
                           a["slots"], a["tables"], ps, advance)
        out_b = torch.empty(rows, dtype=torch.int32, device="cuda")
        scratch = ops.sample_scratch(rows, logits.device)
        parts = 0
        if stage_one == "given":
            parts = 143
            vals = torch.full((rows, parts), float("-inf"), device="cuda")
            idxs = torch.full((rows, parts), 2 ** 31 - 1, dtype=torch.int32, device="cuda")
            for p in range(parts):  # parts of seven logits each; the last holds the six that are left
                lo, hi = 7 * p, min(vocab, 7 * p + 7)
                v, i = logits[:, lo:hi].max(dim=1)
                vals[:, p], idxs[:, p] = v, (i + lo).int()
            scratch[0][:rows * parts] = vals.reshape(-1)
            scratch[1][:rows * parts] = idxs.reshape(-1)
        ops.sample_and_advance(logits, temperature, top_k, top_p, seeds, b["counters"], out_b, scratch, parts,
                               b["tokens_out"], b["token_ids"], b["positions"], b["kv_len"], b["slots"], b["tables"],
                               ps, advance)
        assert torch.equal(out_a, out_b)
        for key in ("counters", "token_ids", "positions", "kv_len", "tokens_out"):
            assert torch.equal(a[key], b[key]), (key, advance)
        for sa, sb in zip(a["slots"], b["slots"]):
            assert torch.equal(sa, sb)
        assert (a["kv_len"][-1] == 0) and (a["slots"][0][-1] == -1)  # the padding row was left alone
        if advance:
            assert torch.equal(a["positions"][:5].cpu(), torch.tensor([7, 8, 16, 23, 32], dtype=torch.int32))
