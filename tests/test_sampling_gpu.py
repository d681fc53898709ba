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
