"""Choices that the engine makes from sizes alone (no GPU): how many runs the decode attention
cuts a request's keys into (the reference's rule of the same kind and its test vectors:
src/dli/model/paged_attention.py:63-74, tests/unit/model/test_paged_attention_gpu.py:114-119)."""

from __future__ import annotations

from dli_amd.parts.attention_kernels import FEW_SPLITS, MAX_SPLITS, MIN_KEYS_PER_SPLIT, choose_splits


def test_enough_programs_already_means_one_run():
    assert choose_splits(requests=64, kv_head_tiles=8, max_keys=4096) == 1
    assert choose_splits(requests=512, kv_head_tiles=1, max_keys=100000) == 1


def test_one_request_with_a_long_context_is_cut():
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=4096) > 1
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=4096) == FEW_SPLITS
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=16384) == 32   # the limit grows with the keys
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=1 << 20) == MAX_SPLITS


def test_short_contexts_are_not_cut_below_the_least_run():
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=64) == 1
    assert choose_splits(requests=1, kv_head_tiles=8, max_keys=2 * MIN_KEYS_PER_SPLIT + 5) == 2


def test_runs_shrink_as_the_batch_grows():
    got = [choose_splits(requests=b, kv_head_tiles=8, max_keys=4096) for b in (1, 2, 4, 8, 16, 32, 64)]
    assert got == sorted(got, reverse=True) and got[0] > got[-1] == 1
    assert all(1 <= s <= MAX_SPLITS for s in got)
