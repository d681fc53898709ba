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


def test_rows_of_a_decode_graph():
    """Powers of two up to 32 rows, then multiples of 16: a product's cost grows with its row tiles."""
    from dli_amd.engine.decode_graph import _batch_bucket

    assert [_batch_bucket(n) for n in (1, 2, 3, 5, 9, 16, 17, 32)] == [1, 2, 4, 8, 16, 16, 32, 32]
    assert [_batch_bucket(n) for n in (33, 40, 48, 49, 64, 65)] == [48, 48, 48, 64, 64, 80]


def test_workgroup_shape_of_the_tile_kernel_from_sizes():
    """The rule read off timings at the 1B, 1.7B and 3B sizes (256 compute units): four k-waves on
    one tile where tiles are few or fill the units evenly with short rows, else on two tiles; a
    vocabulary with long rows does not split k."""
    from dli_amd.kernels.ops import skinny_gemm_shape

    tiled = lambda n, k: skinny_gemm_shape(n, k, tiled=True, units=256)
    assert tiled(2048, 2048) == 0 and tiled(3072, 2048) == 0       # o and q/k/v at the 1B sizes
    assert tiled(8192, 2048) == 0                                   # gate and up at the 1B sizes: 512 tiles
    assert tiled(5120, 3072) == 4 and tiled(8192, 3072) == 4       # q/k/v and gate/up at the 3B sizes
    assert tiled(6144, 2048) == 4                                   # q/k/v at the 1.7B sizes: 384 tiles
    assert tiled(128256, 3072) == 2 and tiled(128256, 2048) == 4   # vocabularies
    assert skinny_gemm_shape(2048, 8192) == 1 and skinny_gemm_shape(2048, 2048) == 0 and skinny_gemm_shape(128256, 2048) == 3


def test_pool_of_generate_from_its_requests():
    """Pages for the requests that can be live together, a page of look ahead each and the share
    that admission keeps back; never more than the memory holds."""
    from dli_amd.engine.generate import pages_for_requests

    assert pages_for_requests([], 16, 4, 100) == 1
    # 100 and 33 tokens in pages of 16: 7 + 1 and 3 + 1 pages; only the two longest are live together
    assert pages_for_requests([100, 33, 20], 16, 2, 10 ** 6) == 12 + 12 // 50 + 8
    assert pages_for_requests([100, 33, 20], 16, 8, 10 ** 6) == 15 + 15 // 50 + 8
    assert pages_for_requests([16] * 1000, 16, 256, 10 ** 6) == 512 + 10 + 8
    assert pages_for_requests([16] * 1000, 16, 256, 300) == 300          # what the memory holds
    assert pages_for_requests([1600, 16], 16, 256, 50) == 50


def test_a_call_records_graphs_where_it_decodes_long_enough():
    from dli_amd.engine.generate import GRAPHS_PAY_FROM, graphs_pay

    assert not graphs_pay([], 64)
    assert not graphs_pay([16, 256], 256)                      # 256 decode steps
    assert graphs_pay([16, GRAPHS_PAY_FROM], 256)
    assert graphs_pay([256] * 600, 256)                        # three rounds of 256 steps
    assert not graphs_pay([256] * 256, 256) and graphs_pay([256] * 257, 256)
