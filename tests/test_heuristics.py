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
    assert not graphs_pay([16, 64], 256)                       # 64 decode steps
    assert graphs_pay([16, GRAPHS_PAY_FROM], 256)
    assert graphs_pay([64] * 600, 256)                         # three rounds of 64 steps
    assert not graphs_pay([64] * 256, 256) and graphs_pay([64] * 257, 256)


def test_which_tiles_of_a_short_launch_have_their_keys_cut():
    """One prompt of 2,048 tokens at the 1B sizes (a tile of 32 queries is 8 workgroups, 256 compute
    units): the 21 longest tiles are cut in two, after which no workgroup is longer than two
    thirds of a unit's work; from 3,072 tokens on nothing is cut; shorter launches cut into more
    runs, never runs of fewer than eight key tiles, never more workgroups than three a unit, and
    nothing where the longest workgroup would stay about as long."""
    import numpy as np

    from dli_amd.parts.attention_kernels import MAX_RUNS, MIN_RUN_TILES, runs_of_tiles

    runs = runs_of_tiles(np.arange(1, 65), 8, 256)       # the launch's work: 65 tiles a unit; runs of up to 43 may stay
    assert runs[:43].tolist() == [1] * 43 and runs[43:].tolist() == [2] * 21
    assert runs_of_tiles(np.arange(1, 97), 8, 256).tolist() == [1] * 96
    runs = runs_of_tiles(np.arange(1, 81), 8, 256)           # room for 16 more entries, 13 used
    assert runs.sum() == 93 and runs[67:].tolist() == [2] * 13
    for tokens in (512, 640, 1024, 1536):
        key_tiles = np.arange(1, tokens // 32 + 1)
        runs = runs_of_tiles(key_tiles, 8, 256)
        assert runs.sum() * 8 <= 3 * 256 and runs.max() <= MAX_RUNS
        assert all(r == 1 or n // r >= MIN_RUN_TILES for n, r in zip(key_tiles.tolist(), runs.tolist()))
        longest = max(-(-n // r) for n, r in zip(key_tiles.tolist(), runs.tolist()))
        assert longest <= 0.85 * key_tiles.max() or runs.max() == 1
    assert runs_of_tiles(np.arange(1, 33), 8, 256).max() >= 3    # 1,024 tokens: more than two runs for the longest
    assert runs_of_tiles(np.arange(1, 9), 8, 256).max() == 1 and runs_of_tiles(np.zeros(0, np.int64), 8, 256).size == 0
    # a portion of 2,048 tokens on top of 14K cached keys: 64 tiles of 450 to 512 key tiles, room for 32 more
    # workgroups a head group, after which the longest whole tile would still walk 480: nothing is cut
    assert runs_of_tiles(np.arange(449, 513), 8, 256).max() == 1
    # 512 tokens on top of 8K keys: 16 tiles of much the same length, room for 80 more entries: six runs each
    assert runs_of_tiles(np.arange(257, 273), 8, 256).tolist() == [6] * 16
    # one prompt of 1,536 tokens: two runs for the upper half, as at 2,048
    assert runs_of_tiles(np.arange(1, 49), 8, 256).tolist() == [1] * 24 + [2] * 24


def test_the_tile_list_of_a_step_lists_every_tile_once_or_all_of_its_runs():
    """Random steps: every tile of every portion is in the list, whole or once per run with the
    same place and number of runs; places count the cut tiles from 0; the launch stays under three
    workgroups a compute unit where anything is cut."""
    import random

    import numpy as np

    from dli_amd.parts.attention_kernels import list_tiles

    rng = random.Random(3)
    for trial in range(200):
        n = rng.randrange(1, 6)
        first = rng.randrange(0, n)
        q_len = np.asarray([1] * first + [rng.randrange(2, 3000) for _ in range(n - first)], np.int64)
        kv_len = q_len + np.asarray([rng.randrange(0, 500) for _ in range(n)], np.int64)
        rows, per_tile, units = rng.choice([(32, 8), (128, 24), (64, 4), (128, 9)]) + (rng.choice([64, 256, 304]),)
        may_cut = rng.random() < 0.8
        ent, q0, code, n_cut, room = list_tiles(q_len, kv_len, first, rows, per_tile, units, may_cut)
        want = {(e, t) for e in range(first, n) for t in range(0, int(q_len[e]), rows)}
        if code is None:
            assert n_cut == 0 and room == 0 and sorted(zip(ent.tolist(), q0.tolist())) == sorted(want)
            continue
        assert may_cut and n_cut > 0
        whole = [(e, t) for e, t, c in zip(ent.tolist(), q0.tolist(), code.tolist()) if c < 0]
        runs = {}
        for e, t, c in zip(ent.tolist(), q0.tolist(), code.tolist()):
            if c >= 0:
                runs.setdefault((e, t), []).append((c & 15, (c >> 4) & 15, c >> 8))
        assert len(whole) == len(set(whole)) and set(whole) | set(runs) == want and not set(whole) & set(runs)
        for r in runs.values():
            n, place = r[0][1], r[0][2]
            assert 2 <= n <= room and sorted(r) == [(i, n, place) for i in range(n)]
        assert max(r[0][1] for r in runs.values()) == room
        assert sorted(r[0][2] for r in runs.values()) == list(range(n_cut))
        assert len(ent) * per_tile <= 3 * units


def test_which_recorded_shape_stands_in_for_one_that_is_not_recorded():
    """Fewest rows first, then the same plans, then the narrowest table; never fewer rows than
    requests, more than four times the shape's own rows, a narrower table, another number of
    steps or another kind of output."""
    from dli_amd.engine import decode_graph
    from dli_amd.engine.decode_graph import DecodeGraphs

    graphs = DecodeGraphs.__new__(DecodeGraphs)   # the choice reads the recorded shapes only
    plans_a, plans_b = (2, 2), (4, 4)

    def choice(key, requests, recorded):
        graphs.captured = {k: f"graph of {k}" for k in recorded}
        got = graphs._stand_in(key, requests)
        return None if got is None else got[0]

    want = (4, plans_a, 64, True, 1)
    assert choice(want, 3, []) is None
    assert choice(want, 3, [(8, plans_b, 64, True, 1), (16, plans_a, 64, True, 1)]) == (8, plans_b, 64, True, 1)
    assert choice(want, 3, [(8, plans_b, 64, True, 1), (8, plans_a, 128, True, 1)]) == (8, plans_a, 128, True, 1)
    assert choice(want, 3, [(8, plans_a, 256, True, 1), (8, plans_a, 128, True, 1)]) == (8, plans_a, 128, True, 1)
    assert choice(want, 3, [(4, plans_b, 128, True, 1)]) == (4, plans_b, 128, True, 1)   # its own rows, other plans
    assert choice(want, 3, [(2, plans_a, 64, True, 1)]) is None                          # too few rows
    assert choice(want, 3, [(8, plans_a, 32, True, 1)]) is None                          # too narrow a table
    assert choice(want, 3, [(8, plans_a, 64, True, 2), (8, plans_a, 64, False, 1)]) is None
    assert choice(want, 3, [(4 * decode_graph.STAND_IN_ROWS, plans_a, 64, True, 1)]) is not None
    assert choice(want, 3, [(4 * decode_graph.STAND_IN_ROWS + 16, plans_a, 64, True, 1)]) is None
