"""The block-table rows that a captured decode step keeps between replays (engine/table_rows.py).

Every case compares the patched rows with rows rebuilt from scratch, which is what the reference
does at every replay (src/dli/engine/cuda_graph.py:218-224)."""

from __future__ import annotations

import random

import numpy as np
import pytest

from dli_amd.cache import CacheManager, GroupSpec, NoFreePagesError
from dli_amd.engine.batch import StepEntry
from dli_amd.engine.table_rows import TableRows

PS = 4


def rebuilt(mgr, entries, group, batch, width):
    want = np.zeros((batch, width), np.int32)
    for i, e in enumerate(entries):
        table = list(mgr.table_ref(e.seq_id, group))[:width]
        want[i, :len(table)] = np.maximum(table, 0)
    return want


def assert_rows(mgr, entries, group, flat, batch, width):
    got = flat.reshape(batch, width)
    want = rebuilt(mgr, entries, group, batch, width)
    for i, e in enumerate(entries):
        read = -(-(e.start + 1) // mgr.page_size)  # pages that this step's keys lie in
        assert list(got[i, :read]) == list(want[i, :read]), (i, e.seq_id, got[i], want[i])
        held = min(len(mgr.table_ref(e.seq_id, group)), width)
        assert list(got[i, :held]) == list(want[i, :held]), (i, e.seq_id, got[i], want[i])


def decode_entry(mgr, seq_id):
    """The entry that decodes the request's last token (all tokens before it computed)."""
    n = mgr.num_tokens(seq_id)
    mgr.mark_computed(seq_id, n - 1)
    return StepEntry(seq_id, (1,), n - 1, (0,))


def test_same_id_allocated_again_gets_its_row_rewritten():
    # The schedule of a preemption by recompute: B sits in row 1, loses its pages, somebody else takes
    # them, B is admitted again under the same id with other pages and returns to row 1.
    mgr = CacheManager(num_pages=15, page_size=PS, enable_prefix_caching=False, watermark=0.0)
    rows, flat = TableRows(2, 8, 1), np.zeros(2 * 8, np.int32)
    mgr.allocate("A", list(range(9)))
    mgr.allocate("B", list(range(100, 118)))
    before = mgr.block_table("B")
    entries = [decode_entry(mgr, "A"), decode_entry(mgr, "B")]
    rows.fill(mgr, entries, 0, flat, 40)
    assert_rows(mgr, entries, 0, flat, 2, 8)
    mgr.free("B")
    mgr.allocate("C", list(range(200, 228)))          # the pool is used by others meanwhile
    mgr.allocate("B", list(range(100, 119)))          # prompt + one output, as after a preemption
    after = mgr.block_table("B")
    assert before[:4] != after[:4]                     # the pages that a patch of the row's end would keep
    entries = [decode_entry(mgr, "A"), decode_entry(mgr, "B")]
    slots = rows.fill(mgr, entries, 0, flat, 40)
    assert_rows(mgr, entries, 0, flat, 2, 8)
    assert list(flat.reshape(2, 8)[1, :len(after)]) == list(after)
    assert slots[1] == after[18 // PS] * PS + 18 % PS
    mgr.check_invariants()


def test_row_taken_over_by_another_request_and_back():
    mgr = CacheManager(num_pages=40, page_size=PS, enable_prefix_caching=False, watermark=0.0)
    rows, flat = TableRows(1, 8, 1), np.zeros(8, np.int32)
    mgr.allocate("A", list(range(14)))
    mgr.allocate("B", list(range(50, 60)))
    for name in ("A", "B", "A", "A", "B"):
        e = [decode_entry(mgr, name)]
        rows.fill(mgr, e, 0, flat, 40)
        assert_rows(mgr, e, 0, flat, 1, 8)
        mgr.mark_computed(name, mgr.num_tokens(name))
        mgr.append_slots(name, [7])


def test_table_longer_than_the_row_is_cut_and_leaves_the_neighbour_alone():
    # Pages reserved ahead of the keys that the step reads: the table is longer than the row.
    mgr = CacheManager(num_pages=64, page_size=PS, enable_prefix_caching=False, watermark=0.0)
    width = 4
    rows, flat = TableRows(2, width, 1), np.zeros(2 * width, np.int32)
    mgr.allocate("A", list(range(4 * PS)))            # 16 tokens: four pages, as wide as the row
    mgr.allocate("B", list(range(100, 106)))
    entries = [decode_entry(mgr, "A"), decode_entry(mgr, "B")]
    rows.fill(mgr, entries, 0, flat, 64)               # both rows known now: the patching branch comes next
    b_row = list(flat.reshape(2, width)[1])
    mgr.reserve_ahead("A", 7)
    assert len(mgr.table_ref("A")) > width
    entries = [StepEntry("A", (1,), 15, (0,)), StepEntry("B", (1,), 5, (0,))]
    rows.fill(mgr, entries, 0, flat, 64)
    assert list(flat.reshape(2, width)[1]) == b_row
    assert list(flat.reshape(2, width)[0]) == list(mgr.table_ref("A")[:width])
    fresh = TableRows(2, width, 1)                     # and the branch that writes a whole row
    flat2 = np.zeros(2 * width, np.int32)
    fresh.fill(mgr, entries, 0, flat2, 64)
    assert list(flat2) == list(flat)


def test_position_outside_the_row_is_refused():
    mgr = CacheManager(num_pages=64, page_size=PS, enable_prefix_caching=False, watermark=0.0)
    mgr.allocate("A", list(range(4 * PS + 2)))
    rows, flat = TableRows(1, 4, 1), np.zeros(4, np.int32)
    with pytest.raises(ValueError, match="outside its block table row"):
        rows.fill(mgr, [decode_entry(mgr, "A")], 0, flat, 64)


def test_copy_on_write_of_the_page_being_written_is_seen():
    mgr = CacheManager(num_pages=40, page_size=PS, enable_prefix_caching=False, watermark=0.0)
    rows, flat = TableRows(1, 8, 1), np.zeros(8, np.int32)
    mgr.allocate("A", list(range(10)))
    e = [decode_entry(mgr, "A")]
    rows.fill(mgr, e, 0, flat, 40)
    mgr.mark_computed("A", 10)
    mgr.fork("A", "child")
    ops = mgr.append_slots("A", [3])                   # page 2 is shared and partly filled: copied
    assert len(ops) == 1 and mgr.block_table("A")[2] == ops[0].dst
    e = [decode_entry(mgr, "A")]
    rows.fill(mgr, e, 0, flat, 40)
    assert_rows(mgr, e, 0, flat, 1, 8)


def test_window_group_rows_are_rewritten_whole():
    mgr = CacheManager([GroupSpec("full"), GroupSpec("window", 6)], num_pages=40, page_size=PS,
                       enable_prefix_caching=False, watermark=0.0)
    rows = TableRows(1, 8, 2)
    flats = [np.zeros(8, np.int32), np.zeros(8, np.int32)]
    mgr.allocate("A", list(range(5)))
    for _ in range(20):
        e = [decode_entry(mgr, "A")]
        for g in range(2):
            rows.fill(mgr, e, g, flats[g], 40)
            assert_rows(mgr, e, g, flats[g], 1, 8)
            assert flats[g].min() >= 0
        mgr.mark_computed("A", mgr.num_tokens("A"))
        mgr.append_slots("A", [9])
    assert mgr.stats().window_pages_released > 0


@pytest.mark.parametrize("seed", range(12))
def test_random_schedules_leave_rows_equal_to_rebuilt_ones(seed):
    """Requests come, grow (also several tokens at once, with pages reserved ahead), fork and write
    into a shared page, lose their pages and come back under the same id, change rows and sit out
    steps, across two captured shapes; after every fill each row equals the manager's table."""
    rng = random.Random(seed)
    mgr = CacheManager(num_pages=48, page_size=PS, enable_prefix_caching=bool(seed % 2), watermark=0.0)
    width = 8
    shapes = {1: (TableRows(1, width, 1), np.zeros(width, np.int32)),
              2: (TableRows(2, width, 1), np.zeros(2 * width, np.int32)),
              4: (TableRows(4, width, 1), np.zeros(4 * width, np.int32))}
    live: dict[str, list[int]] = {}
    names = ["r0", "r1", "r2", "r3", "r4"]
    fills = 0
    for _ in range(300):
        op = rng.random()
        if op < 0.15 and len(live) < 4:
            name = rng.choice([n for n in names if n not in live])
            toks = [rng.randrange(50) for _ in range(rng.randint(2, 12))]
            try:
                mgr.allocate(name, toks)
            except NoFreePagesError:
                continue
            live[name] = toks
            mgr.mark_computed(name, len(toks) - 1)
        elif op < 0.25 and live:
            name = rng.choice(sorted(live))
            toks = live[name]
            mgr.free(name)                              # preempted ...
            if rng.random() < 0.7:
                try:
                    mgr.allocate(name, toks)            # ... and admitted again under the same id
                    mgr.mark_computed(name, len(toks) - 1)
                except NoFreePagesError:
                    del live[name]
            else:
                del live[name]
        elif op < 0.32 and live and len(live) < 4:
            parent = rng.choice(sorted(live))
            child = rng.choice([n for n in names if n not in live])
            mgr.fork(parent, child)
            live[child] = list(live[parent])
        elif live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            chosen = [c for c in chosen if (mgr.num_tokens(c) + 4) <= width * PS]
            if not chosen:
                name = rng.choice(sorted(live))
                mgr.free(name)
                del live[name]
                continue
            batch = 1 if len(chosen) == 1 else 2 if len(chosen) == 2 else 4
            rows, flat = shapes[batch]
            steps = rng.choice([1, 1, 3])
            try:
                for c in chosen:
                    mgr.reserve_ahead(c, steps - 1)
            except NoFreePagesError:
                steps = 1
            entries = [StepEntry(c, (live[c][-1],), mgr.num_tokens(c) - 1, (0,)) for c in chosen]
            rows.fill(mgr, entries, 0, flat, 48)
            fills += 1
            assert_rows(mgr, entries, 0, flat, batch, width)
            for c in chosen:
                try:
                    for j in range(steps):
                        mgr.mark_computed(c, mgr.num_tokens(c))
                        tok = rng.randrange(50)
                        mgr.append_slots(c, [tok])
                        live[c].append(tok)
                        mgr.mark_computed(c, mgr.num_tokens(c) - 1)
                except NoFreePagesError:
                    mgr.free(c)
                    del live[c]
        mgr.check_invariants()
    assert fills > 50
