"""Block-table rows that persist between replays of a captured decode step.

A captured graph reads each request's block table from a fixed host-staged array, one row of
``width`` entries per batch row. Rewriting every row at every replay costs more host time than the
step has at large batches and long contexts, so a row is patched instead, but only where that is
provably the same as rewriting it:

* a row may be patched only if it last held *the same allocation*: the very list object that the
  cache manager keeps for the request (an id is not enough, since a request that was preempted and
  admitted again, or another request under a re-used id, has other pages);
* of that allocation only the entries before the page that was being written when the row was last
  filled are trusted. Later entries may have been appended, or swapped by a copy-on-write (which
  only ever replaces the page that the request's next token goes into), so they are written again;
* groups that give pages back while the request runs (windows) are rewritten whole.

A table may be longer than the row (pages reserved ahead of the keys that the step reads): the
entries beyond ``width`` are never read and are left out.

The reference rebuilds every padded row at each replay (src/dli/engine/cuda_graph.py:218-224);
this module keeps that result and skips the work.
"""

from __future__ import annotations

from typing import Optional, Sequence

import numpy as np


class TableRows:
    """What the rows of one captured graph's block tables hold, per group."""

    def __init__(self, batch: int, width: int, num_groups: int) -> None:
        self.batch, self.width, self.num_groups = batch, width, num_groups
        # per row and group: (the manager's page list, entries of it that can no longer change)
        self._held: list[list[Optional[tuple[list, int]]]] = [[None] * num_groups for _ in range(batch)]

    def forget(self, row: int) -> None:
        self._held[row] = [None] * self.num_groups

    def fill(self, manager, entries: Sequence, group: int, flat: np.ndarray, num_pages: int) -> list[int]:
        """Bring rows ``0..len(entries)`` of ``flat`` (``[batch * width]`` page ids of ``group``)
        up to date with the manager's tables; returns each entry's cache slot for its position
        ``start``. Rows beyond the entries are forgotten."""
        ps, width = manager.page_size, self.width
        whole_only = manager.groups[group].kind != "full"
        slots: list[int] = []
        patch_at: list[int] = []
        patch_page: list[int] = []
        for i, e in enumerate(entries):
            table = manager.table_ref(e.seq_id, group)
            at = e.start // ps
            if at >= width or at >= len(table):
                raise ValueError(f"request {e.seq_id!r}: position {e.start} lies outside its block table row")
            page = table[at]
            if not 0 <= page < num_pages:
                raise ValueError("a block table names a page outside the pool")
            slots.append(page * ps + e.start % ps)
            count = min(len(table), width)
            held = self._held[i][group]
            if held is not None and held[0] is table and not whole_only:
                for k in range(min(held[1], count), count):
                    patch_at.append(i * width + k)
                    patch_page.append(table[k])
            else:
                row = flat[i * width:(i + 1) * width]
                row[:count] = table[:count]
                if whole_only:
                    np.maximum(row, 0, out=row)  # pages that the window has passed are never read
            # entries before the page being written now stay as they are while the allocation lives
            self._held[i][group] = (table, min(at, count))
        if patch_at:
            flat[patch_at] = patch_page
        for i in range(len(entries), self.batch):
            self._held[i][group] = None
        return slots
