"""Choice of attention kernel for a step.

The true 32-bit path, and shapes that the matrix-core kernels do not take, run the vector-unit
kernel over all entries. The bfloat16 path sends entries that bring one token to the split-key
decode kernel and portions to the tiled prefill kernel.
"""

from __future__ import annotations

from typing import Any, Callable, Optional

import numpy as np
import torch

from ..kernels import ops

# From decode steps at batch 1 to 64: two workgroups per compute unit, and at 4K keys at most 16
# runs, were ahead of more of either (the partial results cost a merge that grows with them); a
# request with 32K keys did better with 64 runs than with 16, so the limit grows with the keys.
# Runs of at least 256 keys: with 128, steps at contexts of 512 to 2,048 keys were 0.5 to 2% slower
# at the 1B and 3B sizes and 6% at four kv heads (8 requests of 2,048 keys: 16 runs of 128 keys
# against 8 of 256); with 512 they were 1 to 3% slower again.
WORKGROUPS_PER_UNIT = 2
MIN_KEYS_PER_SPLIT = 256
FEW_SPLITS = 16          # the limit up to 8K keys
KEYS_PER_EXTRA_SPLIT = 512
MAX_SPLITS = 64


def choose_splits(requests: int, kv_head_tiles: int, max_keys: int, units: int = 256) -> int:
    """How many runs to cut each request's keys into for the decode kernel: enough workgroups
    to give every compute unit two workgroups, never runs under 256 keys (reference's rule of the
    same kind: src/dli/model/paged_attention.py:63-74). ``units``: the device's compute units."""
    programs = max(1, requests * kv_head_tiles)
    want = -(-WORKGROUPS_PER_UNIT * units // programs)
    most = max(1, max_keys // MIN_KEYS_PER_SPLIT)
    limit = min(MAX_SPLITS, max(FEW_SPLITS, max_keys // KEYS_PER_EXTRA_SPLIT))
    return max(1, min(want, most, limit))


def planned_splits(requests: int, kv_head_tiles: int, max_keys: int, units: int = 256) -> int:
    """:func:`choose_splits` rounded up to a power of two: the coarse form of the rule, for steps
    that are recorded once and replayed for a range of lengths (each distinct answer is a
    recording of its own)."""
    splits, coarse = choose_splits(requests, kv_head_tiles, max_keys, units), 1
    while coarse < splits:
        coarse *= 2
    return coarse


# A launch of fewer workgroups than this per compute unit is as long as its longest workgroup, and
# cutting the keys of its longest tiles into runs, each a workgroup, shortens that (one prompt of
# 2,048 tokens at the 1B sizes: 43 -> 33 us a layer); with more, the workgroups queue anyway and
# the cut only costs its merge (3,072 tokens: 62 -> 69 us with room for four a unit). A run is not
# shorter than MIN_RUN_TILES tiles of 32 keys, and a tile has at most MAX_RUNS runs (the kernel's
# limit is asked at the first use).
CUT_BELOW_WORKGROUPS_PER_UNIT = 3
MIN_RUN_TILES = 8
MAX_RUNS = 8
LONE_TILE_COST = 1.5   # a tile of a workgroup alone on its SIMDs, in tiles of a busy compute unit


def runs_of_tiles(key_tiles: np.ndarray, workgroups_per_tile: int, units: int, most: int = MAX_RUNS) -> np.ndarray:
    """Into how many runs each tile of a launch has its keys cut (1: whole; ``key_tiles``: the
    number of 32-key tiles that each query tile walks). While the launch stays under three
    workgroups a compute unit, and the longest workgroup is still what the launch waits for (it
    takes longer than the units' work in all), the tile with the longest run gets one more, as long
    as its runs stay long enough; nothing is cut where that does not make the longest workgroup at
    least 15% shorter (tiles of much the same length and no room for all of them: a large portion on top of
    a long context)."""
    import heapq

    runs = np.ones(key_tiles.size, np.int64)
    spare = CUT_BELOW_WORKGROUPS_PER_UNIT * units // max(1, workgroups_per_tile) - key_tiles.size
    if spare <= 0 or key_tiles.size == 0:
        return runs
    share = lambda i: -(-int(key_tiles[i]) // int(runs[i]))   # the tile's longest run
    heap = [(-share(i), i) for i in range(key_tiles.size)]
    heapq.heapify(heap)
    # What a compute unit has to do in all, in tiles of 32 keys of one workgroup. Under a causal
    # mask from the prompt's start, the short tiles' workgroups leave early and the longest runs end
    # alone on their SIMDs, where a tile takes about one and a half times what a full unit needs
    # per tile: cutting stops when the longest run is no longer what the launch waits for. Tiles of
    # much the same length (a portion on top of a long context) all live to the end, and more runs
    # pay until the units are full (512 tokens on 8,192 keys: 155 us whole, 66 with four runs
    # a tile, 57 with six; one prompt of 2,048 tokens: 31.6 us with 21 tiles cut, 33.0 with 32).
    per_unit = float(key_tiles.sum()) * workgroups_per_tile / units
    lone_cost = LONE_TILE_COST if float(key_tiles.mean()) < 0.75 * float(key_tiles.max()) else 2 * LONE_TILE_COST
    while spare > 0:
        longest_run, i = heapq.heappop(heap)
        if -longest_run * lone_cost <= per_unit:
            break   # the launch is as long as its work by now, not as its longest workgroup
        if runs[i] >= most or int(key_tiles[i]) // (int(runs[i]) + 1) < MIN_RUN_TILES:
            break   # the longest workgroup cannot get shorter
        runs[i] += 1
        spare -= 1
        heapq.heappush(heap, (-share(i), i))
    longest = int(key_tiles.max())
    if max(share(i) for i in range(key_tiles.size)) * 20 > longest * 17:
        runs[:] = 1
    return runs


def round_about(order: np.ndarray, per_round: int) -> np.ndarray:
    """``order`` with every second run of ``per_round`` entries turned round."""
    order = order.copy()
    for r0 in range(per_round, order.size, 2 * per_round):
        order[r0:r0 + per_round] = order[r0:r0 + per_round][::-1].copy()
    return order


class PrefillTiles:
    """The tile list of a step's portions for :func:`ops.attention_prefill`, with what the kernel
    needs for the tiles whose keys are cut (``cut`` None: none are)."""

    def __init__(self, entry: torch.Tensor, q0: torch.Tensor, cut: Optional[torch.Tensor] = None, cut_tiles: int = 0,
                 cut_room: int = 0, cut_buf: Optional[torch.Tensor] = None,
                 cut_count: Optional[torch.Tensor] = None) -> None:
        self.entry, self.q0, self.cut, self.cut_tiles, self.cut_room = entry, q0, cut, cut_tiles, cut_room
        self.cut_buf, self.cut_count = cut_buf, cut_count

    @property
    def tiles(self) -> int:
        return int(self.entry.shape[0])


def list_tiles(q_len: np.ndarray, kv_len: np.ndarray, first_entry: int, rows: int, workgroups_per_tile: int,
               units: int, may_cut: bool) -> tuple[np.ndarray, np.ndarray, Optional[np.ndarray], int, int]:
    """The tiles of entries ``first_entry..`` (``q_len`` new tokens over ``kv_len`` keys each) in the
    order in which the prefill kernel wants them: ``(entry, first query, cut code or None, number of
    cut tiles, most runs of a tile)``. Those that see the most keys come first: workgroups start in the order of the list,
    and under a causal mask a tile's work grows with its place in the request; listed by place, the
    longest workgroups start last and the launch ends with a few of them alone on the device (a
    prompt of 8,192 tokens at the 1B sizes: 521 us a layer by place, 393 us longest first). Within
    the sorted list every second run of as many tiles as give every compute unit one workgroup (a
    tile becomes ``workgroups_per_tile`` workgroups, one per group of query heads) is turned round,
    so that a unit that got a long tile in one round gets a short one in the next. A cut tile is
    listed once per run, each time with its share of the keys."""
    ent, q0s = [], []
    for e in range(first_entry, q_len.size):
        for q0 in range(0, int(q_len[e]), rows):
            ent.append(e)
            q0s.append(q0)
    ent_a, q0_a = np.asarray(ent, np.int32), np.asarray(q0s, np.int32)
    if ent_a.size == 0:
        return ent_a, q0_a, None, 0, 0
    length = q_len[ent_a].astype(np.int64)
    keys = kv_len[ent_a].astype(np.int64) - length + np.minimum(q0_a + rows, length)
    key_tiles = -(-keys // 32)
    runs = runs_of_tiles(key_tiles, workgroups_per_tile, units) if may_cut else np.ones(ent_a.size, np.int64)
    per_round = max(1, units // max(1, workgroups_per_tile))
    cut = runs > 1
    n_cut = int(cut.sum())
    if n_cut == 0:
        order = round_about(np.argsort(-keys, kind="stable"), per_round)
        return ent_a[order], q0_a[order], None, 0, 0
    # the list's entries: a tile once per run, each with its share of the keys
    which = np.repeat(np.arange(ent_a.size), runs)
    run = np.concatenate([np.arange(r) for r in runs])
    place = np.cumsum(cut) - 1                       # the cut tiles numbered in list order
    code = np.where(cut[which], run | runs[which] << 4 | place[which] << 8, -1)
    share = -(-key_tiles[which] // runs[which])
    order = round_about(np.argsort(-share, kind="stable"), per_round)
    return ent_a[which][order], q0_a[which][order], code[order].astype(np.int32), n_cut, int(runs.max())


def prefill_tiles(ctx: Any, head_dim: int, q_heads: int, kv_heads: int, first_entry: int, device: torch.device,
                  window: int = 0) -> PrefillTiles:
    """The tile list of the step's portions for :func:`ops.attention_prefill` (made once per step
    and shape; the buffers of the cut tiles serve every layer of that shape in turn)."""
    rows = ops.attention_prefill_tile_rows(head_dim, q_heads, kv_heads)
    units = ops.compute_units(device)
    cut_floats = ops.attention_prefill_cut_floats(head_dim, q_heads, kv_heads)
    # a workgroup takes a tile for 4 * 32 / rows query heads where the kernel's waves share key
    # tiles (heads of 32 and more: the kernel that can also cut a tile's keys), else for one
    per_tile = q_heads * rows // 128 if cut_floats > 0 else q_heads
    may_cut = window == 0 and cut_floats > 0

    def make() -> PrefillTiles:
        q_len = (ctx.q_start_host[1:] - ctx.q_start_host[:-1]).astype(np.int64)
        ent, q0, code, n_cut, room = list_tiles(q_len, np.asarray(ctx.kv_len_host), first_entry, rows, per_tile,
                                                units, may_cut)
        if code is None:
            return PrefillTiles(*ctx.upload([ent, q0]))
        entry_t, q0_t, code_t = ctx.upload([ent, q0, code])
        return PrefillTiles(entry_t, q0_t, code_t, n_cut, room,
                            torch.empty(n_cut * room * cut_floats, device=device, dtype=torch.float32),
                            torch.zeros(n_cut * q_heads, device=device, dtype=torch.int32))

    return ctx.step_lists(("prefill tiles", rows, per_tile, first_entry, may_cut), make)


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                    ctx: Any, grp: Any, q_heads: int, scale: float, window: int = 0,
                    arrival_counters: Optional[Callable[[int], Optional[torch.Tensor]]] = None,
                    planned: Optional[int] = None) -> None:
    """Attention of every row of the step over its request's pages, into ``out``.
    ``arrival_counters(n)``: the caller's ``n`` counters with which the decode kernel merges its
    runs of keys by itself (see ``ops.attention_decode``), or None. ``planned``: the number of
    runs that the mixer promised for this step when it was recorded (``Mixer.decode_plan``)."""
    if ctx.num_tokens == 0:
        return
    _, kv_heads, page_size, head_dim = k_pages.shape
    if not ops.attention_mfma_supports(head_dim, page_size, k_pages.dtype):
        rows = ops.attention_generic_tile_rows(head_dim)
        tile_entry, tile_q0 = ctx.q_tiles(rows)
        ops.attention_generic(q, k_pages, v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                              tile_entry, tile_q0, q_heads, scale, window)
        return
    nd = ctx.num_decode
    if nd > 0:
        splits, part_o, part_ml = _decode_splits(ctx, nd, q_heads, kv_heads, head_dim, q.device, planned)
        arrivals = None
        if arrival_counters is not None and 1 < splits <= ops.SELF_MERGING_SPLITS:
            arrivals = arrival_counters(nd * kv_heads * (-(-(q_heads // kv_heads) // 16)))
        ops.attention_decode(q[:nd], k_pages, v_pages, out[:nd], ctx.kv_len, grp.block_tables, q_heads,
                             scale, window, splits, part_o, part_ml, arrivals=arrivals)
    if ctx.num_entries > nd:
        t = prefill_tiles(ctx, head_dim, q_heads, kv_heads, nd, q.device, window)
        ops.attention_prefill(q, k_pages, v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables, t.entry, t.q0,
                              q_heads, scale, window, t.cut, t.cut_tiles, t.cut_room, t.cut_buf, t.cut_count)


def decode_attention_unmerged(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, ctx: Any, grp: Any,
                              q_heads: int, scale: float, window: int, wanted,
                              planned: Optional[int] = None) -> Any:
    """Attention of a step in which every row is one request's single token, without the kernel
    that merges the runs of keys: ``(splits, part_o, part_ml)`` for the product that merges while
    it loads (``ops.skinny_gemm_merged``), or None (nothing has run) where the step's keys are
    not split or ``wanted(splits)`` says that this product does not take them."""
    _, kv_heads, page_size, head_dim = k_pages.shape
    nd = ctx.num_decode
    if nd != ctx.num_tokens or not ops.attention_mfma_supports(head_dim, page_size, k_pages.dtype):
        return None
    splits, part_o, part_ml = _decode_splits(ctx, nd, q_heads, kv_heads, head_dim, q.device, planned)
    if splits < 2 or not wanted(splits):
        return None
    ops.attention_decode(q[:nd], k_pages, v_pages, None, ctx.kv_len, grp.block_tables, q_heads, scale, window,
                         splits, part_o, part_ml, merge=False)
    return splits, part_o, part_ml


def head_tiles(q_heads: int, kv_heads: int) -> int:
    """Workgroups that one request's token gives the decode kernel per run of keys: a workgroup
    takes up to 16 query heads of one kv head."""
    return kv_heads * -(-(q_heads // kv_heads) // 16)


def step_splits(ctx: Any, nd: int, q_heads: int, kv_heads: int, device: torch.device,
                planned: Optional[int] = None) -> int:
    """Runs of keys for the ``nd`` single-token rows of this step: what was planned when the step
    was recorded, else the rule applied to the step's own lengths."""
    return planned or choose_splits(nd, head_tiles(q_heads, kv_heads), ctx.max_decode_kv_len,
                                    ops.compute_units(device))


def _decode_splits(ctx: Any, nd: int, q_heads: int, kv_heads: int, head_dim: int, device: torch.device,
                   planned: Optional[int] = None):
    splits = step_splits(ctx, nd, q_heads, kv_heads, device, planned)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty(nd * q_heads * splits * head_dim, device=device, dtype=torch.float32)
        part_ml = torch.empty(nd * q_heads * splits * 2, device=device, dtype=torch.float32)
    return splits, part_o, part_ml
