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
WORKGROUPS_PER_UNIT = 2
MIN_KEYS_PER_SPLIT = 128
FEW_SPLITS = 16          # the limit up to 8K keys
KEYS_PER_EXTRA_SPLIT = 512
MAX_SPLITS = 64


def choose_splits(requests: int, kv_head_tiles: int, max_keys: int, units: int = 256) -> int:
    """How many runs to cut each request's keys into for the decode kernel: enough workgroups
    to give every compute unit two workgroups, never runs under 128 keys (reference's rule of the
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
# cutting the keys of its longest tiles into two runs, each a workgroup, shortens that (one prompt
# of 2,048 tokens at the 1B sizes: 43 -> 32 us a layer before the runs are added up); with more, the
# workgroups queue anyway and the cut only costs its merge. A run is not shorter than MIN_RUN_TILES
# tiles of 32 keys.
CUT_BELOW_WORKGROUPS_PER_UNIT = 3
MIN_RUN_TILES = 8


def tiles_to_cut(key_tiles: np.ndarray, workgroups_per_tile: int, units: int) -> np.ndarray:
    """Which tiles of a launch have their keys cut into two runs (a mask over ``key_tiles``, the
    number of 32-key tiles that each query tile walks): the longest ones, as many as keep the
    launch under three workgroups a compute unit, and only those longer than half the longest
    (cutting a shorter one would not shorten the longest workgroup) and long enough for two runs."""
    cut = np.zeros(key_tiles.size, bool)
    spare = CUT_BELOW_WORKGROUPS_PER_UNIT * units // max(1, workgroups_per_tile) - key_tiles.size
    if spare <= 0 or key_tiles.size == 0:
        return cut
    longest = int(key_tiles.max())
    wanted = np.flatnonzero((key_tiles > -(-longest // 2)) & (key_tiles >= 2 * MIN_RUN_TILES))
    wanted = wanted[np.argsort(-key_tiles[wanted], kind="stable")][:spare]
    cut[wanted] = True
    return cut


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
                 cut_buf: Optional[torch.Tensor] = None, cut_count: Optional[torch.Tensor] = None) -> None:
        self.entry, self.q0, self.cut, self.cut_tiles = entry, q0, cut, cut_tiles
        self.cut_buf, self.cut_count = cut_buf, cut_count

    @property
    def tiles(self) -> int:
        return int(self.entry.shape[0])


def list_tiles(q_len: np.ndarray, kv_len: np.ndarray, first_entry: int, rows: int, workgroups_per_tile: int,
               units: int, may_cut: bool) -> tuple[np.ndarray, np.ndarray, Optional[np.ndarray], int]:
    """The tiles of entries ``first_entry..`` (``q_len`` new tokens over ``kv_len`` keys each) in the
    order in which the prefill kernel wants them: ``(entry, first query, cut code or None, number of
    cut tiles)``. Those that see the most keys come first: workgroups start in the order of the list,
    and under a causal mask a tile's work grows with its place in the request; listed by place, the
    longest workgroups start last and the launch ends with a few of them alone on the device (a
    prompt of 8,192 tokens at the 1B sizes: 521 us a layer by place, 393 us longest first). Within
    the sorted list every second run of as many tiles as give every compute unit one workgroup (a
    tile becomes ``workgroups_per_tile`` workgroups, one per group of query heads) is turned round,
    so that a unit that got a long tile in one round gets a short one in the next. A cut tile is
    listed twice, each time with half its keys."""
    ent, q0s = [], []
    for e in range(first_entry, q_len.size):
        for q0 in range(0, int(q_len[e]), rows):
            ent.append(e)
            q0s.append(q0)
    ent_a, q0_a = np.asarray(ent, np.int32), np.asarray(q0s, np.int32)
    if ent_a.size == 0:
        return ent_a, q0_a, None, 0
    length = q_len[ent_a].astype(np.int64)
    keys = kv_len[ent_a].astype(np.int64) - length + np.minimum(q0_a + rows, length)
    key_tiles = -(-keys // 32)
    cut = tiles_to_cut(key_tiles, workgroups_per_tile, units) if may_cut else np.zeros(ent_a.size, bool)
    n_cut = int(cut.sum())
    per_round = max(1, units // max(1, workgroups_per_tile))
    if n_cut == 0:
        order = round_about(np.argsort(-keys, kind="stable"), per_round)
        return ent_a[order], q0_a[order], None, 0
    # the list's entries: whole tiles once, cut tiles twice (run 0 and run 1), each with its share of the keys
    which = np.concatenate([np.flatnonzero(~cut), np.flatnonzero(cut), np.flatnonzero(cut)])
    place = np.cumsum(cut) - 1                       # the cut tiles numbered in list order
    code = np.full(which.size, -1, np.int64)
    n_whole = int((~cut).sum())
    code[n_whole:n_whole + n_cut] = 0 | 2 << 4 | place[cut] << 8
    code[n_whole + n_cut:] = 1 | 2 << 4 | place[cut] << 8
    share = np.where(code >= 0, -(-key_tiles[which] // 2), key_tiles[which])
    order = round_about(np.argsort(-share, kind="stable"), per_round)
    return ent_a[which][order], q0_a[which][order], code[order].astype(np.int32), n_cut


def prefill_tiles(ctx: Any, head_dim: int, q_heads: int, kv_heads: int, first_entry: int, device: torch.device,
                  window: int = 0) -> PrefillTiles:
    """The tile list of the step's portions for :func:`ops.attention_prefill` (made once per step
    and shape; the buffers of the cut tiles serve every layer of that shape in turn)."""
    rows = ops.attention_prefill_tile_rows(head_dim, q_heads, kv_heads)
    # a workgroup takes a tile for 4 * 32 / rows query heads where it shares tiles (head sizes that
    # are multiples of 32), else for one
    per_tile = q_heads * rows // 128 if head_dim % 32 == 0 else q_heads
    units = ops.compute_units(device)
    cut_floats = ops.attention_prefill_cut_floats(head_dim, q_heads, kv_heads)
    may_cut = window == 0 and cut_floats > 0

    def make() -> PrefillTiles:
        q_len = (ctx.q_start_host[1:] - ctx.q_start_host[:-1]).astype(np.int64)
        ent, q0, code, n_cut = list_tiles(q_len, np.asarray(ctx.kv_len_host), first_entry, rows, per_tile, units, may_cut)
        if code is None:
            return PrefillTiles(*ctx.upload([ent, q0]))
        entry_t, q0_t, code_t = ctx.upload([ent, q0, code])
        return PrefillTiles(entry_t, q0_t, code_t, n_cut,
                            torch.empty(n_cut * cut_floats, device=device, dtype=torch.float32),
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
                              q_heads, scale, window, t.cut, t.cut_tiles, t.cut_buf, t.cut_count)


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
