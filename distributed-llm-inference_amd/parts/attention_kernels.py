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


def longest_first(ctx: Any, rows: int, units: int = 256, workgroups_per_tile: int = 8) -> Callable:
    """The order in which the prefill kernel wants a step's query tiles: those that see the most
    keys first. Workgroups start in the order of the list, and under a causal mask a tile's work
    grows with its place in the request: listed by place, the longest workgroups start last and
    the launch ends with a few of them alone on the device (a prompt of 8,192 tokens at the 1B
    sizes: 521 us a layer by place, 393 us longest first). Within the sorted list every second
    run of as many tiles as give every compute unit one workgroup (a tile of the list becomes
    ``workgroups_per_tile`` workgroups, one per group of query heads) is turned round, so that a
    unit that got a long tile in one round gets a short one in the next."""
    per_xcd = max(1, units // max(1, workgroups_per_tile))

    def arrange(entries: np.ndarray, firsts: np.ndarray) -> np.ndarray:
        q_len = (ctx.q_start_host[entries + 1] - ctx.q_start_host[entries]).astype(np.int64)
        keys = ctx.kv_len_host[entries].astype(np.int64) - q_len + np.minimum(firsts + rows, q_len)
        order = np.argsort(-keys, kind="stable")
        for r0 in range(per_xcd, order.size, 2 * per_xcd):
            order[r0:r0 + per_xcd] = order[r0:r0 + per_xcd][::-1].copy()
        return order

    return arrange


def prefill_tiles(ctx: Any, head_dim: int, q_heads: int, kv_heads: int, first_entry: int, device: torch.device):
    """The tile list of the step's portions for :func:`ops.attention_prefill`."""
    rows = ops.attention_prefill_tile_rows(head_dim, q_heads, kv_heads)
    # a workgroup takes a tile for 4 * 32 / rows query heads where it shares tiles (head sizes that
    # are multiples of 32), else for one
    per_tile = q_heads * rows // 128 if head_dim % 32 == 0 else q_heads
    units = ops.compute_units(device)
    return ctx.q_tiles(rows, first_entry=first_entry, arrange=longest_first(ctx, rows, units, per_tile),
                       arranged_as=f"longest first, rounds of {max(1, units // max(1, per_tile))}")


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
        tile_entry, tile_q0 = prefill_tiles(ctx, head_dim, q_heads, kv_heads, nd, q.device)
        ops.attention_prefill(q, k_pages, v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                              tile_entry, tile_q0, q_heads, scale, window)


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
