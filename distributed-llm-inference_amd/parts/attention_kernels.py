"""Choice of attention kernel for a step.

The true 32-bit path, and shapes that the matrix-core kernels do not take, run the vector-unit
kernel over all entries. The bfloat16 path sends entries that bring one token to the split-key
decode kernel and portions to the tiled prefill kernel when their shapes allow it.
"""

from __future__ import annotations

from typing import Any

import torch

from ..kernels import ops


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                    ctx: Any, grp: Any, q_heads: int, scale: float, window: int = 0) -> None:
    """Attention of every row of the step over its request's pages, into ``out``."""
    if ctx.num_tokens == 0:
        return
    head_dim = k_pages.shape[3]
    rows = ops.attention_generic_tile_rows(head_dim)
    tile_entry, tile_q0 = ctx.q_tiles(rows)
    ops.attention_generic(q, k_pages, v_pages, out, ctx.q_start, ctx.kv_len, grp.block_tables,
                          tile_entry, tile_q0, q_heads, scale, window)
