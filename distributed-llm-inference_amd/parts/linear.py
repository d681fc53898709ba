"""``y = x W^T + b`` for both paths.

On the 32-bit path the product is the engine's own IEEE single-precision kernel. On the bfloat16
path it is the vendor library's matrix product (the reference's engine uses a library product
there as well: ``F.linear``, src/dli/model/llama.py:72-74,95,190,305), bfloat16 operands with
32-bit accumulation and the bias added inside; the library is called directly, with its choice of
kernel cached per shape, because a framework's dispatch costs more host time than the product
takes on the GPU when a step has a few hundred tokens.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import DecodeStream, Norm, Runtime


def linear(rt: Runtime, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [n, k] @ weight[m, k].T (+ bias [m]) -> [n, m]`` in the runtime's activation type."""
    n, m = x.shape[0], weight.shape[0]
    if out is None:
        out = rt.empty(n, m)
    if n == 0:
        return out
    if rt.dtype == torch.float32:
        ops.gemm_f32(x, weight, out, bias=bias)
        return out
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.shape[1] != weight.shape[1]:
        raise ops.KernelArgumentError("linear: operands must be bfloat16 [n, k] and [m, k]")
    if not ops.gemm_bf16(x, weight, out, bias):
        # a shape for which the direct call finds no kernel: the same library through torch
        torch.mm(x, weight.t(), out=out)
        if bias is not None:
            ops.add(out, None, out, bias=bias)
    return out


def decode_copy(rt: Runtime, weight: Optional[torch.Tensor], epilogue: int) -> Optional[torch.Tensor]:
    """The matrix once more in the tile order of the decode product (``ops.tile_weights``), or
    ``None`` where that would not be used: another type, sizes that do not tile, a product that
    neither the few-row tile kernel nor the kernel for 17 to 64 rows reads in that order, or a
    runtime that does not want it."""
    if (weight is None or not rt.is_bf16 or not rt.decode_weight_copy or weight.dtype != torch.bfloat16
            or weight.dim() != 2 or not weight.is_cuda):
        return None
    if not (ops.tiled_weights_help(weight.shape[0], weight.shape[1], epilogue, weight.device)
            or ops.mid_tiles_help(weight.shape[0], weight.shape[1], epilogue)):
        return None
    # (rows that are no whole blocks of 128: zero-filled to whole blocks, for the 17-to-64-row kernel alone)
    return ops.tile_weights(weight, whole_blocks=False)


# From this many rows on, the kernel that makes the residual sum also applies the norm that follows
# (one workgroup per row), so that the 256 workgroups of the next product need not each normalise
# every row again: 2% of a decode step at 48 rows and 1% at 64 at the 1B sizes; with 17 to 32 rows
# normalising inside the product is cheaper than a finishing kernel of so few workgroups (steps
# 0.5 to 1% slower), so below it the sums of squares are handed on as they are.
NORM_WITH_THE_SUM_FROM_ROWS = 33


def finish_residual(rt: Runtime, stream: DecodeStream, partial: torch.Tensor, bias: Optional[torch.Tensor],
                    following: Optional[Norm]) -> None:
    """The residual sum of a product that left partial sums, and with it the norm that follows
    where that is known, the rows are many enough for it to pay and narrow enough for one
    workgroup each."""
    fused = following.fused_params() if following is not None and hasattr(following, "fused_params") else None
    rows, width = stream.x.shape
    if (fused is not None and rows >= NORM_WITH_THE_SUM_FROM_ROWS and width <= ops.MID_NORMED_WIDTH
            and fused[0].shape[0] == width):
        normed = rt.empty(rows, width)
        ssq = ops.mid_finish_residual(partial, stream.x, bias, norm_w=fused[0], eps=fused[1], normed_out=normed)
        stream.wrote(ssq, normed, following)
    else:
        stream.wrote(ops.mid_finish_residual(partial, stream.x, bias))
