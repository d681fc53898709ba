"""Chooses one token per logits row on the GPU.

Each stochastic request draws from its own counter-based random stream: draw ``n`` of a request
uses Philox4x32-10 keyed by the request's seed with counter ``n``. What a request draws therefore
depends on its seed and on how many tokens it has sampled, never on its neighbours in the batch,
and a request that is preempted and recomputed continues its stream where it stopped, because
recomputation samples nothing (reference: src/dli/sampling.py:1-10).
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams

_MASK63 = (1 << 63) - 1


def sample(logits: torch.Tensor, params: Sequence[SamplingParams], seeds: Sequence[Optional[int]],
           draw_indices: Sequence[int]) -> list[int]:
    """One token id per row of float32 ``logits [rows, vocab]`` (device tensor).

    ``seeds[i]`` may be ``None`` only for greedy rows; ``draw_indices[i]`` is the number of tokens
    that request has sampled so far.
    """
    rows = logits.shape[0]
    if not len(params) == len(seeds) == len(draw_indices) == rows:
        raise ValueError("logits, params, seeds and draw_indices must have one entry per row")
    if rows == 0:
        return []
    for i, (p, s) in enumerate(zip(params, seeds)):
        if not p.greedy and s is None:
            raise ValueError(f"row {i} samples stochastically but has no seed for its generator")
    dev = logits.device
    host = torch.tensor(
        [[0.0 if p.greedy else p.temperature for p in params], [p.top_p for p in params]], dtype=torch.float32)
    ints = torch.tensor([p.top_k for p in params], dtype=torch.int32)
    longs = torch.tensor([[(s or 0) & _MASK63 for s in seeds], [int(d) for d in draw_indices]], dtype=torch.int64)
    fdev, idev, ldev = host.to(dev), ints.to(dev), longs.to(dev)
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    ops.sample(logits, fdev[0], idev, fdev[1], ldev[0], ldev[1], out)
    return out.cpu().tolist()
