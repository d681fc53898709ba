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


def sampling_tuple(params: SamplingParams, seed: Optional[int], draw_index: int) -> tuple:
    """``(temperature, top_k, top_p, seed, draw index)`` as the sampling kernel takes them;
    temperature 0 stands for every greedy request."""
    if not params.greedy and seed is None:
        raise ValueError("a request that samples stochastically has no seed for its generator")
    return (0.0 if params.greedy else float(params.temperature), int(params.top_k), float(params.top_p),
            int(seed or 0) & _MASK63, int(draw_index))


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
    tuples = [sampling_tuple(p, s, d) for p, s, d in zip(params, seeds, draw_indices)]
    dev = logits.device
    floats = torch.tensor([[t[0] for t in tuples], [t[2] for t in tuples]], dtype=torch.float32).to(dev)
    top_k = torch.tensor([t[1] for t in tuples], dtype=torch.int32).to(dev)
    longs = torch.tensor([[t[3] for t in tuples], [t[4] for t in tuples]], dtype=torch.int64).to(dev)
    out = torch.empty(rows, dtype=torch.int32, device=dev)
    ops.sample(logits, floats[0], top_k, floats[1], longs[0], longs[1], out)
    return out.cpu().tolist()
