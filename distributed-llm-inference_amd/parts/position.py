"""Rotary position encoding: the table of inverse frequencies.

``inv_freq[i] = theta^(-2i/d)``; ``linear`` divides all by ``factor``; ``llama3`` keeps
wavelengths below ``original/high_freq_factor``, divides those above
``original/low_freq_factor`` by ``factor`` and blends in between with
``s = (original/wavelen - low) / (high - low)``: ``(1 - s) * f / factor + s * f``
(reference: src/dli/model/rope.py:21-47). The table is computed once on the host in double
precision and rounded to float32; the rotation itself happens in the attention mixer's fused
cache-write kernel, from ``float(position) * inv_freq`` in 32-bit.
"""

from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from .base import PositionEncoding, RotaryTable, Runtime
from .registry import register_part


def rotary_inverse_frequencies(dim: int, theta: float, rope_type: str = "default", factor: float = 1.0,
                               low_freq_factor: float = 1.0, high_freq_factor: float = 4.0,
                               original_max_position_embeddings: int = 8192) -> np.ndarray:
    """``[dim/2]`` float32 inverse frequencies."""
    if dim <= 0 or dim % 2:
        raise ValueError(f"rotary dimension {dim} must be positive and even")
    exponents = np.arange(0, dim, 2, dtype=np.float64) / dim
    inv = 1.0 / np.power(float(theta), exponents)
    if rope_type == "default":
        pass
    elif rope_type == "linear":
        inv = inv / factor
    elif rope_type == "llama3":
        old = float(original_max_position_embeddings)
        low_wavelen, high_wavelen = old / low_freq_factor, old / high_freq_factor
        wavelen = 2.0 * math.pi / inv
        smooth = (old / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        blended = (1.0 - smooth) * inv / factor + smooth * inv
        inv = np.where(wavelen > low_wavelen, inv / factor, np.where(wavelen < high_wavelen, inv, blended))
    else:
        raise ValueError(f"unsupported rope_type {rope_type!r}")
    return inv.astype(np.float32)


_TABLES: dict = {}


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    def __init__(self, runtime: Runtime, *, dim: int, theta: float, rope_type: str = "default",
                 factor: float = 1.0, low_freq_factor: float = 1.0, high_freq_factor: float = 4.0,
                 original_max_position_embeddings: int = 8192) -> None:
        super().__init__(runtime)
        self.dim = dim
        self.inv_freq_host = rotary_inverse_frequencies(
            dim, theta, rope_type, factor, low_freq_factor, high_freq_factor,
            original_max_position_embeddings)
        self._table: Optional[torch.Tensor] = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def finalize(self) -> None:
        # equal tables share one device tensor, so that what a step derives from a table (the cos
        # and sin of its positions) is derived once for all layers
        key = (str(self.rt.device), self.inv_freq_host.tobytes())
        hit = _TABLES.get(key)
        if hit is None:
            hit = _TABLES[key] = torch.from_numpy(self.inv_freq_host.copy()).to(self.rt.device)
        self._table = hit

    def rotary_table(self) -> Optional[RotaryTable]:
        if self._table is None:
            self.finalize()
        return RotaryTable(self._table, self.dim, "half")


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """Keys and queries are used as projected."""

    def __init__(self, runtime: Runtime) -> None:
        super().__init__(runtime)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only
