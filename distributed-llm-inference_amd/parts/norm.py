"""RMSNorm: ``w * cast(x * rsqrt(mean(x^2) + eps))`` with 32-bit statistics; eps inside the root,
no bias, no ``1 + w`` (reference: src/dli/model/llama.py:27-44)."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from ..kernels import ops
from .base import Norm, Runtime
from .registry import register_part
from .spec import WeightSpec


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    def __init__(self, runtime: Runtime, *, width: int, eps: float) -> None:
        super().__init__(runtime)
        self.width, self.eps = width, float(eps)
        self.weight: torch.Tensor | None = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.width,), role="float32", init="norm")}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"]

    def fused_params(self) -> tuple[torch.Tensor, float]:
        """Weight and eps, for a consumer that computes this norm inside its own kernel."""
        return self.weight, self.eps

    def native_fields(self) -> Optional[dict]:
        w = self.weight
        if type(self) is not RMSNorm:
            return None  # a subclass computes something else: it must describe itself
        if w is None or w.dtype != torch.float32 or not w.is_cuda or not w.is_contiguous() or w.data_ptr() % 32:
            return None
        return {"kind": "rms_norm", "w": w, "eps": self.eps, "width": self.width}

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = torch.empty_like(x)
        if delta is None:
            ops.rms_norm(x, self.weight, self.eps, out)
        else:
            ops.rms_norm(x, self.weight, self.eps, out, delta=delta, sum_out=x)
        return out
