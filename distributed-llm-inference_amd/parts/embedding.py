"""Token embedding: a row gather, no scaling (reference: src/dli/model/llama.py:221,291)."""

from __future__ import annotations

from typing import Mapping

import torch

from ..kernels import ops
from .base import DecodeStream, Embedding, Runtime
from .registry import register_part
from .spec import WeightSpec


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, runtime: Runtime, *, vocab_size: int, hidden_size: int) -> None:
        super().__init__(runtime)
        self.vocab_size, self.hidden_size = vocab_size, hidden_size
        self.weight: torch.Tensor | None = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {"weight": WeightSpec((self.vocab_size, self.hidden_size))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"]

    def table(self) -> torch.Tensor:
        assert self.weight is not None
        return self.weight

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        out = self.rt.empty(ids.shape[0], self.hidden_size)
        ops.embedding(self.table(), ids, out)
        return out

    def streams(self, ctx) -> bool:
        return self.rt.is_bf16

    def forward_stream(self, ids: torch.Tensor) -> DecodeStream:
        n = ids.shape[0]
        out = self.rt.empty(n, self.hidden_size)
        ssq = torch.empty(1, n, device=self.rt.device, dtype=torch.float32)
        ops.embedding_ssq(self.table(), ids, out, ssq)
        return DecodeStream(out, ssq)
