"""Output head: ``logits = x W^T`` with ``W`` the embedding table when tied, else its own matrix;
no bias, no scaling (reference: src/dli/model/llama.py:237-240,304-305). Logits leave in float32."""

from __future__ import annotations

from typing import Mapping, Optional

import torch

from ..kernels import ops
from .base import ArgmaxStage, DecodeStream, Head, Norm, Runtime
from .linear import decode_copy, linear
from .registry import register_part
from .spec import WeightSpec


@register_part("head", "linear_head")
class LinearHead(Head):
    def __init__(self, runtime: Runtime, *, vocab_size: int, hidden_size: int, tied: bool) -> None:
        super().__init__(runtime)
        self.vocab_size, self.hidden_size, self.tied = vocab_size, hidden_size, tied
        self.weight: Optional[torch.Tensor] = None
        self.weight_tiled: Optional[torch.Tensor] = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {} if self.tied else {"weight": WeightSpec((self.vocab_size, self.hidden_size))}

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        if not self.tied:
            self.weight = tensors["weight"]

    def tie(self, table: torch.Tensor) -> None:
        if self.tied:
            self.weight = table

    def finalize(self) -> None:
        self.weight_tiled = decode_copy(self.rt, self.weight, ops.SKINNY_F32)

    FEW_ROWS = 16  # up to here the decode product streams the table faster than the library does

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = x.shape[0]
        if (self.rt.is_bf16 and 0 < rows <= self.FEW_ROWS and x.dtype == torch.bfloat16
                and ops.skinny_gemm_supports(rows, self.hidden_size, self.rt.dtype)):
            # the usual case of a prompt's step: logits for its last row only
            out = torch.empty(rows, self.vocab_size, device=self.rt.device, dtype=torch.float32)
            self._few_rows(x, out)
            return out
        if self.rt.is_bf16 and rows > 0 and x.dtype == torch.bfloat16:
            # many rows: the library's product, leaving the 32-bit sums as the logits
            out = torch.empty(rows, self.vocab_size, device=self.rt.device, dtype=torch.float32)
            if ops.gemm_bf16(x, self.weight, out):
                return out
        logits = linear(self.rt, x, self.weight)
        if logits.dtype == torch.float32:
            return logits
        out = torch.empty(logits.shape, device=logits.device, dtype=torch.float32)
        ops.to_float(logits, out)
        return out

    def streams(self, ctx) -> bool:
        return self.rt.is_bf16 and (ctx.num_tokens > self.FEW_ROWS
                                    or ops.skinny_gemm_supports(ctx.num_tokens, self.hidden_size, self.rt.dtype))

    def forward_stream(self, stream: DecodeStream, norm: Norm, argmax: Optional[ArgmaxStage] = None) -> torch.Tensor:
        """Logits of every row of the stream, the final norm computed inside the product (with
        more than a few rows: the norm kernel, then the library product). ``argmax``: where the
        kernel that makes the logits may leave the first stage of every row's argmax."""
        if stream.x.shape[0] > self.FEW_ROWS:
            ready = stream.normed_by(norm)  # the last residual sum's kernel may have normalised already
            return self.forward(ready if ready is not None else norm.forward(stream.x))
        norm_w, eps = norm.fused_params()
        out = torch.empty(stream.x.shape[0], self.vocab_size, device=self.rt.device, dtype=torch.float32)
        parts = self._few_rows(stream.x, out, best=argmax.scratch if argmax is not None else None,
                               norm_w=norm_w, eps=eps, ssq_in=stream.ssq)
        if argmax is not None:
            argmax.parts = parts
        return out

    def _few_rows(self, x: torch.Tensor, out: torch.Tensor, best=None, **norm) -> int:
        """At most 16 rows: the kernel whose workgroups stay and walk the table (a long stream:
        at the 1B sizes 89 to 100 us for 1 to 16 rows against 92 to 112 with a workgroup per pair
        of tiles), where it takes the sizes; else the few-row product."""
        if self.weight_tiled is not None and ops.head_gemm_supports(x.shape[0], self.vocab_size, self.hidden_size, x.dtype):
            return ops.head_gemm(x, self.weight_tiled, out, best=best, **norm)
        ops.skinny_gemm(x, self.weight, w_tiled=self.weight_tiled, epilogue=ops.SKINNY_F32, out=out, **norm)
        return 0
