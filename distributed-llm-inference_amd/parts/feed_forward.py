"""Gated feed-forward: ``down(act(gate(x)) * up(x))`` with ``act = silu`` (SwiGLU; reference:
src/dli/model/llama.py:180-191). Gate and up matrices are stacked at load, so one product gives
both halves; the activation kernel reads them side by side."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .base import DecodeStream, FeedForward, Norm, Runtime
from .linear import decode_copy, finish_residual, linear
from .registry import register_part
from .spec import WeightSpec


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, runtime: Runtime, *, hidden_size: int, intermediate_size: int,
                 activation: str = "silu", bias: bool = False) -> None:
        super().__init__(runtime)
        if activation != "silu":
            raise ValueError(f"gated_mlp has no kernel for activation {activation!r} (only 'silu')")
        self.hidden_size, self.intermediate_size, self.bias = hidden_size, intermediate_size, bias
        self.w_gate_up = self.b_gate_up = self.w_down = self.b_down = None
        self.w_gate_up_tiled = self.w_down_tiled = None

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def weight_specs(self) -> dict[str, WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        specs = {"gate_proj.weight": WeightSpec((i, h)), "up_proj.weight": WeightSpec((i, h)),
                 "down_proj.weight": WeightSpec((h, i))}
        if self.bias:
            specs.update({"gate_proj.bias": WeightSpec((i,)), "up_proj.bias": WeightSpec((i,)),
                          "down_proj.bias": WeightSpec((h,))})
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], 0).contiguous()
        self.w_down = tensors["down_proj.weight"]
        if self.bias:
            self.b_gate_up = torch.cat([tensors["gate_proj.bias"], tensors["up_proj.bias"]], 0).contiguous()
            self.b_down = tensors["down_proj.bias"]

    def finalize(self) -> None:
        self.w_gate_up_tiled = decode_copy(self.rt, self.w_gate_up, ops.SKINNY_SWIGLU)
        self.w_down_tiled = decode_copy(self.rt, self.w_down, ops.SKINNY_RESIDUAL)

    def native_fields(self):
        from .native import _bf16_matrix, _bf16_vector

        h, i = self.hidden_size, self.intermediate_size
        if type(self) is not GatedMLP:
            return None  # a subclass computes something else: it must describe itself
        if not (self.rt.is_bf16 and _bf16_matrix(self.w_gate_up, 2 * i, h) and _bf16_matrix(self.w_down, h, i)
                and _bf16_vector(self.b_gate_up, 2 * i) and _bf16_vector(self.b_down, h)):
            return None
        return {"kind": "gated_silu", "w_gate_up": self.w_gate_up, "b_gate_up": self.b_gate_up, "w_down": self.w_down, "b_down": self.b_down,
                "hidden": h, "intermediate": i}

    def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
        gate_up = linear(self.rt, x, self.w_gate_up, self.b_gate_up)
        act = self.rt.empty(x.shape[0], self.intermediate_size)
        ops.silu_mul(gate_up, act)
        return linear(self.rt, act, self.w_down, self.b_down)

    FEW_ROWS = 16  # the few-row product kernels; 17 to 64 rows take the one that shares activations

    def streams(self, ctx: Any) -> bool:
        n = ctx.num_tokens
        if not (self.rt.is_bf16 and self.hidden_size % 8 == 0):
            return False
        if n > self.FEW_ROWS:
            return (self.w_gate_up_tiled is not None and self.w_down_tiled is not None
                    and ops.mid_gemm_supports(n, self.hidden_size, self.rt.dtype)
                    and ops.mid_gemm_supports(n, self.intermediate_size, self.rt.dtype))
        return (ops.skinny_gemm_supports(n, self.hidden_size, self.rt.dtype)
                and ops.skinny_gemm_supports(n, self.intermediate_size, self.rt.dtype))

    def forward_stream(self, stream: DecodeStream, norm: Norm, ctx: Any, following: Optional[Norm] = None) -> None:
        """``stream.x += mlp(norm(stream.x))``, norm and sum inside the two products' kernels.
        ``following``: the norm that the stream meets next; with 17 to 64 rows the kernel that makes
        the residual sum applies it as well, so that the next product reads normalised rows."""
        n = stream.x.shape[0]
        norm_w, eps = norm.fused_params()
        if n > self.FEW_ROWS:
            ready = stream.normed_by(norm)
            if ready is not None:
                act = ops.mid_gemm(ready, self.w_gate_up_tiled, tiled=True, n=self.intermediate_size,
                                   epilogue=ops.MID_SWIGLU, bias=self.b_gate_up)
            else:
                act = ops.mid_gemm(stream.x, self.w_gate_up_tiled, tiled=True, n=self.intermediate_size,
                                   epilogue=ops.MID_SWIGLU, bias=self.b_gate_up, norm_w=norm_w, eps=eps,
                                   ssq_in=stream.ssq)
            partial = ops.mid_gemm(act, self.w_down_tiled, tiled=True, n=self.hidden_size, epilogue=ops.MID_PARTIAL)
            finish_residual(self.rt, stream, partial, self.b_down, following)
            return
        act = self.rt.empty(n, self.intermediate_size)
        ops.skinny_gemm(stream.x, self.w_gate_up, w_tiled=self.w_gate_up_tiled, epilogue=ops.SKINNY_SWIGLU, out=act,
                        bias=self.b_gate_up, norm_w=norm_w, eps=eps, ssq_in=stream.ssq)
        stream.wrote(ops.skinny_gemm(act, self.w_down, w_tiled=self.w_down_tiled, epilogue=ops.SKINNY_RESIDUAL,
                                     stream=stream.x, bias=self.b_down))
