"""Pre-norm arrangement: ``x + mixer(norm(x))`` then ``x + feed_forward(norm(x))``
(reference: src/dli/model/llama.py:194-213). The residual sums are made inside the norms that
follow them (32-bit sum, rounded to the activation type, then normalised)."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from .base import Block, DecodeStream, Part, Runtime
from .registry import register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    roles = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")

    def __init__(self, runtime: Runtime) -> None:
        super().__init__(runtime)

    def graph_capturable(self, page_size: int) -> bool:
        return True  # kernels on device arrays only

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        h = parts["mixer_norm"].forward(x, delta)          # x <- x + delta
        a = parts["mixer"].forward(h, ctx, cache)
        h = parts["feed_forward_norm"].forward(x, a)       # x <- x + a
        f = parts["feed_forward"].forward(h, ctx)
        return x, f

    # the arrangement of parts that the loop in C implements (``DLI_BLOCK_PRENORM_RMS_GQA_SILU``)
    NATIVE_KIND = 1
    NATIVE_PARTS = {"mixer_norm": "rms_norm", "mixer": "gqa_rotary_half", "feed_forward_norm": "rms_norm",
                    "feed_forward": "gated_silu"}

    def native_fields(self, parts: Mapping[str, Part]) -> Optional[dict]:
        """This arrangement with its parts' tensors and constants, for the loop in C that issues a
        step's launches. That loop hard-codes one order of work, so the answer is ``None`` unless
        this is exactly this class (a subclass must describe itself), each of the four parts
        names exactly the kind that the loop computes, and all agree on the width."""
        if type(self) is not PreNormBlock:
            return None
        fields = {role: parts[role].native_fields() for role in self.NATIVE_PARTS}
        if any(f is None or f.get("kind") != self.NATIVE_PARTS[role] for role, f in fields.items()):
            return None
        n1, n2, mix, ff = (fields[r] for r in ("mixer_norm", "feed_forward_norm", "mixer", "feed_forward"))
        if not n1["width"] == n2["width"] == mix["hidden"] == ff["hidden"]:
            return None
        return {**mix, **ff, "kind": self.NATIVE_KIND, "norm1_w": n1["w"], "eps1": n1["eps"], "norm2_w": n2["w"],
                "eps2": n2["eps"]}

    def streams(self, ctx: Any, parts: Mapping[str, Part]) -> bool:
        fused_norms = all(hasattr(parts[r], "fused_params") for r in ("mixer_norm", "feed_forward_norm"))
        return fused_norms and parts["mixer"].streams(ctx) and parts["feed_forward"].streams(ctx)

    def first_norm(self, parts: Mapping[str, Part]) -> Optional[Part]:
        return parts["mixer_norm"]

    def forward_stream(self, stream: DecodeStream, ctx: Any, cache: Any, parts: Mapping[str, Part],
                       following: Optional[Part] = None) -> None:
        """``following``: the norm that whatever comes after this block applies first (the last
        kernel of the block may apply it while it writes the stream)."""
        parts["mixer"].forward_stream(stream, parts["mixer_norm"], ctx, cache, following=parts["feed_forward_norm"])
        parts["feed_forward"].forward_stream(stream, parts["feed_forward_norm"], ctx, following=following)
