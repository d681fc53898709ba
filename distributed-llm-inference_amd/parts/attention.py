"""Grouped-query self-attention over the paged cache, with position encoding and cache write.

Order of work (reference: src/dli/model/llama.py:61-96,112-177): project q, k, v (one fused
product: the three checkpoint matrices are stacked at load), rotate q and k and write rotated k and
raw v at each token's cache slot (one kernel), attend to the request's pages (causal by absolute
position, scale ``1/sqrt(head_dim)`` unless given, query head ``h`` reads kv head
``h // (heads / kv_heads)``), project the result. Keys are cached after rotation: positions are
absolute, so cached keys never change.

Parameters only: the part knows its own sizes, not the model it sits in.
``window`` > 0 restricts each query to the last ``window`` keys. ``shares_kv`` makes a mixer that
has no k/v projections and reads the pages another schedule entry wrote.
"""

from __future__ import annotations

import math
from typing import Any, Mapping, Optional

import torch

from ..kernels import ops
from .attention_kernels import decode_attention_unmerged, head_tiles, paged_attention, planned_splits
from .base import DecodeStream, Mixer, Norm, PagedKVSpec, Part, Runtime
from .linear import decode_copy, finish_residual, linear
from .registry import build_part, register_part
from .spec import PartSpec, WeightSpec

# Decode steps with this many rows rotate and write the cache in the epilogue of the q/k/v
# product, which reads a copy of the matrix whose tiles hold whole rotary pairs: no rotation
# kernel runs. (A variant that rotated inside the attention kernel instead, repeating the rotation
# in every split of the keys, was slower from four rows on and no faster below.)
ROPE_IN_PRODUCT_ROWS = range(1, 17)
# Decode steps with this many rows leave the merge of the runs of keys to the o projection, whose
# waves merge the k that they multiply while their first weights are on their way. Every workgroup
# of that product repeats the merge of all rows, so it pays for one row only (a batch-1 step at
# the 1B sizes: 0.902 ms against 0.935 with the attention launch that merges in its last
# workgroups; at two rows 1.002 against 0.994; at three and four rows 6% slower than even a
# separate merge kernel).
MERGE_IN_PRODUCT_ROWS = 1
FEW_ROWS = 16  # up to here the few-row product kernels run; from 17 to 64 rows the one that shares activations


@register_part("mixer", "gqa_attention")
class GQAttention(Mixer):
    def __init__(self, runtime: Runtime, *, hidden_size: int, num_heads: int, num_kv_heads: int,
                 head_dim: int, position: Optional[PartSpec] = None, qkv_bias: bool = False,
                 o_bias: bool = False, window: int = 0, scale: Optional[float] = None,
                 shares_kv: bool = False) -> None:
        super().__init__(runtime)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not group onto {num_kv_heads} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ops.KernelArgumentError(
                f"attention takes head_dim in steps of 16 from 16 to 256, not {head_dim}")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.window, self.shares_kv = head_dim, int(window), shares_kv
        self.qkv_bias, self.o_bias = qkv_bias, o_bias
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.position = build_part("position", position or PartSpec("none"), runtime)
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = None
        self.w_qkv_tiled = self.w_o_tiled = None
        self.w_qkv_rope = self.b_qkv_rope = None  # tile order with rotary pairs, for the product that rotates
        self._arrivals: Optional[torch.Tensor] = None

    ARRIVAL_COUNTERS = 4096  # keys are cut into runs only when requests x kv heads are few

    def arrival_counters(self, needed: int) -> Optional[torch.Tensor]:
        """``needed`` counters with which a decode attention launch merges its runs of keys by
        itself (``ops.attention_decode``): zero when made, and every launch leaves them zero. They
        are this layer's own, since launches that share counters must not overlap, and they are
        made once and kept, since captured graphs hold their address. None (then the merge
        kernel runs) if more are needed than there are, or if they would have to be made while
        the stream is being captured into a graph: their memory would belong to that graph."""
        if needed > self.ARRIVAL_COUNTERS:
            return None
        if self._arrivals is None:
            if torch.cuda.is_current_stream_capturing():
                return None
            self._arrivals = torch.zeros(self.ARRIVAL_COUNTERS, device=self.rt.device, dtype=torch.int32)
        return self._arrivals

    # -- weights
    def weight_specs(self) -> dict[str, WeightSpec]:
        q, kv, h = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim, self.hidden_size
        names = {"q_proj": q} if self.shares_kv else {"q_proj": q, "k_proj": kv, "v_proj": kv}
        specs = {f"{n}.weight": WeightSpec((rows, h)) for n, rows in names.items()}
        if self.qkv_bias:
            specs.update({f"{n}.bias": WeightSpec((rows,)) for n, rows in names.items()})
        specs["o_proj.weight"] = WeightSpec((h, q))
        if self.o_bias:
            specs["o_proj.bias"] = WeightSpec((h,))
        return specs

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        names = ["q_proj"] if self.shares_kv else ["q_proj", "k_proj", "v_proj"]
        self.w_qkv = torch.cat([tensors[f"{n}.weight"] for n in names], dim=0).contiguous()
        self.b_qkv = (torch.cat([tensors[f"{n}.bias"] for n in names], dim=0).contiguous()
                      if self.qkv_bias else None)
        self.w_o = tensors["o_proj.weight"]
        self.b_o = tensors.get("o_proj.bias") if self.o_bias else None

    def finalize(self) -> None:
        self.w_qkv_tiled = decode_copy(self.rt, self.w_qkv, ops.SKINNY_STORE)
        self.w_o_tiled = decode_copy(self.rt, self.w_o, ops.SKINNY_RESIDUAL)
        table = self.position.rotary_table()
        if table is not None and table.pairing != "half":
            raise ops.KernelArgumentError(
                f"the attention kernels rotate pairs (i, i + dim/2); the position encoding asks for "
                f"the pairing {table.pairing!r} (give it an apply() instead of a rotary table)")
        if table is not None and (table.dim % 2 or not 0 < table.dim <= self.head_dim):
            raise ops.KernelArgumentError(
                f"rotary dimension {table.dim} does not fit heads of {self.head_dim}")
        if (self.w_qkv_tiled is not None and not self.shares_kv and table is not None
                and table.dim == self.head_dim):
            # the rotation covers the whole head: the product can rotate in its epilogue, and
            # this order of the features replaces the plain tile order
            nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
            self.w_qkv_rope = ops.tile_weights_qkv_rope(self.w_qkv, nh, nkv, d)
            if self.b_qkv is not None:
                order = ops.qkv_rope_feature_order(nh, nkv, d).to(self.b_qkv.device)
                self.b_qkv_rope = self.b_qkv[order].contiguous()
            self.w_qkv_tiled = None  # every step that would read it takes the other copy

    def sub_parts(self) -> dict[str, Part]:
        return {"position": self.position}

    def native_fields(self) -> Optional[dict]:
        from .native import _bf16_matrix, _bf16_vector

        nh, nkv, d, h = self.num_heads, self.num_kv_heads, self.head_dim, self.hidden_size
        table = self.position.rotary_table()
        if type(self) is not GQAttention:
            return None  # a subclass computes something else: it must describe itself
        if not self.rt.is_bf16 or self.shares_kv or table is None or table.pairing != "half":
            return None
        if not (_bf16_matrix(self.w_qkv, (nh + 2 * nkv) * d, h) and _bf16_matrix(self.w_o, h, nh * d)
                and _bf16_vector(self.b_qkv, (nh + 2 * nkv) * d) and _bf16_vector(self.b_o, h)):
            return None
        return {"kind": "gqa_rotary_half", "w_qkv": self.w_qkv, "b_qkv": self.b_qkv, "w_o": self.w_o, "b_o": self.b_o,
                "inv_freq": table.inv_freq, "rotary_dim": table.dim, "hidden": h, "q_heads": nh, "kv_heads": nkv,
                "head_dim": d, "scale": self.scale, "window": self.window, "plan_owner": id(self)}

    def cache_spec(self) -> Optional[PagedKVSpec]:
        return None if self.shares_kv else PagedKVSpec(self.num_kv_heads, self.head_dim, self.window)

    def graph_capturable(self, page_size: int) -> bool:
        # the matrix-core decode path is all kernels on the step's device arrays
        return (self.rt.is_bf16 and ops.attention_mfma_supports(self.head_dim, page_size, self.rt.dtype)
                and self.position.graph_capturable(page_size))

    def decode_plan(self, requests: int, max_keys: int) -> Optional[int]:
        """Into how many runs the decode kernel cuts each request's keys in a recorded step."""
        return planned_splits(requests, head_tiles(self.num_heads, self.num_kv_heads), max_keys,
                              ops.compute_units(self.rt.device))

    # -- step
    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        if cache is None or cache.kind != "paged":
            raise RuntimeError("gqa_attention needs a paged cache")
        nh, d = self.num_heads, self.head_dim
        nkv = 0 if self.shares_kv else self.num_kv_heads
        if not self.shares_kv and not cache.writable:
            raise RuntimeError("this attention writes its cache but was given a read-only one")
        grp = ctx.groups[cache.group]
        qkv = linear(self.rt, x, self.w_qkv, self.b_qkv)
        table = self.position.rotary_table()
        if table is None:
            n = x.shape[0]
            q_view = qkv[:, :nh * d].view(n, nh, d)
            k_view = qkv[:, nh * d:(nh + nkv) * d].view(n, nkv, d) if nkv else None
            self.position.apply(q_view, k_view, ctx.positions)
            inv_freq, rotary_dim = None, 0
        else:
            inv_freq, rotary_dim = table.inv_freq, table.dim
        ops.rope_kv_write(qkv, ctx.positions, inv_freq, rotary_dim, grp.slots if nkv else None,
                          cache.k_pages if nkv else None, cache.v_pages if nkv else None, nh, nkv, d)
        q = qkv[:, :nh * d]
        out = self.rt.empty(x.shape[0], nh * d)
        paged_attention(q, cache.k_pages, cache.v_pages, out, ctx, grp, nh, self.scale, self.window,
                        self.arrival_counters, planned=ctx.decode_plans.get(id(self)))
        return linear(self.rt, out, self.w_o, self.b_o)

    # -- decode steps with few rows: the norm before and the residual sum after are fused into
    #    the two projections' kernels
    def streams(self, ctx: Any) -> bool:
        nh, d, n = self.num_heads, self.head_dim, ctx.num_tokens
        if not (self.rt.is_bf16 and ctx.num_decode == ctx.num_entries and self.hidden_size % 8 == 0
                and ops.attention_mfma_supports(d, ctx.page_size, self.rt.dtype)):
            return False
        if n > FEW_ROWS:
            # 17 to 64 rows: the product kernel that shares the activations through LDS; it reads
            # the tile-ordered copies and leaves rotation and cache write to its finishing kernel
            return (self.w_qkv_rope is not None and self.w_o_tiled is not None
                    and ops.mid_gemm_supports(n, self.hidden_size, self.rt.dtype)
                    and ops.mid_gemm_supports(n, nh * d, self.rt.dtype))
        return (ops.skinny_gemm_supports(n, self.hidden_size, self.rt.dtype)
                and ops.skinny_gemm_supports(n, nh * d, self.rt.dtype))

    def forward_stream(self, stream: DecodeStream, norm: Norm, ctx: Any, cache: Any,
                       following: Optional[Norm] = None) -> None:
        """``stream.x += attention(norm(stream.x))``, the norm inside the first product's kernel and
        the sum inside the last one's. ``following``: the norm that the stream meets next."""
        nh, d = self.num_heads, self.head_dim
        nkv = 0 if self.shares_kv else self.num_kv_heads
        grp = ctx.groups[cache.group]
        n = stream.x.shape[0]
        norm_w, eps = norm.fused_params()
        if n > FEW_ROWS:
            self._forward_stream_mid(stream, norm, ctx, cache, grp, following)
            return
        qkv = self.rt.empty(n, (nh + 2 * nkv) * d)
        if self.w_qkv_rope is not None and n in ROPE_IN_PRODUCT_ROWS and self.hidden_size % 128 == 0:
            # product, rotation and cache write in one kernel; only q comes back
            angles = self.position.step_angles(ctx, qkv.dtype)
            ops.skinny_gemm_qkv_rope(stream.x, self.w_qkv_rope, qkv, angles, grp.slots, cache.k_pages, cache.v_pages,
                                     nh, bias=self.b_qkv_rope, norm_w=norm_w, eps=eps, ssq_in=stream.ssq)
        else:
            ops.skinny_gemm(stream.x, self.w_qkv, w_tiled=self.w_qkv_tiled, epilogue=ops.SKINNY_STORE, out=qkv,
                            bias=self.b_qkv, norm_w=norm_w, eps=eps, ssq_in=stream.ssq)
            table = self.position.rotary_table()
            if table is None:
                q_view = qkv[:, :nh * d].view(n, nh, d)
                k_view = qkv[:, nh * d:(nh + nkv) * d].view(n, nkv, d) if nkv else None
                self.position.apply(q_view, k_view, ctx.positions)
                inv_freq, rotary_dim = None, 0
            else:
                inv_freq, rotary_dim = table.inv_freq, table.dim
            ops.rope_kv_write(qkv, ctx.positions, inv_freq, rotary_dim, grp.slots if nkv else None,
                              cache.k_pages if nkv else None, cache.v_pages if nkv else None, nh, nkv, d)
        if n <= MERGE_IN_PRODUCT_ROWS and self.w_o_tiled is not None:
            # the o projection merges the runs of keys itself while its first
            # weights are on their way, and no merge kernel runs between the two
            left = decode_attention_unmerged(
                qkv[:, :nh * d], cache.k_pages, cache.v_pages, ctx, grp, nh, self.scale, self.window,
                lambda splits: ops.skinny_gemm_merged_supports(n, self.hidden_size, nh, d, splits, qkv.device),
                planned=ctx.decode_plans.get(id(self)))
            if left is not None:
                splits, part_o, part_ml = left
                stream.wrote(ops.skinny_gemm_merged(part_o, part_ml, splits, nh, d, self.w_o_tiled, stream.x,
                                                    bias=self.b_o))
                return
        out = self.rt.empty(n, nh * d)
        paged_attention(qkv[:, :nh * d], cache.k_pages, cache.v_pages, out, ctx, grp, nh, self.scale, self.window,
                        self.arrival_counters, planned=ctx.decode_plans.get(id(self)))
        stream.wrote(ops.skinny_gemm(out, self.w_o, w_tiled=self.w_o_tiled, epilogue=ops.SKINNY_RESIDUAL,
                                     stream=stream.x, bias=self.b_o))

    def _forward_stream_mid(self, stream: DecodeStream, norm: Norm, ctx: Any, cache: Any, grp: Any,
                            following: Optional[Norm]) -> None:
        """The same for 17 to 64 rows: both products split k over workgroups and leave 32-bit
        partial sums; the kernel that rotates and writes the cache, and the one that makes the
        residual sum (and applies the norm that follows), add them up."""
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        n = stream.x.shape[0]
        ready = stream.normed_by(norm)
        if ready is not None:
            partial = ops.mid_gemm(ready, self.w_qkv_rope, tiled=True, n=(nh + 2 * nkv) * d, epilogue=ops.MID_PARTIAL)
        else:
            norm_w, eps = norm.fused_params()
            partial = ops.mid_gemm(stream.x, self.w_qkv_rope, tiled=True, n=(nh + 2 * nkv) * d,
                                   epilogue=ops.MID_PARTIAL, norm_w=norm_w, eps=eps, ssq_in=stream.ssq)
        q = self.rt.empty(n, nh * d)
        angles = self.position.step_angles(ctx, q.dtype)
        ops.mid_finish_qkv(partial, q, angles, grp.slots, cache.k_pages, cache.v_pages, nh, bias=self.b_qkv_rope)
        out = self.rt.empty(n, nh * d)
        paged_attention(q, cache.k_pages, cache.v_pages, out, ctx, grp, nh, self.scale, self.window,
                        self.arrival_counters, planned=ctx.decode_plans.get(id(self)))
        partial = ops.mid_gemm(out, self.w_o_tiled, tiled=True, n=self.hidden_size, epilogue=ops.MID_PARTIAL)
        finish_residual(self.rt, stream, partial, self.b_o, following)
