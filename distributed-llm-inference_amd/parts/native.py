"""The layers of a step issued from one call into the HIP library.

A step that holds portions of prompts is launched kernel by kernel (only decode-only steps replay
graphs). Going through every part's ``forward`` costs eleven checked calls and as many temporaries
a layer: more host time than the GPU needs for a step of a few hundred tokens. When every block of
the model is the pre-norm arrangement of RMSNorm, rotary grouped-query attention over pages and a
gated feed-forward, in bfloat16, the same launches are issued from a loop in C instead
(``csrc/block_steps.hip``): the parts describe themselves once (:meth:`Part.native_fields`), the
step describes its batch once, and one call runs all layers. Anything else (another block or
part, the 32-bit path, a shape the matrix-core attention or the vendor library does not take)
runs part by part as before; the results are the same either way, the kernels being the same.

The structures mirror ``csrc/block_steps.h`` field by field.
"""

from __future__ import annotations

import ctypes
from typing import Any, Optional, Sequence

import torch

from ..kernels import ops
from .attention_kernels import prefill_tiles, step_splits

MAX_GROUPS, MAX_SHAPES = 4, 4
_p, _i32, _i64, _f = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float


class StepShape(ctypes.Structure):
    _fields_ = [("tile_entry", _p), ("tile_q0", _p), ("tiles", _i32), ("decode_splits", _i32), ("tile_cut", _p),
                ("cut_buf", _p), ("cut_count", _p), ("cut_tiles", _i32), ("cut_room", _i32)]


class StepArgs(ctypes.Structure):
    _fields_ = [("rows", _i32), ("num_decode", _i32), ("num_entries", _i32), ("page_size", _i32), ("device", _i32),
                ("pad0", _i32), ("positions", _p), ("q_start", _p), ("kv_len", _p), ("slots", _p * MAX_GROUPS),
                ("block_tables", _p * MAX_GROUPS), ("table_stride", _i32 * MAX_GROUPS),
                ("shapes", StepShape * MAX_SHAPES), ("part_o", _p), ("part_ml", _p), ("normed", _p), ("qkv", _p),
                ("attn", _p), ("mixed", _p), ("gate_up", _p), ("act", _p), ("ffn_out", _p), ("gemm_workspace", _p),
                ("gemm_workspace_bytes", _i64)]


class BlockArgs(ctypes.Structure):
    _fields_ = [("norm1_w", _p), ("norm2_w", _p), ("w_qkv", _p), ("b_qkv", _p), ("w_o", _p), ("b_o", _p),
                ("w_gate_up", _p), ("b_gate_up", _p), ("w_down", _p), ("b_down", _p), ("inv_freq", _p),
                ("k_pages", _p), ("v_pages", _p), ("eps1", _f), ("eps2", _f), ("scale", _f), ("rotary_dim", _i32),
                ("hidden", _i32), ("q_heads", _i32), ("kv_heads", _i32), ("head_dim", _i32), ("intermediate", _i32),
                ("window", _i32), ("group", _i32), ("shape", _i32), ("kind", _i32)]


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _bf16_matrix(t: Any, rows: int, cols: int) -> bool:
    return (isinstance(t, torch.Tensor) and t.dtype == torch.bfloat16 and t.is_cuda and t.dim() == 2
            and tuple(t.shape) == (rows, cols) and t.is_contiguous() and t.data_ptr() % 16 == 0)


def _bf16_vector(t: Any, n: int) -> bool:
    return t is None or (isinstance(t, torch.Tensor) and t.dtype == torch.bfloat16 and t.is_cuda
                         and tuple(t.shape) == (n,) and t.is_contiguous())


class NativeBlocks:
    """The model's schedule as an array of :class:`BlockArgs`, bound to one list of layer caches."""

    def __init__(self, blocks: Sequence[dict], caches: Sequence[Any], device: torch.device) -> None:
        self.device = device
        self.array = (BlockArgs * len(blocks))()
        # (head_dim, q_heads, kv_heads, whether a window is set: such layers' tiles are never cut), by shape index
        self.shapes: list[tuple[int, int, int, bool]] = []
        self.plan_owners: list[int] = []                 # per shape, the first mixer of that shape
        self.keep = []                                   # tensors whose addresses the array holds
        self.widths = dict(hidden=0, qkv=0, attn=0, gate_up=0, act=0)
        for a, f, cache in zip(self.array, blocks, caches):
            shape = (f["head_dim"], f["q_heads"], f["kv_heads"], f["window"] > 0)
            if shape not in self.shapes:
                self.shapes.append(shape)
                self.plan_owners.append(f.get("plan_owner", 0))
            for name in ("norm1_w", "norm2_w", "w_qkv", "b_qkv", "w_o", "b_o", "w_gate_up", "b_gate_up", "w_down",
                         "b_down", "inv_freq"):
                setattr(a, name, _ptr(f[name]))
                self.keep.append(f[name])
            a.k_pages, a.v_pages = cache.k_pages.data_ptr(), cache.v_pages.data_ptr()
            self.keep += [cache.k_pages, cache.v_pages]
            for name in ("eps1", "eps2", "scale", "rotary_dim", "hidden", "q_heads", "kv_heads", "head_dim",
                         "intermediate", "window"):
                setattr(a, name, f[name])
            a.group, a.shape, a.kind = cache.group, self.shapes.index(shape), f["kind"]
            d, qh, kvh, _ = shape
            w = self.widths
            w["hidden"] = max(w["hidden"], f["hidden"])
            w["qkv"] = max(w["qkv"], (qh + 2 * kvh) * d)
            w["attn"] = max(w["attn"], qh * d)
            w["gate_up"] = max(w["gate_up"], 2 * f["intermediate"])
            w["act"] = max(w["act"], f["intermediate"])

    @staticmethod
    def build(model: Any, caches: Sequence[Any]) -> Optional["NativeBlocks"]:
        """``None`` unless every schedule entry is a block that describes itself and writes a
        paged cache of its own."""
        if not model.rt.is_bf16 or not model.spec.schedule:
            return None
        fields = []
        for entry, cache in zip(model.spec.schedule, caches):
            layer = model.layers[entry.layer]
            f = layer.block.native_fields(layer.parts)
            if (f is None or not isinstance(f.get("kind"), int) or cache is None or cache.kind != "paged" or not cache.writable
                    or not 0 <= cache.group < MAX_GROUPS or cache.window != f["window"]):
                return None
            kvh, d = f["kv_heads"], f["head_dim"]
            if (cache.k_pages.dtype != torch.bfloat16 or tuple(cache.k_pages.shape[1:]) != (kvh, cache.k_pages.shape[2], d)
                    or not ops.attention_mfma_supports(d, cache.k_pages.shape[2], torch.bfloat16)):
                return None
            fields.append(f)
        native = NativeBlocks(fields, caches, model.rt.device)
        return native if len(native.shapes) <= MAX_SHAPES else None

    def run(self, x: torch.Tensor, ctx: Any) -> Optional[torch.Tensor]:
        """All blocks on the residual stream ``x [rows, hidden]`` (updated in place). Returns the
        last block's feed-forward output, which the caller's final norm adds to ``x``; ``None`` if
        the library has no kernel for one of the products at this number of rows (nothing ran)."""
        n = ctx.num_tokens
        if x.dtype != torch.bfloat16 or tuple(x.shape) != (n, self.widths["hidden"]) or not x.is_contiguous():
            return None
        if len(ctx.groups) > MAX_GROUPS:
            return None
        w = self.widths
        sizes = [n * w["hidden"], n * w["qkv"], n * w["attn"], n * w["hidden"], n * w["gate_up"], n * w["act"],
                 n * w["hidden"]]
        starts, at = [], 0
        for size in sizes:
            starts.append(at)
            at += -(-size // 16) * 16                      # every buffer starts on a 32-byte boundary
        scratch = torch.empty(at, device=self.device, dtype=torch.bfloat16)
        base = scratch.data_ptr()
        s = StepArgs()
        s.rows, s.num_decode, s.num_entries, s.page_size = n, ctx.num_decode, ctx.num_entries, ctx.page_size
        s.device = self.device.index if self.device.index is not None else torch.cuda.current_device()
        s.positions, s.q_start, s.kv_len = ctx.positions.data_ptr(), ctx.q_start.data_ptr(), ctx.kv_len.data_ptr()
        for g, grp in enumerate(ctx.groups):
            s.slots[g], s.block_tables[g] = grp.slots.data_ptr(), grp.block_tables.data_ptr()
            s.table_stride[g] = grp.block_tables.stride(0)
        nd = ctx.num_decode
        parts_o = parts_ml = 0
        keep = [scratch]
        for i, (d, qh, kvh, windowed) in enumerate(self.shapes):
            sh = s.shapes[i]
            if ctx.num_entries > nd:
                t = prefill_tiles(ctx, d, qh, kvh, nd, self.device, window=1 if windowed else 0)
                sh.tile_entry, sh.tile_q0, sh.tiles = t.entry.data_ptr(), t.q0.data_ptr(), t.tiles
                if t.cut is not None:
                    sh.tile_cut, sh.cut_tiles, sh.cut_room = t.cut.data_ptr(), t.cut_tiles, t.cut_room
                    sh.cut_buf, sh.cut_count = t.cut_buf.data_ptr(), t.cut_count.data_ptr()
            if nd > 0:
                # mixers of one shape plan alike, so the first one's answer for a recorded step holds for all
                splits = step_splits(ctx, nd, qh, kvh, self.device, ctx.decode_plans.get(self.plan_owners[i]))
                sh.decode_splits = splits
                if splits > 1:
                    parts_o = max(parts_o, nd * qh * splits * d)
                    parts_ml = max(parts_ml, nd * qh * splits * 2)
        if parts_o:
            part_o = torch.empty(parts_o, device=self.device, dtype=torch.float32)
            part_ml = torch.empty(parts_ml, device=self.device, dtype=torch.float32)
            s.part_o, s.part_ml = part_o.data_ptr(), part_ml.data_ptr()
            keep += [part_o, part_ml]
        (s.normed, s.qkv, s.attn, s.mixed, s.gate_up, s.act, s.ffn_out) = [base + 2 * st for st in starts]
        workspace, nbytes = ops.gemm_workspace(self.device)
        s.gemm_workspace, s.gemm_workspace_bytes = workspace.data_ptr(), nbytes
        if not ops.prenorm_blocks(x, self.array, len(self.array), s):
            return None
        ffn_out = scratch[starts[6]:starts[6] + n * w["hidden"]].view(n, w["hidden"])
        return ffn_out
