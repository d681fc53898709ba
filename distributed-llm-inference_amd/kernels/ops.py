"""Typed wrappers around the library's ``extern "C"`` entry points.

Every wrapper checks on the host that the operands have the device, type, layout and sizes that
its kernel and launch grid assume, and raises :class:`KernelArgumentError` otherwise: a kernel is
never launched on operands it was not written for. torch supplies device memory and the current
stream; nothing here computes with torch.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import build

_c_int, _c_i64, _c_float, _c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class KernelArgumentError(ValueError):
    """Operands that a kernel does not take."""


class KernelLaunchError(RuntimeError):
    """The HIP runtime refused a launch."""


_SIGNATURES = {
    "dli_embedding": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_rms_norm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_silu_mul": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_add": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_gather_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_to_float": [_c_ptr, _c_ptr, _c_i64, _c_int, _c_ptr],
    "dli_copy_pages": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_i64, _c_i64, _c_int, _c_ptr],
    "dli_fill": [_c_ptr, _c_float, _c_i64, _c_int, _c_ptr],
    "dli_skinny4_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr,
                         _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_skinny4_tile_features": [_c_int, _c_int],
    "dli_rope_kv_write": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                          _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_gemm_f32_nt": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int,
                        _c_int, _c_int, _c_ptr],
    "dli_sample": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                   _c_ptr],
    "dli_sample_scratch_per_row": [],
    "dli_sample_and_advance": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                               _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                               _c_int, _c_ptr],
    "dli_decode_advance": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                           _c_int, _c_int, _c_ptr],
    "dli_skinny_gemm_max_rows": [],
    "dli_skinny_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr,
                        _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_skinny_gemm_qkv_rope": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_ptr],
    "dli_head_gemm_supports": [_c_int, _c_int, _c_int],
    "dli_head_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int,
                      _c_int, _c_ptr, _c_ptr, _c_ptr],
    "dli_head_gemm_workgroups": [_c_int, _c_int],
    "dli_skinny_gemm_merged": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_int,
                               _c_int, _c_int, _c_ptr],
    "dli_mid_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_int,
                     _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_mid_finish_residual": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_mid_finish_residual_normed": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_i64,
                                       _c_int, _c_int, _c_ptr],
    "dli_mid_finish_qkv": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int,
                           _c_int, _c_int, _c_int, _c_ptr],
    "dli_gemm_bf16": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64,
                      _c_int, _c_ptr],
    "dli_gemm_bf16_f32": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64,
                      _c_int, _c_ptr],
    "dli_gemm_bf16_usable": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_i64, _c_int],
    "dli_prenorm_blocks_bf16": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr],
    "dli_embedding_ssq": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_attention_generic_tile_rows": [_c_int],
    "dli_attention_mfma_supports": [_c_int, _c_int],
    "dli_attention_prefill_tile_rows": [_c_int, _c_int, _c_int],
    "dli_attention_decode_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_self_merging_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr,
                                               _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                               _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_partial_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_bf16_static": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int,
                                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_rope_angles": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_attention_prefill_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                   _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                                   _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "dli_attention_prefill_cut_floats": [_c_int, _c_int, _c_int],
    "dli_attention_prefill_max_cuts": [],
    "dli_attention_generic": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr,
                              _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                              _c_int, _c_int, _c_ptr],
}

_lib: Optional[ctypes.CDLL] = None


def library() -> ctypes.CDLL:
    """The loaded HIP library with argument types declared (compiled at the first call if absent)."""
    global _lib
    if _lib is None:
        lib = build.load()
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name, None)
            if fn is None:
                raise build.KernelBuildError(f"{build.loaded_path()} lacks the entry point {name}")
            fn.argtypes = argtypes
            fn.restype = _c_int
        _lib = lib
    return _lib


def _check(status: int, name: str) -> None:
    if status == 0:
        return
    if status == -1:
        raise KernelArgumentError(f"{name}: the kernel does not take these sizes")
    raise KernelLaunchError(f"{name}: launch failed (status {status})")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> _c_ptr:
    """The current stream's handle. The raw getter skips the Stream object that
    ``torch.cuda.current_stream()`` builds at every call (a hundred calls a step)."""
    if _raw_stream is not None:
        return _c_ptr(_raw_stream(torch.cuda.current_device()))
    return _c_ptr(torch.cuda.current_stream().cuda_stream)


def _is_bf16(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return 1
    if dtype == torch.float32:
        return 0
    raise KernelArgumentError(f"activation type {dtype} is neither float32 nor bfloat16")


def _ptr(t: Optional[torch.Tensor]) -> _c_ptr:
    return _c_ptr(0 if t is None else t.data_ptr())


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def _dense(t: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None, ndim: Optional[int] = None) -> None:
    # the messages are put together only when a check fails: this runs hundreds of times a step
    if t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype) and (ndim is None or t.dim() == ndim):
        return
    _require(t.is_cuda, f"{name} is not on the GPU")
    _require(t.is_contiguous(), f"{name} is not contiguous")
    _require(dtype is None or t.dtype == dtype, f"{name} has type {t.dtype}, expected {dtype}")
    _require(ndim is None or t.dim() == ndim, f"{name} has {t.dim()} dimensions, expected {ndim}")


def _rows(t: torch.Tensor, name: str, dtype: torch.dtype) -> None:
    """A 2-D operand whose rows are contiguous (a row stride larger than the width is allowed)."""
    if t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1] and t.dtype == dtype:
        return
    _require(t.is_cuda, f"{name} is not on the GPU")
    _require(t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1],
             f"{name} is not a matrix with contiguous rows")
    _require(t.dtype == dtype, f"{name} has type {t.dtype}, expected {dtype}")


# ----------------------------------------------------------------------------- element-wise

def embedding(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """``out[t] = table[ids[t]]``; ids int32 and already checked against the table's rows."""
    _dense(table, "table", ndim=2)
    _dense(ids, "ids", torch.int32, 1)
    _dense(out, "out", table.dtype, 2)
    _require(out.shape == (ids.shape[0], table.shape[1]), "out must be [len(ids), width]")
    _check(library().dli_embedding(_ptr(table), _ptr(ids), _ptr(out), ids.shape[0], table.shape[1],
                                   _is_bf16(table.dtype), _stream()), "embedding")


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, sum_out: Optional[torch.Tensor] = None) -> None:
    """``out = weight * cast(x * rsqrt(mean(x^2) + eps))``. With ``delta``: x is first replaced by
    ``x + delta`` (written to ``sum_out``, which may be ``x`` itself)."""
    _dense(x, "x", ndim=2)
    _dense(weight, "weight", torch.float32, 1)
    _dense(out, "out", x.dtype, 2)
    _require(weight.shape[0] == x.shape[1], "weight length differs from the row width")
    _require(out.shape == x.shape, "out differs from x in shape")
    if delta is not None:
        _dense(delta, "delta", x.dtype, 2)
        _require(sum_out is not None, "delta needs sum_out")
        _dense(sum_out, "sum_out", x.dtype, 2)
        _require(delta.shape == x.shape and sum_out.shape == x.shape, "delta/sum_out differ from x in shape")
    _check(library().dli_rms_norm(_ptr(x), _ptr(delta), _ptr(weight), _ptr(sum_out), _ptr(out), x.shape[0],
                                  x.shape[1], float(eps), _is_bf16(x.dtype), _stream()), "rms_norm")


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """``out = silu(gate_up[:, :I]) * gate_up[:, I:]``."""
    _dense(gate_up, "gate_up", ndim=2)
    _dense(out, "out", gate_up.dtype, 2)
    _require(gate_up.shape[1] == 2 * out.shape[1] and gate_up.shape[0] == out.shape[0],
             "gate_up must be [rows, 2*I] for out [rows, I]")
    _check(library().dli_silu_mul(_ptr(gate_up), _ptr(out), out.shape[0], out.shape[1],
                                  _is_bf16(out.dtype), _stream()), "silu_mul")


def add(a: torch.Tensor, b: Optional[torch.Tensor], out: torch.Tensor,
        bias: Optional[torch.Tensor] = None) -> None:
    """``out = (a + bias) + b``; sums in 32-bit. ``out`` may alias ``a`` or ``b``."""
    _dense(a, "a", ndim=2)
    _dense(out, "out", a.dtype, 2)
    _require(out.shape == a.shape, "out differs from a in shape")
    if b is not None:
        _dense(b, "b", a.dtype, 2)
        _require(b.shape == a.shape, "b differs from a in shape")
    if bias is not None:
        _dense(bias, "bias", a.dtype, 1)
        _require(bias.shape[0] == a.shape[1], "bias length differs from the row width")
    _check(library().dli_add(_ptr(a), _ptr(b), _ptr(bias), _ptr(out), a.shape[0], a.shape[1],
                             _is_bf16(a.dtype), _stream()), "add")


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """``out[i] = x[rows[i]]``; rows int32, already checked against x's rows."""
    _dense(x, "x", ndim=2)
    _dense(rows, "rows", torch.int32, 1)
    _dense(out, "out", x.dtype, 2)
    _require(out.shape == (rows.shape[0], x.shape[1]), "out must be [len(rows), width]")
    _check(library().dli_gather_rows(_ptr(x), _ptr(rows), _ptr(out), rows.shape[0], x.shape[1],
                                     _is_bf16(x.dtype), _stream()), "gather_rows")


def to_float(x: torch.Tensor, out: torch.Tensor) -> None:
    _dense(x, "x")
    _dense(out, "out", torch.float32)
    _require(out.numel() == x.numel(), "out differs from x in size")
    _check(library().dli_to_float(_ptr(x), _ptr(out), x.numel(), _is_bf16(x.dtype), _stream()), "to_float")


def fill(x: torch.Tensor, value: float) -> None:
    _dense(x, "x")
    _check(library().dli_fill(_ptr(x), float(value), x.numel(), _is_bf16(x.dtype), _stream()), "fill")


def copy_pages(pool: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """Copy page ``src[i]`` onto page ``dst[i]`` in every layer, keys and values.

    ``pool`` is ``[layers, 2, pages, ...]`` (or ``[layers, 1, pages, ...]`` where keys and values
    live in tensors of their own); the page ids are int32 and already range-checked.
    """
    _dense(pool, "pool")
    _require(pool.dim() >= 4 and pool.shape[1] in (1, 2), "pool must be [layers, 1 or 2, pages, ...]")
    _dense(src, "src", torch.int32, 1)
    _dense(dst, "dst", torch.int32, 1)
    _require(src.shape == dst.shape, "src and dst differ in length")
    pages = pool.shape[2]
    page_elems = pool[0, 0, 0].numel()
    _check(library().dli_copy_pages(_ptr(pool), _ptr(src), _ptr(dst), src.shape[0], pool.shape[0] * pool.shape[1], pages,
                                    page_elems, _is_bf16(pool.dtype), _stream()), "copy_pages")


# ----------------------------------------------------------------------------- position + cache write

def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor],
                  rotary_dim: int, slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], q_heads: int, kv_heads: int, head_dim: int) -> None:
    """Rotate q (in place) and k, and write rotated k and raw v at each token's cache slot.

    ``qkv`` is ``[tokens, (q_heads + 2*kv_heads) * head_dim]``; ``k_pages`` is
    ``[pages, kv_heads, page_size, head_dim]`` and ``v_pages`` ``[pages, kv_heads, head_dim,
    page_size]``; ``slots[t] = page * page_size + offset`` (negative: the token is not cached).
    """
    _rows(qkv, "qkv", qkv.dtype)
    n = qkv.shape[0]
    _require(qkv.shape[1] == (q_heads + 2 * kv_heads) * head_dim, "qkv width differs from (q+2kv)*head_dim")
    _dense(positions, "positions", torch.int32, 1)
    _require(positions.shape[0] == n, "positions differ from qkv in rows")
    page_size = 1
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32, 1)
        _require(inv_freq.shape[0] * 2 == rotary_dim, "inv_freq must hold rotary_dim/2 frequencies")
    if kv_heads > 0:
        _require(slots is not None and k_pages is not None and v_pages is not None,
                 "kv heads need slots and pages")
        _dense(slots, "slots", torch.int32, 1)
        _require(slots.shape[0] == n, "slots differ from qkv in rows")
        _dense(k_pages, "k_pages", qkv.dtype, 4)
        _dense(v_pages, "v_pages", qkv.dtype, 4)
        page_size = k_pages.shape[2]
        _require(k_pages.shape[1] == kv_heads and k_pages.shape[3] == head_dim,
                 "k_pages must be [pages, kv_heads, page_size, head_dim]")
        _require(v_pages.shape == (k_pages.shape[0], kv_heads, head_dim, page_size),
                 "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _check(library().dli_rope_kv_write(
        _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(inv_freq), rotary_dim, _ptr(slots), _ptr(k_pages),
        _ptr(v_pages), n, q_heads, kv_heads, head_dim, page_size, _is_bf16(qkv.dtype), _stream()),
        "rope_kv_write")


# ----------------------------------------------------------------------------- matrix products

def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
             residual: Optional[torch.Tensor] = None) -> None:
    """``out = a @ w.T (+ bias) (+ residual)`` in IEEE single precision; ``w`` is ``[n, k]``."""
    _rows(a, "a", torch.float32)
    _rows(w, "w", torch.float32)
    _rows(out, "out", torch.float32)
    m, k = a.shape
    n = w.shape[0]
    _require(w.shape[1] == k, "a and w differ in inner size")
    _require(out.shape == (m, n), "out must be [rows of a, rows of w]")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == n, "bias length differs from rows of w")
    ldr = 0
    if residual is not None:
        _rows(residual, "residual", torch.float32)
        _require(residual.shape == (m, n), "residual differs from out in shape")
        ldr = residual.stride(0)
    _check(library().dli_gemm_f32_nt(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(bias), _ptr(residual),
                                     ldr, _ptr(out), out.stride(0), m, n, k, _stream()), "gemm_f32")


SKINNY_STORE, SKINNY_SWIGLU, SKINNY_RESIDUAL, SKINNY_F32 = 0, 1, 2, 3


def skinny_gemm_supports(rows: int, k: int, dtype: torch.dtype) -> bool:
    """Whether the decode product kernel takes ``rows`` activation rows of width ``k``."""
    return dtype == torch.bfloat16 and 0 < rows <= 64 and k > 0 and k % 32 == 0


def skinny_gemm_shape(n: int, k: int, tiled: bool = False, units: int = 256) -> int:
    """Workgroup shape for ``n`` output features of depth ``k``: with few tiles of 16 features the
    waves of a workgroup split k, with many they split the tiles so that the activations are read
    once per 8 tiles. From cold-cache timings on MI355X (``units`` compute units); with tiled
    weights at the 1B, 1.7B and 3B sizes: four k-waves on one tile each where the tiles are no
    more than the compute units or fill them evenly with short rows (6.5 us against 6.8 and 7.4
    for q/k/v at the 1B sizes, 16.2 against 16.8 for gate and up), else on two tiles each, which
    halves the workgroups and with them the uneven last round (11.5 us against 13.9 for q/k/v
    at the 3B sizes, 8.6 against 10.1 at the 1.7B sizes)."""
    tiles = -(-n // 16)
    if tiled:
        if tiles >= 2048 and k >= 3072:
            return 2   # a vocabulary with long rows: no split of k
        if tiles <= units or (tiles % units == 0 and k <= 2048):
            return 0
        return 4
    if tiles >= 768:   # a vocabulary
        return 3
    return 1 if k >= 4096 else 0


def tiled_weights_help(w_rows: int, k: int, epilogue: int, device: torch.device) -> bool:
    """Whether a second copy of a ``[w_rows, k]`` weight in tile order (:func:`tile_weights`)
    would be used: the sizes allow it and steps of 5 to 16 rows run this product on the
    16x16-tile kernel."""
    n = w_rows // 2 if epilogue == SKINNY_SWIGLU else w_rows
    if k % 128 != 0 or n % 16 != 0 or n == 0:
        return False
    return skinny_gemm_plan(8, n, k, epilogue, device)[0] == "tiles16"


def tile_weights(w: torch.Tensor, whole_blocks: bool = True) -> torch.Tensor:
    """``w [n, k]`` (bfloat16, n % 16 == 0, k % 128 == 0) in the order in which the 16x16-tile
    kernel's lanes read it: ``t[tile][block][q][g][c][8] = w[16*tile + c][128*block + 32*g + 8*q + ...]``,
    so that each load of a wave is 1 KB of consecutive memory. Same number of elements, flat.
    ``whole_blocks=False`` takes any k % 8 == 0 and fills the last block of 128 with zeros (the copy
    then has ``n * padded_k(k)`` elements; only :func:`mid_gemm` reads such a copy)."""
    _dense(w, "w", torch.bfloat16, 2)
    n, k = w.shape
    if k % 128 != 0 and not whole_blocks:
        _require(k % 8 == 0, "tile order needs k % 8 == 0")
        w = torch.nn.functional.pad(w, (0, padded_k(k) - k))
        k = w.shape[1]
    _require(n % 16 == 0 and k % 128 == 0, "tile order needs n % 16 == 0 and k % 128 == 0")
    t = w.view(n // 16, 16, k // 128, 4, 4, 8)       # tile, c, block, g, q, 8
    return t.permute(0, 2, 4, 3, 1, 5).contiguous().view(-1)


def padded_k(k: int) -> int:
    """``k`` rounded up to whole blocks of 128."""
    return -(-k // 128) * 128


_compute_units: dict[int, int] = {}


def compute_units(device: torch.device) -> int:
    """Compute units of the device (256 on MI355X)."""
    return _units(device)


def _units(device: torch.device) -> int:
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _compute_units:
        _compute_units[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _compute_units[index]


def skinny_gemm_plan(rows: int, n: int, k: int, epilogue: int, device: torch.device,
                     blocks4: Optional[int] = None, tiled: bool = False) -> tuple[str, int, int]:
    """How :func:`skinny_gemm` runs a product: ``(kernel, shape, parts)``.

    ``"blocks4"`` is the 4x4-block kernel (at most 16 rows), ``"tiles16"`` the 16x16-tile kernel
    (at most 64 rows); ``shape`` is that kernel's workgroup shape. ``parts`` is the number of parts
    that the residual epilogue leaves of each row's sum of squares. The choice follows cold-cache
    timings on MI355X: the block kernel reads whole cache lines of the weights and only the rows of
    activations that exist, which wins for one to four rows; with more rows the activations'
    traffic grows and the tile kernel, which reads them once per 16 features, is ahead.
    ``tiled``: a copy of the weights in tile order is at hand (at most 16 rows); the tile kernel
    then reads whole lines too and takes over from two rows on, and below that where the
    product has few features.
    """
    if blocks4 is None and rows <= 16 and k % 8 == 0:
        # long rows and so few features that tiles of 16 would leave half the compute units idle
        # (2048 at the 1B sizes; not 3072 at the 3B sizes, where the tile kernel is ahead from 4 rows on)
        deep = k >= 4096 and -(-n // 16) * 2 <= _units(device)
        if deep:
            blocks4 = 1   # (the shape of 16 k-waves was ahead for one to four rows until the loads of
            #               a wave's chunks overlapped: now 9.8 against 10.8 us for down at the 1B sizes)
        elif rows <= 4:
            out_feats = n * (2 if epilogue == SKINNY_SWIGLU else 1)
            few = out_feats <= 16 * _units(device)
            if not (tiled and (rows >= 2 or few)):
                blocks4 = 1 if few else 0
    if blocks4 is not None:
        feats = int(library().dli_skinny4_tile_features(blocks4, epilogue))
        return "blocks4", blocks4, -(-n // feats)
    shape = skinny_gemm_shape(n, k, tiled and rows <= 16, _units(device))
    if tiled and rows <= MERGED_ROWS and shape == 0 and -(-n // 16) <= _units(device):
        # Few tiles and very few rows: eight k-waves are as fast as four (4.3 against 4.4 us for o at
        # the 1B sizes), and the o projection that merges the attention's runs of keys itself, whose
        # waves each merge the k they multiply, is faster with them; it has to add in the same order
        # as this one to give the same bits.
        shape = 1
    return "tiles16", shape, -(-n // 16)


def skinny_gemm(x: torch.Tensor, w: torch.Tensor, *, epilogue: int, out: Optional[torch.Tensor] = None,
                bias: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
                ssq_in: Optional[torch.Tensor] = None, stream: Optional[torch.Tensor] = None,
                ssq_out: Optional[torch.Tensor] = None, shape: Optional[int] = None,
                blocks4: Optional[int] = None, w_tiled: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``y = xhat @ w.T`` for at most 64 rows of bfloat16 ``x``, with fused surroundings.

    ``norm_w``/``eps``/``ssq_in [parts, rows]``: xhat is the RMSNorm of x, the row sums of squares
    being given in parts. Epilogues: ``SKINNY_STORE`` (``out`` bfloat16 ``[rows, n]``),
    ``SKINNY_SWIGLU`` (``w`` is ``[2n, k]``: gate rows then up rows; ``out [rows, n]`` gets
    ``silu(gate) * up``), ``SKINNY_RESIDUAL`` (``stream [rows, n]`` becomes ``stream + y`` in place;
    the parts of its row sums of squares are returned as ``[parts, rows]``, in ``ssq_out`` if that
    is given with the shape :func:`skinny_gemm_plan` names), ``SKINNY_F32`` (``out`` float32).
    ``shape`` forces the 16x16-tile kernel with that workgroup shape, ``blocks4`` the 4x4-block
    kernel with that one (at most 16 rows). ``w_tiled``: the same weights in tile order
    (:func:`tile_weights`), read instead of ``w`` when the 16x16-tile kernel runs at most 16 rows.
    """
    _rows(x, "x", torch.bfloat16)
    _dense(w, "w", torch.bfloat16, 2)
    m, k = x.shape
    _require(w.shape[1] == k, "x and w differ in inner size")
    _require(skinny_gemm_supports(m, k, x.dtype), f"the decode product takes 1..64 rows and k % 32 == 0, not {m} x {k}")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    n = w.shape[0] // 2 if epilogue == SKINNY_SWIGLU else w.shape[0]
    up_offset = n if epilogue == SKINNY_SWIGLU else 0
    if epilogue == SKINNY_SWIGLU:
        _require(w.shape[0] == 2 * n, "swiglu needs gate rows and up rows")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == w.shape[0], "bias length differs from rows of w")
    if k % 128 != 0:
        w_tiled = None   # a copy in whole blocks with a zero-filled last one: the 17-to-64-row kernel's alone
    if shape is not None:
        _require(shape in (0, 1, 2, 3, 4), "shape must be 0..4")
        kernel, a, n_parts = "tiles16", shape, -(-n // 16)
    else:
        if blocks4 is not None:
            _require(blocks4 in (0, 1, 2) and m <= 16 and k % 8 == 0, "blocks4 must be 0..2, with at most 16 rows")
        kernel, a, n_parts = skinny_gemm_plan(m, n, k, epilogue, x.device, blocks4,
                                              tiled=w_tiled is not None and m <= 16)
    tiled = w_tiled is not None and kernel == "tiles16" and m <= 16
    if tiled:
        _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
        _require(w_tiled.numel() == w.numel() and k % 128 == 0 and n % 16 == 0 and w_tiled.data_ptr() % 16 == 0,
                 "w_tiled must hold the same weights in tile order (n % 16 == 0, k % 128 == 0)")
    parts = 0
    if norm_w is not None:
        _require(epilogue != SKINNY_RESIDUAL, "the residual epilogue takes no fused norm")
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    ldo = lds = 0
    if epilogue == SKINNY_RESIDUAL:
        _require(stream is not None, "the residual epilogue needs stream")
        _rows(stream, "stream", torch.bfloat16)
        _require(stream.shape == (m, n), "stream must be [rows, n]")
        if ssq_out is None:
            ssq_out = torch.empty(n_parts, m, device=x.device, dtype=torch.float32)
        _dense(ssq_out, "ssq_out", torch.float32, 2)
        _require(ssq_out.shape == (n_parts, m), f"ssq_out must be [{n_parts}, rows] for this product")
        _require(stream.data_ptr() % 8 == 0, "stream must be 8-byte aligned")
        lds = stream.stride(0)
    else:
        _require(out is not None, "this epilogue needs out")
        _rows(out, "out", torch.float32 if epilogue == SKINNY_F32 else torch.bfloat16)
        _require(out.shape == (m, n), "out must be [rows, n]")
        _require(out.data_ptr() % 16 == 0, "out must be 16-byte aligned")
        ldo = out.stride(0)
    if kernel == "tiles16":
        _check(library().dli_skinny_gemm(
            _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled if tiled else w),
            _ptr(bias), _ptr(out), ldo, _ptr(stream), lds, _ptr(ssq_out), m, n, k, up_offset, epilogue, a,
            int(tiled), _stream()), "skinny_gemm")
    else:
        _check(library().dli_skinny4_gemm(
            _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w), _ptr(bias), _ptr(out), ldo,
            _ptr(stream), lds, _ptr(ssq_out), m, n, k, up_offset, epilogue, a, _stream()), "skinny4_gemm")
    return ssq_out if epilogue == SKINNY_RESIDUAL else None


def head_gemm_supports(rows: int, n: int, k: int, dtype: torch.dtype) -> bool:
    """Whether :func:`head_gemm` takes this product (at most 16 rows, ``n % 16 == 0``, ``k`` one
    of 1024, 2048, 3072, 4096)."""
    return dtype == torch.bfloat16 and bool(library().dli_head_gemm_supports(int(rows), int(n), int(k)))


def head_gemm(x: torch.Tensor, w_tiled: torch.Tensor, out: torch.Tensor, norm_w: Optional[torch.Tensor] = None,
              eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None, workgroups: int = 0,
              best: Optional[tuple[torch.Tensor, torch.Tensor]] = None) -> int:
    """``out = xhat @ w.T`` as float32 for at most 16 rows and the many rows of a vocabulary:
    workgroups that stay for the whole launch walk the tiles of ``w_tiled`` (:func:`tile_weights`
    of ``w [n, k]``) in turn, each wave keeping its normalised activations in registers. ``norm_w``,
    ``eps``, ``ssq_in [parts, rows]``: the RMSNorm of ``x`` as in :func:`skinny_gemm`. The sums are
    those of :func:`skinny_gemm` with ``shape=4``, to the bit. ``workgroups``: how many (0: one per
    compute unit). ``best``: float32 values and int32 indices (the scratch of :func:`sample_scratch`); each
    workgroup then leaves every row's best logit and its lowest index among the logits it made, as
    ``[rows, parts]`` at the start of both, and the number of parts comes back (the first stage of
    :func:`sample_and_advance`'s argmax); without it 0."""
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _rows(out, "out", torch.float32)
    n = out.shape[1]
    _require(out.shape[0] == m, "out must be [rows, n]")
    _require(head_gemm_supports(m, n, k, x.dtype), f"the logits kernel takes 1..16 rows, n % 16 == 0 and k of 1024 to "
             f"4096 in steps of 1024, not {m} x {k} -> {n}")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [n, k] in tile order")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and out.stride(0) % 4 == 0 and out.data_ptr() % 16 == 0,
             "operands must be 16-byte aligned")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    groups = 0
    if best is not None:
        groups = int(library().dli_head_gemm_workgroups(n, int(workgroups)))
        _dense(best[0], "best values", torch.float32)
        _dense(best[1], "best indices", torch.int32)
        _require(best[0].numel() >= m * groups and best[1].numel() >= m * groups, "the argmax's scratch is too small")
    _check(library().dli_head_gemm(_ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled),
                                   _ptr(out), out.stride(0), m, n, k, int(workgroups),
                                   _ptr(best[0]) if best is not None else None,
                                   _ptr(best[1]) if best is not None else None, _stream()), "head_gemm")
    return groups


MERGED_ROWS, MERGED_SPLITS, _MERGED_RANGE = 4, 16, 512  # csrc/skinny_gemm.hip: MERGE_ROWS, MERGE_SPLITS, MERGE_RANGE


def skinny_gemm_merged_supports(rows: int, n: int, heads: int, head_dim: int, splits: int,
                                device: torch.device) -> bool:
    """Whether :func:`skinny_gemm_merged` takes this o projection: few rows, few runs of keys, a
    product that the 16x16-tile kernel runs with k split over the waves of a workgroup."""
    k = heads * head_dim
    if not (0 < rows <= MERGED_ROWS and 2 <= splits <= MERGED_SPLITS and head_dim % 4 == 0 and k % 128 == 0
            and n % 16 == 0):
        return False
    return _merged_shape(rows, n, k, device) is not None


def _merged_shape(rows: int, n: int, k: int, device: torch.device) -> Optional[int]:
    """The workgroup shape (0: four k-waves, 1: eight) with which the merging o projection runs:
    that of the plain product with the residual sum, so that both add in the same order, or None
    if that one runs on another kernel or a wave's run of k does not fit the merge's buffer."""
    kernel, shape, _ = skinny_gemm_plan(rows, n, k, SKINNY_RESIDUAL, device, tiled=True)
    if kernel != "tiles16" or shape not in (0, 1):
        return None
    return shape if -(-(k // 128) // (4 if shape == 0 else 8)) * 128 <= _MERGED_RANGE else None


def skinny_gemm_merged(part_o: torch.Tensor, part_ml: torch.Tensor, splits: int, heads: int, head_dim: int,
                       w_tiled: torch.Tensor, stream: torch.Tensor, bias: Optional[torch.Tensor] = None,
                       ssq_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``stream += merge(part_o, part_ml) @ w.T (+ bias)`` for at most four rows: the o projection
    of a decode step fed with the partial results that :func:`attention_decode` leaves with
    ``merge=False`` (``part_o [rows, heads, splits, head_dim]``, ``part_ml [rows, heads, splits, 2]``),
    merged inside the product's kernel with the arithmetic of the merge kernel. Returns the parts
    of the rows' sums of squares like the residual epilogue of :func:`skinny_gemm`."""
    _rows(stream, "stream", torch.bfloat16)
    m, n = stream.shape
    k = heads * head_dim
    _require(skinny_gemm_merged_supports(m, n, heads, head_dim, splits, stream.device),
             f"the merging o projection takes 1..{MERGED_ROWS} rows and 2..{MERGED_SPLITS} runs of keys, "
             f"not {m} rows, {splits} runs, {heads} heads of {head_dim}")
    _dense(part_o, "part_o", torch.float32)
    _dense(part_ml, "part_ml", torch.float32)
    _require(part_o.numel() >= m * heads * splits * head_dim and part_ml.numel() >= m * heads * splits * 2,
             "partial-result buffers are too small")
    _require(part_o.data_ptr() % 16 == 0 and part_ml.data_ptr() % 8 == 0, "partial results must be 16-byte aligned")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [n, heads*head_dim] in tile order")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from rows of w")
    _, _, n_parts = skinny_gemm_plan(m, n, k, SKINNY_RESIDUAL, stream.device, tiled=True)
    shape = _merged_shape(m, n, k, stream.device)
    if ssq_out is None:
        ssq_out = torch.empty(n_parts, m, device=stream.device, dtype=torch.float32)
    _dense(ssq_out, "ssq_out", torch.float32, 2)
    _require(ssq_out.shape == (n_parts, m), f"ssq_out must be [{n_parts}, rows] for this product")
    _require(stream.data_ptr() % 8 == 0, "stream must be 8-byte aligned")
    _check(library().dli_skinny_gemm_merged(
        _ptr(part_o), _ptr(part_ml), int(splits), int(heads), int(head_dim), _ptr(w_tiled), _ptr(bias), _ptr(stream),
        stream.stride(0), _ptr(ssq_out), m, n, shape, _stream()), "skinny_gemm_merged")
    return ssq_out


_GEMM_WORKSPACE_BYTES = 64 << 20
_gemm_workspaces: dict[int, torch.Tensor] = {}


MID_PARTIAL, MID_SWIGLU, MID_STORE = 0, 1, 2
MID_ROWS = 64


def mid_gemm_supports(rows: int, k: int, dtype: torch.dtype) -> bool:
    """Whether the product kernel for decode steps of up to 64 rows takes this shape."""
    return dtype == torch.bfloat16 and 0 < rows <= MID_ROWS and k > 0 and k % 8 == 0


MID_SHAPES = ((4, 1), (4, 2))              # (waves, kwaves) that are built for the plain products
MID_SHAPES_GATED = ((2, 1), (2, 2), (2, 4))  # and for the gated one


def mid_gemm_plan(n: int, k: int, epilogue: int, units: int, rows: int = 64) -> tuple[int, int, int]:
    """``(waves, kwaves, splits)`` for a product of ``n`` output features of depth ``k``.

    A workgroup has ``waves`` feature tiles of 16 and ``kwaves`` waves on each, which split its
    range of k; ``splits`` workgroups share a feature tile's whole k (a gated product is never
    split: its epilogue needs whole sums). These launches last a few trips to memory, so the plan
    aims at one workgroup on every compute unit with eight to sixteen waves, each with few blocks
    of 128 k to fetch."""
    tiles, blocks = -(-n // 16), -(-k // 128)
    if epilogue == MID_SWIGLU:
        # (two against four k-waves a tile, cold weights: 21.1 and 21.4 us at 32 rows, 23.4 and 23.0
        # at 48, 28.7 and 26.1 at 64 at the 1B sizes; with k of 3072 24.8 and 24.5, 29.9 and 27.2, 37.4
        # and 31.9. In a decode step of 64 rows, where part of the weights is warm: 2.93 to 2.96 ms with
        # either at the 1B sizes, 5.48 against 5.39 ms at the 3B sizes. Four tiles a workgroup, or one,
        # were behind at every number of rows.)
        return 2, (4 if rows > 32 and blocks >= 24 else 2) if blocks >= 2 else 1, 1
    if epilogue == MID_STORE:
        return 4, 2 if blocks >= 2 else 1, 1
    waves = 4
    groups = -(-tiles // waves)
    splits = max(1, min(blocks, round(units / groups)))
    kwaves = 2 if blocks // splits >= 2 else 1
    return waves, kwaves, splits


def mid_tiles_help(w_rows: int, k: int, epilogue: int) -> bool:
    """Whether decode steps of 17 to 64 rows would read a copy of a ``[w_rows, k]`` weight in tile
    order (:func:`tile_weights`, of whole blocks of k, zero-filled): the layer products do, where
    the features tile."""
    n = w_rows // 2 if epilogue == SKINNY_SWIGLU else w_rows
    return epilogue in (SKINNY_STORE, SKINNY_SWIGLU, SKINNY_RESIDUAL) and k % 8 == 0 and n % 16 == 0 and n > 0


def mid_gemm(x: torch.Tensor, w: torch.Tensor, *, epilogue: int, tiled: bool = False, n: Optional[int] = None,
             out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
             norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None,
             splits: Optional[int] = None, waves: Optional[int] = None,
             kwaves: Optional[int] = None) -> torch.Tensor:
    """``y = xhat @ w.T`` for at most 64 rows of bfloat16 ``x [rows, k]``, k a multiple of 8.

    ``w`` is ``[n, k]`` (``[2n, k]``, gate rows then up rows, for ``MID_SWIGLU``), or the same in
    tile order (:func:`tile_weights`, flat; of whole blocks, zero-filled where k is no multiple
    of 128) with ``tiled`` and ``n`` given. ``norm_w``/``eps``/
    ``ssq_in [parts, rows]``: xhat is the RMSNorm of x. ``MID_PARTIAL`` returns float32
    ``[splits, rows, n]`` whose sum over the splits, in their order, is the product (no bias; the
    finishing kernels add them up); ``MID_STORE`` and ``MID_SWIGLU`` return bfloat16 ``[rows, n]``.
    """
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _require(mid_gemm_supports(m, k, x.dtype), f"this product takes 1..64 rows and k % 8 == 0, not {m} x {k}")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    sets = 2 if epilogue == MID_SWIGLU else 1
    if tiled:
        _dense(w, "w", torch.bfloat16, 1)
        _require(n is not None and n % 16 == 0 and w.numel() == sets * n * padded_k(k),
                 "tiled weights need n % 16 == 0 features of depth k, in whole blocks of 128")
    else:
        _dense(w, "w", torch.bfloat16, 2)
        _require(w.shape[1] == k and w.shape[0] % sets == 0, "x and w differ in inner size")
        n = w.shape[0] // sets
    _require(epilogue in (MID_PARTIAL, MID_SWIGLU, MID_STORE), "unknown epilogue")
    plan_waves, plan_kwaves, plan_splits = mid_gemm_plan(n, k, epilogue, _units(x.device), m)
    waves = plan_waves if waves is None else waves
    kwaves = plan_kwaves if kwaves is None else kwaves
    splits = plan_splits if splits is None else splits
    built = MID_SHAPES_GATED if epilogue == MID_SWIGLU else MID_SHAPES
    _require((waves, kwaves) in built and 1 <= splits <= -(-k // 128),
             f"(waves, kwaves) must be one of {built}, splits 1..k/128")
    if epilogue == MID_PARTIAL:
        _require(bias is None and n % 4 == 0, "partial products take no bias, n % 4 == 0")
        if out is None:
            out = torch.empty(splits, m, n, device=x.device, dtype=torch.float32)
        _dense(out, "out", torch.float32, 3)
        _require(out.shape == (splits, m, n), "out must be [splits, rows, n]")
        ldo = n
    else:
        _require(splits == 1, "only partial products are split")
        if out is None:
            out = torch.empty(m, n, device=x.device, dtype=torch.bfloat16)
        _rows(out, "out", torch.bfloat16)
        _require(out.shape == (m, n) and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0, "out must be [rows, n], rows 8-byte aligned")
        ldo = out.stride(0)
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == sets * n, "bias length differs from rows of w")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    _check(library().dli_mid_gemm(
        _ptr(x), x.stride(0), _ptr(ssq_in) if norm_w is not None else None, parts, _ptr(norm_w), float(eps), _ptr(w),
        int(tiled), _ptr(bias), _ptr(out), ldo, m, n, k, n if epilogue == MID_SWIGLU else 0, epilogue, splits, waves,
        kwaves, _stream()), "mid_gemm")
    return out


MID_NORMED_WIDTH = 8192  # the widest row that the normalising finish holds in one workgroup


def mid_finish_residual(partial: torch.Tensor, stream: torch.Tensor, bias: Optional[torch.Tensor] = None,
                        ssq_out: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                        eps: float = 0.0, normed_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``stream += sum over splits of partial (+ bias)`` in place (32-bit sum, the product rounded
    to bfloat16 first, as the fused epilogue of the few-row product does), and each row's sum of
    squares of the new stream, in parts of 1024 features, as float32 ``[parts, rows]`` for the norm
    that follows.

    With ``norm_w`` (float32 ``[n]``, ``n <= MID_NORMED_WIDTH``), ``eps`` and ``normed_out``
    (bfloat16 ``[rows, n]``) that norm is applied here as well: ``normed_out`` gets the RMSNorm of
    the new stream with the two roundings of the fused norm prologues, for a product that then
    reads it as it is; the sums of squares come back whole, as ``[1, rows]``."""
    _dense(partial, "partial", torch.float32, 3)
    _rows(stream, "stream", torch.bfloat16)
    splits, m, n = partial.shape
    _require(stream.shape == (m, n) and n % 4 == 0 and stream.stride(0) % 4 == 0 and stream.data_ptr() % 8 == 0,
             "stream must be [rows, n] with n % 4 == 0")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from n")
    parts = 1 if norm_w is not None else -(-n // 1024)
    if ssq_out is None:
        ssq_out = torch.empty(parts, m, device=stream.device, dtype=torch.float32)
    _dense(ssq_out, "ssq_out", torch.float32, 2)
    _require(ssq_out.shape == (parts, m), f"ssq_out must be [{parts}, rows]")
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == n and norm_w.data_ptr() % 16 == 0, "norm weight must have n aligned values")
        _require(n <= MID_NORMED_WIDTH, f"rows wider than {MID_NORMED_WIDTH} are normalised by the product that reads them")
        _require(normed_out is not None, "the normalised rows need normed_out")
        _rows(normed_out, "normed_out", torch.bfloat16)
        _require(normed_out.shape == (m, n) and normed_out.stride(0) % 4 == 0 and normed_out.data_ptr() % 8 == 0,
                 "normed_out must be [rows, n]")
        _check(library().dli_mid_finish_residual_normed(
            _ptr(partial), splits, _ptr(bias), _ptr(stream), stream.stride(0), _ptr(ssq_out), _ptr(norm_w), float(eps),
            _ptr(normed_out), normed_out.stride(0), m, n, _stream()), "mid_finish_residual")
        return ssq_out
    _check(library().dli_mid_finish_residual(_ptr(partial), splits, _ptr(bias), _ptr(stream), stream.stride(0),
                                             _ptr(ssq_out), m, n, _stream()), "mid_finish_residual")
    return ssq_out


def mid_finish_qkv(partial: torch.Tensor, out: torch.Tensor, angles: torch.Tensor, slots: torch.Tensor,
                   k_pages: torch.Tensor, v_pages: torch.Tensor, q_heads: int,
                   bias: Optional[torch.Tensor] = None) -> None:
    """The fused q/k/v projection's partial products ``[splits, rows, (q + 2 kv) * head_dim]``, in
    the feature order of :func:`tile_weights_qkv_rope` (``bias`` too): summed over the splits,
    rotated, q written to ``out[:, :q_heads * head_dim]`` in the usual order, rotated k and v into
    the cache pages at ``slots`` (negative: not cached). ``angles``: :func:`rope_angles`."""
    _dense(partial, "partial", torch.float32, 3)
    _rows(out, "out", torch.bfloat16)
    splits, m, n = partial.shape
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    _, kv_heads, page_size, head_dim = k_pages.shape
    _require(v_pages.shape == (k_pages.shape[0], kv_heads, head_dim, page_size), "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(head_dim % 16 == 0 and n == (q_heads + 2 * kv_heads) * head_dim, "partial width differs from (q + 2 kv) * head_dim")
    _require(out.shape[0] == m and out.shape[1] >= q_heads * head_dim and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0,
             "out must hold the q heads of every row")
    _dense(angles, "angles", torch.float32, 3)
    _require(angles.shape == (m, 2, head_dim // 2), "angles must be [rows, 2, head_dim / 2]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == m, "slots differ from partial in rows")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from the features")
    _check(library().dli_mid_finish_qkv(_ptr(partial), splits, _ptr(bias), _ptr(angles), _ptr(slots), _ptr(out),
                                        out.stride(0), _ptr(k_pages), _ptr(v_pages), m, q_heads, kv_heads, head_dim,
                                        page_size, _stream()), "mid_finish_qkv")


def gemm_workspace(device: torch.device) -> tuple[torch.Tensor, int]:
    """The device buffer that the vendor library's products may use, and its size in bytes."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    workspace = _gemm_workspaces.get(index)
    if workspace is None:
        workspace = _gemm_workspaces[index] = torch.empty(_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return workspace, _GEMM_WORKSPACE_BYTES


def prenorm_blocks(x: torch.Tensor, blocks, count: int, step) -> bool:
    """Run ``count`` pre-norm blocks (ctypes array of ``parts.native.BlockArgs``) on the residual
    stream ``x`` for the step described by ``step`` (``parts.native.StepArgs``), all launches
    issued from C. Whoever fills the structures has checked shapes and sizes. False, with nothing
    launched, where an argument or a product's shape is refused."""
    _rows(x, "x", torch.bfloat16)
    status = library().dli_prenorm_blocks_bf16(_ptr(x), ctypes.cast(blocks, ctypes.c_void_p), int(count),
                                               ctypes.cast(ctypes.pointer(step), ctypes.c_void_p), _stream())
    if status == -1:
        return False
    _check(status, "prenorm_blocks")
    return True


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None) -> bool:
    """``out = x @ w.T (+ bias)`` for bfloat16 matrices with contiguous rows through the vendor
    library, 32-bit accumulation, the bias added before the one rounding (``out`` float32: the
    sums as they are, unrounded). The library's choice
    of kernel is looked up once per shape. Returns False where the library has no kernel for the
    shape (nothing was computed then)."""
    _rows(x, "x", torch.bfloat16)
    _rows(w, "w", torch.bfloat16)
    _require(out.dtype in (torch.bfloat16, torch.float32), "out must be bfloat16 or float32")
    _rows(out, "out", out.dtype)
    rows, k = x.shape
    feats = w.shape[0]
    _require(w.shape[1] == k and out.shape == (rows, feats), "x [n, k], w [m, k] and out [n, m] do not fit")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == feats, "bias length differs from rows of w")
    index = x.device.index if x.device.index is not None else torch.cuda.current_device()
    workspace = _gemm_workspaces.get(index)
    if workspace is None:
        workspace = _gemm_workspaces[index] = torch.empty(_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    call = library().dli_gemm_bf16 if out.dtype == torch.bfloat16 else library().dli_gemm_bf16_f32
    status = call(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(bias), _ptr(out), out.stride(0),
                  rows, feats, k, _ptr(workspace), _GEMM_WORKSPACE_BYTES, index, _stream())
    if status == -1:
        return False
    _check(status, "gemm_bf16")
    return True


def qkv_rope_feature_order(q_heads: int, kv_heads: int, head_dim: int) -> torch.Tensor:
    """The order of the fused projection's features in which :func:`skinny_gemm_qkv_rope` wants
    its weights and bias: tile ``t`` of a q or k head holds the head's dimensions ``8t..8t+7`` and
    ``half+8t..half+8t+7`` (eight rotary pairs); v heads keep their order. int64 ``[features]``."""
    _require(head_dim % 16 == 0 and q_heads > 0 and kv_heads > 0, "heads of a multiple of 16 dimensions")
    half = head_dim // 2
    within = torch.tensor([(8 * (f // 16) + f % 8) + (half if f % 16 >= 8 else 0) for f in range(head_dim)])
    heads = []
    for h in range(q_heads + 2 * kv_heads):
        local = within if h < q_heads + kv_heads else torch.arange(head_dim)
        heads.append(h * head_dim + local)
    return torch.cat(heads)


def tile_weights_qkv_rope(w: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int) -> torch.Tensor:
    """The fused q/k/v matrix in tile order (:func:`tile_weights`) with the features in
    :func:`qkv_rope_feature_order`."""
    _dense(w, "w", torch.bfloat16, 2)
    _require(w.shape[0] == (q_heads + 2 * kv_heads) * head_dim, "w must hold the q, k and v heads")
    order = qkv_rope_feature_order(q_heads, kv_heads, head_dim).to(w.device)
    return tile_weights(w[order].contiguous(), whole_blocks=False)


def skinny_gemm_qkv_rope(x: torch.Tensor, w_tiled: torch.Tensor, q_out: torch.Tensor, angles: torch.Tensor,
                         slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, q_heads: int, *,
                         bias: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                         eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None,
                         shape: Optional[int] = None) -> None:
    """The fused q/k/v projection of at most 16 decode rows with rotation and cache write inside:
    ``q_out[row, head*head_dim + dim]`` (a ``[rows, >= q_heads*head_dim]`` bfloat16 buffer) gets the
    rotated queries; the rotated keys and the values go to the pages at ``slots[row]`` (negative:
    not cached). ``w_tiled`` comes from :func:`tile_weights_qkv_rope`, ``bias`` (optional) is in
    :func:`qkv_rope_feature_order`, ``angles [rows, 2, head_dim/2]`` from :func:`rope_angles`.
    ``norm_w``/``eps``/``ssq_in`` as in :func:`skinny_gemm`."""
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size), "v_pages must be [pages, kv_heads, head_dim, page_size]")
    n = (q_heads + 2 * kv_heads) * head_dim
    _require(0 < m <= 16 and k % 128 == 0 and head_dim % 16 == 0 and q_heads > 0,
             f"this product takes 1..16 rows, k % 128 == 0 and head_dim % 16 == 0, not {m} x {k}, {head_dim}")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [(q + 2 kv) * head_dim, k]")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "x must be 16-byte aligned")
    _rows(q_out, "q_out", torch.bfloat16)
    _require(q_out.shape[0] == m and q_out.shape[1] >= q_heads * head_dim and q_out.stride(0) % 8 == 0
             and q_out.data_ptr() % 16 == 0, "q_out must be [rows, >= q_heads * head_dim], 16-byte aligned")
    _dense(angles, "angles", torch.float32, 3)
    _require(angles.shape == (m, 2, head_dim // 2) and angles.data_ptr() % 16 == 0, "angles must be [rows, 2, head_dim/2]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == m, "one slot per row")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from the features")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    if shape is None:
        shape = skinny_gemm_shape(n, k, tiled=True, units=_units(x.device))
        if shape == 0:
            shape = 1  # with the rotation in its epilogue eight k-waves are ahead (7.0 against 7.7 us at the 1B sizes)
    _require(shape in (0, 1, 2, 3, 4), "shape must be 0..4")
    _check(library().dli_skinny_gemm_qkv_rope(
        _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled), _ptr(bias), _ptr(q_out),
        q_out.stride(0), _ptr(angles), _ptr(slots), _ptr(k_pages), _ptr(v_pages), m, k, q_heads, kv_heads, head_dim,
        page_size, shape, _stream()), "skinny_gemm_qkv_rope")


def embedding_ssq(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, ssq: torch.Tensor) -> None:
    """``out[t] = table[ids[t]]`` and ``ssq[0, t] = sum(out[t]^2)`` (bfloat16 table)."""
    _dense(table, "table", torch.bfloat16, 2)
    _dense(ids, "ids", torch.int32, 1)
    _dense(out, "out", torch.bfloat16, 2)
    _dense(ssq, "ssq", torch.float32, 2)
    _require(out.shape == (ids.shape[0], table.shape[1]) and ssq.shape == (1, ids.shape[0]),
             "out [len(ids), width], ssq [1, len(ids)]")
    _check(library().dli_embedding_ssq(_ptr(table), _ptr(ids), _ptr(out), _ptr(ssq), ids.shape[0], table.shape[1],
                                       _stream()), "embedding_ssq")

# ----------------------------------------------------------------------------- attention

def attention_generic_tile_rows(head_dim: int) -> int:
    rows = library().dli_attention_generic_tile_rows(head_dim)
    if rows <= 0:
        raise KernelArgumentError(
            f"attention takes head_dim in steps of 16 up to 256, not {head_dim}")
    return rows


def attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                      tile_entry: torch.Tensor, tile_q0: torch.Tensor, q_heads: int, scale: float,
                      window: int = 0) -> None:
    """Paged causal attention for a batch of portions (vector units, 32-bit arithmetic).

    ``q`` and ``out`` are ``[tokens, q_heads*head_dim]`` (rows contiguous, any row stride);
    ``q_start [entries+1]``, ``kv_len [entries]``, ``block_tables [entries, width]`` describe the
    requests; ``tile_entry/tile_q0`` list the query tiles of ``attention_generic_tile_rows`` rows.
    """
    _dense(k_pages, "k_pages", ndim=4)
    dtype = k_pages.dtype
    _rows(q, "q", dtype)
    _rows(out, "out", dtype)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", dtype, 4)
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size),
             "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(q.shape[1] == q_heads * head_dim and out.shape == q.shape, "q/out must be [tokens, q_heads*head_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    for name, t in (("q_start", q_start), ("kv_len", kv_len), ("tile_entry", tile_entry), ("tile_q0", tile_q0)):
        _dense(t, name, torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
    _check(library().dli_attention_generic(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start),
        _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0),
        tile_entry.shape[0], q_heads, kv_heads, head_dim, page_size, float(scale), int(window),
        _is_bf16(dtype), _stream()), "attention_generic")



def attention_mfma_supports(head_dim: int, page_size: int, dtype: torch.dtype) -> bool:
    """Whether the matrix-core attention kernels take this shape (else: the generic kernel)."""
    return dtype == torch.bfloat16 and bool(library().dli_attention_mfma_supports(head_dim, page_size))


def attention_prefill_tile_rows(head_dim: int, q_heads: int, kv_heads: int) -> int:
    """Queries per tile of the tile list that :func:`attention_prefill` expects for this shape."""
    rows = int(library().dli_attention_prefill_tile_rows(head_dim, q_heads, kv_heads))
    _require(rows > 0, "query heads are not a multiple of kv heads")
    return rows


def attention_prefill_cut_floats(head_dim: int, q_heads: int, kv_heads: int) -> int:
    """float32 values that :func:`attention_prefill` wants in ``cut_buf`` per run of a tile whose
    keys are cut into runs; 0 where this shape's kernel cuts no tiles."""
    n = int(library().dli_attention_prefill_cut_floats(head_dim, q_heads, kv_heads))
    _require(n >= 0, "query heads are not a multiple of kv heads")
    return n


def attention_prefill_max_cuts() -> int:
    """The most runs that :func:`attention_prefill` lets a tile's keys be cut into."""
    return int(library().dli_attention_prefill_max_cuts())


def _check_paged(q, k_pages, v_pages, out, q_heads):
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _rows(q, "q", torch.bfloat16)
    _rows(out, "out", torch.bfloat16)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size),
             "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(q.shape[1] == q_heads * head_dim and out.shape == q.shape, "q/out must be [rows, q_heads*head_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    _require(q.stride(0) % 4 == 0 and out.stride(0) % 4 == 0 and q.data_ptr() % 8 == 0 and out.data_ptr() % 8 == 0,
             "q/out rows must be 8-byte aligned")
    _require(bool(library().dli_attention_mfma_supports(head_dim, page_size)),
             f"the matrix-core attention takes head_dim 16..128 in steps of 16 and pages of a multiple of 16, "
             f"not head_dim {head_dim}, page size {page_size}")
    return kv_heads, page_size, head_dim


def attention_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: Optional[torch.Tensor],
                     kv_len: torch.Tensor, block_tables: torch.Tensor, q_heads: int, scale: float,
                     window: int = 0, splits: int = 1, part_o: Optional[torch.Tensor] = None,
                     part_ml: Optional[torch.Tensor] = None, merge: bool = True,
                     arrivals: Optional[torch.Tensor] = None) -> None:
    """Decode attention: row ``e`` of ``q`` is request ``e``'s single query over its ``kv_len[e]`` keys.

    With ``splits > 1`` each request's keys are cut into that many runs whose partial results go
    through ``part_o [rows, q_heads, splits, head_dim]`` and ``part_ml [rows, q_heads, splits, 2]``
    (float32) and are merged by a second kernel; with ``merge=False`` (``splits > 1`` only) they
    are left there for :func:`skinny_gemm_merged` and ``out`` is not written (it may be None).
    ``arrivals``: int32 counters (one per request, kv head and 16 query heads of its group; zero before
    the first launch, and every launch leaves them zero) with which the launch merges by itself, the
    workgroup that finishes last doing the second kernel's work with the same result to the bit
    (up to :data:`SELF_MERGING_SPLITS` runs; beyond that the second kernel runs as without them).
    """
    _require(merge or splits > 1, "without a merge there must be two or more runs of keys")
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out if out is not None else q, q_heads)
    _require(merge is False or out is not None, "out is needed unless the partial results are left unmerged")
    rows = q.shape[0]
    _dense(kv_len, "kv_len", torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    _require(kv_len.shape[0] >= rows and block_tables.shape[0] >= rows, "one kv_len and table row per request")
    _require(1 <= splits <= 65535 and rows <= 65535, "splits and requests must fit the grid")
    if splits > 1:
        _require(part_o is not None and part_ml is not None, "splits > 1 needs the partial-result buffers")
        _dense(part_o, "part_o", torch.float32)
        _dense(part_ml, "part_ml", torch.float32)
        _require(part_o.numel() >= rows * q_heads * splits * head_dim and part_ml.numel() >= rows * q_heads * splits * 2,
                 "partial-result buffers are too small")
    if not merge:
        _check(library().dli_attention_decode_partial_bf16(
            _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(part_o), _ptr(part_ml), _ptr(kv_len),
            _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size, float(scale),
            int(window), int(splits), _stream()), "attention_decode")
        return
    if arrivals is not None and splits > 1:
        _dense(arrivals, "arrivals", torch.int32, 1)
        _require(arrivals.numel() >= rows * kv_heads * ((q_heads // kv_heads + 15) // 16),
                 "one arrival counter per request, kv head and tile of 16 heads")
        _check(library().dli_attention_decode_self_merging_bf16(
            _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml),
            _ptr(arrivals), _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads,
            head_dim, page_size, float(scale), int(window), int(splits), _stream()), "attention_decode")
        return
    _check(library().dli_attention_decode_bf16(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml),
        _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size,
        float(scale), int(window), int(splits), _stream()), "attention_decode")


SELF_MERGING_SPLITS = 16  # csrc/merge_splits.h: MERGE_SPLITS

STATIC_SCRATCH_FLOATS = 2 * 1024 * 1024  # csrc/no_alloc.h: DLI_STATIC_SCRATCH_FLOATS


def attention_decode_static(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                            kv_len: torch.Tensor, block_tables: torch.Tensor, q_heads: int, scale: float,
                            window: int = 0, splits: int = 1) -> None:
    """:func:`attention_decode` for callers that cannot allocate: the partial results of the key
    splits live in a static device array of :data:`STATIC_SCRATCH_FLOATS` floats inside the
    library (one per GPU, shared by every call on it: calls that overlap on one GPU race)."""
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out, q_heads)
    rows = q.shape[0]
    _dense(kv_len, "kv_len", torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    _require(kv_len.shape[0] >= rows and block_tables.shape[0] >= rows, "one kv_len and table row per request")
    _require(1 <= splits <= 65535 and rows <= 65535, "splits and requests must fit the grid")
    status = library().dli_attention_decode_bf16_static(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size, float(scale),
        int(window), int(splits), _stream())
    if status == -3:
        raise KernelArgumentError(
            f"attention_decode_static: {rows} requests x {q_heads} heads x {splits} splits x {head_dim} need more "
            f"than the {STATIC_SCRATCH_FLOATS} floats of static scratch")
    _check(status, "attention_decode_static")


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``[tokens, 2, half]`` float32: cos and sin of ``float(position) * inv_freq``, rounded to
    ``dtype`` as the rotation kernels round them. One table serves every layer of a step."""
    _dense(positions, "positions", torch.int32, 1)
    _dense(inv_freq, "inv_freq", torch.float32, 1)
    n, half = positions.shape[0], inv_freq.shape[0]
    table = torch.empty(n, 2, half, device=positions.device, dtype=torch.float32)
    _check(library().dli_rope_angles(_ptr(positions), _ptr(inv_freq), _ptr(table), n, half, _is_bf16(dtype),
                                     _stream()), "rope_angles")
    return table


def attention_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                      tile_entry: torch.Tensor, tile_q0: torch.Tensor, q_heads: int, scale: float,
                      window: int = 0, tile_cut: Optional[torch.Tensor] = None, cut_tiles: int = 0, cut_room: int = 0,
                      cut_buf: Optional[torch.Tensor] = None, cut_count: Optional[torch.Tensor] = None) -> None:
    """Matrix-core attention for portions; operands as :func:`attention_generic`, tiles of
    :func:`attention_prefill_tile_rows` queries (the tile list must be built with that height, in
    any order: every tile has a workgroup of its own and workgroups start in the list's order, so
    the tiles with the most keys belong first).

    ``tile_cut`` (int32, one per list entry; only without a window and where
    :func:`attention_prefill_cut_floats` is not 0): -1 for a whole tile, or ``run | runs << 4 |
    place << 8`` for one of the 2 to :func:`attention_prefill_max_cuts` runs of a tile that is
    listed once per run and whose keys that many workgroups share, ``place`` numbering the
    ``cut_tiles`` cut tiles from 0. ``cut_room``: the most runs of any tile; ``cut_buf``: float32,
    ``cut_tiles * cut_room * attention_prefill_cut_floats(...)`` values; ``cut_count``: int32,
    ``cut_tiles * q_heads`` counters, zero before the first launch (every launch leaves them zero;
    launches that share them must not overlap)."""
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out, q_heads)
    for name, t in (("q_start", q_start), ("kv_len", kv_len), ("tile_entry", tile_entry), ("tile_q0", tile_q0)):
        _dense(t, name, torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
    if tile_cut is not None:
        _dense(tile_cut, "tile_cut", torch.int32, 1)
        _require(tile_cut.shape == tile_entry.shape, "tile_cut differs in length from the tile list")
        per = attention_prefill_cut_floats(head_dim, q_heads, kv_heads)
        _require(per > 0 and window == 0, "this shape's kernel cuts no tiles, or a window is set")
        _require(cut_buf is not None and cut_count is not None and cut_tiles > 0, "cut tiles need their buffers")
        _require(2 <= cut_room <= attention_prefill_max_cuts(), "cut_room outside what the kernel takes")
        _dense(cut_buf, "cut_buf", torch.float32, 1)
        _dense(cut_count, "cut_count", torch.int32, 1)
        _require(cut_buf.shape[0] >= cut_tiles * cut_room * per and cut_count.shape[0] >= cut_tiles * q_heads,
                 "cut_buf or cut_count too small for the cut tiles")
    _check(library().dli_attention_prefill_bf16(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0), tile_entry.shape[0], q_heads,
        kv_heads, head_dim, page_size, float(scale), int(window), _ptr(tile_cut), int(cut_tiles), int(cut_room),
        _ptr(cut_buf), _ptr(cut_count), _stream()), "attention_prefill")

# ----------------------------------------------------------------------------- sampling

def sample_scratch(rows: int, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
    """Scratch that :func:`sample` needs for ``rows`` rows (values and indices of the argmax's
    first stage: its own chunks, or one part per workgroup of a logits kernel that does that stage)."""
    per = max(int(library().dli_sample_scratch_per_row()), compute_units(device))
    return (torch.empty(rows * per, device=device, dtype=torch.float32),
            torch.empty(rows * per, device=device, dtype=torch.int32))


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           seeds: torch.Tensor, counters: torch.Tensor, out: torch.Tensor,
           scratch: Optional[tuple[torch.Tensor, torch.Tensor]] = None) -> None:
    """One token per row of float32 ``logits [rows, vocab]``.

    Rows with ``temperature == 0`` or ``top_k == 1`` take the argmax (lowest id on ties); the others
    apply temperature, top-k (``<= 0``: off), top-p and draw with Philox(seed, counter).
    """
    _rows(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _dense(temperature, "temperature", torch.float32, 1)
    _dense(top_k, "top_k", torch.int32, 1)
    _dense(top_p, "top_p", torch.float32, 1)
    _dense(seeds, "seeds", torch.int64, 1)
    _dense(counters, "counters", torch.int64, 1)
    _dense(out, "out", torch.int32, 1)
    for name, t in (("temperature", temperature), ("top_k", top_k), ("top_p", top_p), ("seeds", seeds),
                    ("counters", counters), ("out", out)):
        _require(t.shape[0] == rows, f"{name} must have one value per row")
    if scratch is None:
        scratch = sample_scratch(rows, logits.device)
    per = int(library().dli_sample_scratch_per_row())
    _dense(scratch[0], "scratch values", torch.float32)
    _dense(scratch[1], "scratch indices", torch.int32)
    _require(scratch[0].numel() >= rows * per and scratch[1].numel() >= rows * per, "sampling scratch is too small")
    _check(library().dli_sample(_ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(top_k),
                                _ptr(top_p), _ptr(seeds), _ptr(counters), _ptr(scratch[0]), _ptr(scratch[1]),
                                _ptr(out), _stream()), "sample")


def sample_and_advance(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                       seeds: torch.Tensor, counters: torch.Tensor, out: torch.Tensor,
                       scratch: tuple[torch.Tensor, torch.Tensor], parts: int, tokens_out: torch.Tensor,
                       token_ids: torch.Tensor, positions: torch.Tensor, kv_len: torch.Tensor,
                       slots: Sequence[torch.Tensor], tables: Sequence[torch.Tensor], page_size: int,
                       advance: bool) -> None:
    """:func:`sample` and :func:`decode_advance` in one launch (for decode steps recorded into a
    graph): the thread that chooses a row's token hands it on. ``parts`` > 0: ``scratch`` already
    holds the first stage of every row's argmax as ``[rows, parts]`` (:func:`head_gemm` with
    ``best``), and the kernel that reads all logits for it does not run."""
    _rows(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _dense(temperature, "temperature", torch.float32, 1)
    _dense(top_p, "top_p", torch.float32, 1)
    _dense(seeds, "seeds", torch.int64, 1)
    _dense(counters, "counters", torch.int64, 1)
    for name, t in (("top_k", top_k), ("out", out), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _dense(t, name, torch.int32, 1)
    for name, t in (("temperature", temperature), ("top_k", top_k), ("top_p", top_p), ("seeds", seeds),
                    ("counters", counters), ("out", out), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _require(t.shape[0] == rows, f"{name} must have one value per row")
    per = int(library().dli_sample_scratch_per_row())
    _dense(scratch[0], "scratch values", torch.float32)
    _dense(scratch[1], "scratch indices", torch.int32)
    need = rows * (parts if parts > 0 else per)
    _require(0 <= parts <= 1024 and scratch[0].numel() >= need and scratch[1].numel() >= need,
             "sampling scratch is too small")
    _require(len(slots) == len(tables) <= 4, "one slot vector and one table per group, at most 4 groups")
    width = 1
    for g, (sl, tb) in enumerate(zip(slots, tables)):
        _dense(sl, f"slots[{g}]", torch.int32, 1)
        _dense(tb, f"tables[{g}]", torch.int32, 2)
        _require(sl.shape[0] == rows and tb.shape[0] == rows, "slots and tables must have one row per request")
        _require(g == 0 or tb.shape[1] == width, "the groups' tables differ in width")
        width = tb.shape[1]
    n = len(slots)
    slot_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in slots] + [None] * (4 - n)))
    table_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in tables] + [None] * (4 - n)))
    _check(library().dli_sample_and_advance(
        _ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
        _ptr(counters), _ptr(scratch[0]), _ptr(scratch[1]), int(parts), _ptr(out), _ptr(tokens_out), _ptr(token_ids),
        _ptr(positions), _ptr(kv_len), ctypes.cast(slot_ptrs, ctypes.c_void_p), ctypes.cast(table_ptrs, ctypes.c_void_p),
        n, width, int(page_size), int(bool(advance)), _stream()), "sample_and_advance")


def decode_advance(sampled: torch.Tensor, tokens_out: torch.Tensor, token_ids: torch.Tensor,
                   positions: torch.Tensor, kv_len: torch.Tensor, counters: torch.Tensor,
                   slots: Sequence[torch.Tensor], tables: Sequence[torch.Tensor], page_size: int,
                   advance: bool) -> None:
    """Hand the sampled tokens of a decode step to the next one on the device.

    ``tokens_out[i] = sampled[i]``; with ``advance`` every row that has keys gets its sampled token
    as next input, position, key count and draw counter plus one, and in each group of layers the
    cache slot of the new position from its block-table row (``tables[g]`` is ``[rows, width]``).
    """
    rows = sampled.shape[0]
    for name, t in (("sampled", sampled), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _dense(t, name, torch.int32, 1)
        _require(t.shape[0] == rows, f"{name} must have one entry per row")
    _dense(counters, "counters", torch.int64, 1)
    _require(counters.shape[0] == rows, "counters must have one entry per row")
    _require(len(slots) == len(tables) <= 4, "one slot vector and one table per group, at most 4 groups")
    width = 1
    for g, (sl, tb) in enumerate(zip(slots, tables)):
        _dense(sl, f"slots[{g}]", torch.int32, 1)
        _dense(tb, f"tables[{g}]", torch.int32, 2)
        _require(sl.shape[0] == rows and tb.shape[0] == rows, "slots and tables must have one row per request")
        _require(g == 0 or tb.shape[1] == width, "the groups' tables differ in width")
        width = tb.shape[1]
    n = len(slots)
    slot_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in slots] + [None] * (4 - n)))
    table_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in tables] + [None] * (4 - n)))
    _check(library().dli_decode_advance(
        _ptr(sampled), _ptr(tokens_out), _ptr(token_ids), _ptr(positions), _ptr(kv_len), _ptr(counters),
        ctypes.cast(slot_ptrs, ctypes.c_void_p), ctypes.cast(table_ptrs, ctypes.c_void_p), n, width,
        int(page_size), rows, int(bool(advance)), _stream()), "decode_advance")
