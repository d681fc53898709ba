"""A plain, slow Llama decoder: whole sequences, no cache, one function for each part.

Written from the reference's formulas (each function cites file:line under ``src/dli``), with
nothing imported from the engine. It reads ``config.json`` as a raw dictionary and the weights with
the ``safetensors`` library, so the engine's own parser, reader and writer are checked against
something that shares no code with them. Everything runs on the CPU. ``dtype`` is float64 by default:
the engine's 32-bit path is then compared with a result whose own rounding is negligible. The two
places where the reference fixes 32-bit arithmetic whatever the model's dtype (rotary frequencies
and angles) keep it.
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from typing import Any, Mapping, Sequence

import torch


# --------------------------------------------------------------------------- position encoding

def rope_settings(cfg: Mapping[str, Any]) -> dict[str, Any]:
    """Rotary constants of a config.json dictionary (model/config.py:130-150).

    ``rope_parameters`` wins over ``rope_scaling``; ``type`` is the old spelling of ``rope_type``;
    theta defaults to 10000, low/high factors to 1 and 4, the original context to
    ``max_position_embeddings`` and then 8192.
    """
    merged = {**dict(cfg.get("rope_scaling") or {}), **dict(cfg.get("rope_parameters") or {})}
    theta = merged.get("rope_theta", cfg.get("rope_theta", 10000.0))
    if theta is None:
        theta = 10000.0
    kind = merged.get("rope_type", merged.get("type", "default"))
    out = {"theta": float(theta), "rope_type": kind}
    if kind != "default":
        out["factor"] = float(merged["factor"])
        out["low_freq_factor"] = float(merged.get("low_freq_factor", 1.0))
        out["high_freq_factor"] = float(merged.get("high_freq_factor", 4.0))
        out["original_max_position_embeddings"] = int(
            merged.get("original_max_position_embeddings", cfg.get("max_position_embeddings", 8192))
        )
    return out


def inverse_frequencies(rope: Mapping[str, Any], head_dim: int) -> torch.Tensor:
    """Per-pair inverse frequencies ``[head_dim // 2]`` in float32 (model/rope.py:21-47)."""
    exponents = torch.arange(0, head_dim, 2, dtype=torch.int64).to(torch.float32) / head_dim
    inv_freq = 1.0 / (rope["theta"] ** exponents)
    kind = rope["rope_type"]
    if kind == "default":
        return inv_freq
    if kind == "linear":
        return inv_freq / rope["factor"]
    if kind == "llama3":
        old_ctx = rope["original_max_position_embeddings"]
        low_wavelen = old_ctx / rope["low_freq_factor"]
        high_wavelen = old_ctx / rope["high_freq_factor"]
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > low_wavelen, inv_freq / rope["factor"], inv_freq)
        smooth = (old_ctx / wavelen - rope["low_freq_factor"]) / (
            rope["high_freq_factor"] - rope["low_freq_factor"]
        )
        smoothed = (1 - smooth) * scaled / rope["factor"] + smooth * scaled
        medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
        return torch.where(medium, smoothed, scaled)
    raise ValueError(f"rope_type {kind!r}")


def rope_cos_sin(inv_freq: torch.Tensor, positions: torch.Tensor, dtype: torch.dtype):
    """``cos``/``sin`` tables ``[n, head_dim]``: float32 angles, then the cast (model/rope.py:50-60)."""
    angles = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
    emb = torch.cat((angles, angles), dim=-1).to(torch.float64)  # exact cos/sin of the fp32 angle
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """``cat(-x[d/2:], x[:d/2])``: dimension i pairs with i + d/2 (model/rope.py:63-65)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate ``x [heads, n, d]`` by per-token angles (model/rope.py:68-70)."""
    return x * cos + rotate_half(x) * sin


# --------------------------------------------------------------------------- norm

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``weight * (x * rsqrt(mean(x^2) + eps))``, eps inside the root (model/llama.py:40-44)."""
    h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return weight * h


# --------------------------------------------------------------------------- attention

def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """``x W^T + b`` with ``W [out, in]`` (``nn.Linear``; model/llama.py:56-59)."""
    y = x @ weight.transpose(0, 1)
    return y if bias is None else y + bias


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """Whole-sequence causal attention (model/llama.py:147-177).

    ``q [heads, n, d]``, ``k, v [kv_heads, n, d]``. Query head h reads KV head ``h // fan_out``
    (contiguous groups, :158-163); scores are scaled by ``1/sqrt(d)``; key j is visible to query i
    iff ``j <= i`` (:168-176 with ``past == 0``).
    """
    heads, n, d = q.shape
    fan_out = heads // k.shape[0]
    out = torch.empty_like(q)
    visible = torch.tril(torch.ones(n, n, dtype=torch.bool))
    for h in range(heads):
        kh, vh = k[h // fan_out], v[h // fan_out]
        scores = (q[h] @ kh.transpose(0, 1)) / math.sqrt(d)
        scores = scores.masked_fill(~visible, float("-inf"))
        out[h] = torch.softmax(scores, dim=-1) @ vh
    return out


def attention_block(x, w: Mapping[str, torch.Tensor], prefix: str, cfg, cos, sin) -> torch.Tensor:
    """Projections, rotation of q and k, attention, output projection (model/llama.py:61-96)."""
    n = x.shape[0]
    nh, nkv, d = cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    q = linear(x, w[prefix + "q_proj.weight"], w.get(prefix + "q_proj.bias"))
    k = linear(x, w[prefix + "k_proj.weight"], w.get(prefix + "k_proj.bias"))
    v = linear(x, w[prefix + "v_proj.weight"], w.get(prefix + "v_proj.bias"))
    q = q.view(n, nh, d).transpose(0, 1)
    k = k.view(n, nkv, d).transpose(0, 1)
    v = v.view(n, nkv, d).transpose(0, 1)
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    out = causal_attention(q, k, v)
    merged = out.transpose(0, 1).reshape(n, nh * d)
    return linear(merged, w[prefix + "o_proj.weight"], w.get(prefix + "o_proj.bias"))


# --------------------------------------------------------------------------- feed-forward

def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def swiglu_mlp(x, w: Mapping[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))`` (model/llama.py:180-191)."""
    gate = linear(x, w[prefix + "gate_proj.weight"], w.get(prefix + "gate_proj.bias"))
    up = linear(x, w[prefix + "up_proj.weight"], w.get(prefix + "up_proj.bias"))
    return linear(silu(gate) * up, w[prefix + "down_proj.weight"], w.get(prefix + "down_proj.bias"))


# --------------------------------------------------------------------------- whole model

def model_sizes(cfg: Mapping[str, Any]) -> dict[str, Any]:
    """Sizes with the reference's defaults (model/config.py:104-127)."""
    nh = int(cfg["num_attention_heads"])
    hidden = int(cfg["hidden_size"])
    return {
        "num_heads": nh,
        "num_kv_heads": int(cfg.get("num_key_value_heads") or nh),
        "head_dim": int(cfg.get("head_dim") or hidden // nh),
        "num_layers": int(cfg["num_hidden_layers"]),
        "eps": float(cfg["rms_norm_eps"]),
        "tied": bool(cfg.get("tie_word_embeddings", False)),
    }


def decoder_layer(x, w, i: int, sizes, cos, sin) -> torch.Tensor:
    """Pre-norm block: ``x + attn(norm(x))`` then ``x + mlp(norm(x))`` (model/llama.py:194-213)."""
    p = f"model.layers.{i}."
    x = x + attention_block(
        rms_norm(x, w[p + "input_layernorm.weight"], sizes["eps"]), w, p + "self_attn.", sizes, cos, sin
    )
    return x + swiglu_mlp(rms_norm(x, w[p + "post_attention_layernorm.weight"], sizes["eps"]), w, p + "mlp.")


def forward_logits(
    weights: Mapping[str, torch.Tensor],
    cfg: Mapping[str, Any],
    token_ids: Sequence[int],
    *,
    dtype: torch.dtype = torch.float64,
    first_position: int = 0,
) -> torch.Tensor:
    """Logits ``[n, vocab]`` at every position of one whole sequence (model/llama.py:249-305).

    ``first_position`` shifts all positions by a constant (attention then sees the same distances).
    """
    sizes = model_sizes(cfg)
    w = {k: t.to(dtype) for k, t in weights.items()}
    ids = torch.tensor(list(token_ids), dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(ids))
    h = w["model.embed_tokens.weight"][ids]
    inv_freq = inverse_frequencies(rope_settings(cfg), sizes["head_dim"])
    cos, sin = rope_cos_sin(inv_freq, positions, dtype)
    for i in range(sizes["num_layers"]):
        h = decoder_layer(h, w, i, sizes, cos, sin)
    h = rms_norm(h, w["model.norm.weight"], sizes["eps"])
    head = w["model.embed_tokens.weight"] if sizes["tied"] else w["lm_head.weight"]
    return linear(h, head)


def greedy_generate(weights, cfg, prompt: Sequence[int], max_new_tokens: int, **kw) -> list[int]:
    """Argmax decoding that recomputes the whole sequence each step (generate.py:21-87,
    ``use_cache=False``); ties go to the lowest id."""
    tokens = list(prompt)
    out: list[int] = []
    for _ in range(max_new_tokens):
        logits = forward_logits(weights, cfg, tokens, **kw)
        nxt = int(torch.argmax(logits[-1]).item())
        out.append(nxt)
        tokens.append(nxt)
    return out


# --------------------------------------------------------------------------- sampling

def sampling_probabilities(logits: torch.Tensor, temperature: float, top_k: int, top_p: float) -> torch.Tensor:
    """Distribution that one stochastic row is drawn from (sampling.py:83-110).

    Temperature, then top-k by rank in a descending sort, softmax, then top-p: a token is dropped
    iff the mass of strictly more likely tokens reaches ``top_p``; softmax again over the rest.
    Returned in vocabulary order.
    """
    x = logits.to(torch.float64) / temperature
    sorted_logits, order = torch.sort(x, descending=True, stable=True)
    vocab = x.shape[-1]
    k = top_k if top_k > 0 else vocab
    ranks = torch.arange(vocab)
    sorted_logits = sorted_logits.masked_fill(ranks >= k, float("-inf"))
    probs = torch.softmax(sorted_logits, dim=-1)
    preceding = torch.cumsum(probs, dim=-1) - probs
    sorted_logits = sorted_logits.masked_fill(preceding >= top_p, float("-inf"))
    probs = torch.softmax(sorted_logits, dim=-1)
    out = torch.zeros(vocab, dtype=torch.float64)
    out[order] = probs
    return out


# --------------------------------------------------------------------------- files

def load_folder(model_dir: str | Path) -> tuple[dict[str, Any], dict[str, torch.Tensor]]:
    """``config.json`` as a dictionary and every tensor of the folder's safetensors files."""
    from safetensors.torch import load_file

    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    weights: dict[str, torch.Tensor] = {}
    for f in sorted(model_dir.glob("*.safetensors")):
        weights.update(load_file(str(f)))
    return cfg, weights
