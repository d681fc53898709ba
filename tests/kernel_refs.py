"""Plain PyTorch references of single kernels (float64 on the CPU), for the kernel tests."""

from __future__ import annotations

import math

import torch


def ref_rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    x = x.double()
    return w.double() * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))


def ref_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    """x [tokens, heads, d]; NeoX pairing (i, i + rotary_dim/2) on the first rotary_dim dims."""
    ang = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
    cos, sin = ang.double().cos()[:, None, :], ang.double().sin()[:, None, :]
    h = rotary_dim // 2
    x = x.double()
    x1, x2 = x[..., :h], x[..., h:rotary_dim]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., rotary_dim:]), dim=-1)


def gather_keys(k_pages: torch.Tensor, v_pages: torch.Tensor, table: list[int], n_keys: int):
    """Keys/values [kv_heads, n_keys, d] of one request from K [P,kvh,bs,d] and V [P,kvh,d,bs]."""
    bs = k_pages.shape[2]
    ks, vs = [], []
    for j in range(n_keys):
        page, off = table[j // bs], j % bs
        ks.append(k_pages[page, :, off, :])
        vs.append(v_pages[page, :, :, off])
    return torch.stack(ks, 1).double(), torch.stack(vs, 1).double()


def ref_paged_attention(q, k_pages, v_pages, q_start, kv_len, tables, q_heads, scale, window=0):
    """q [tokens, q_heads*d] -> out [tokens, q_heads*d] in float64, request by request."""
    kvh, d = k_pages.shape[1], k_pages.shape[3]
    group = q_heads // kvh
    out = torch.zeros(q.shape, dtype=torch.float64)
    for e in range(len(kv_len)):
        t0, t1 = q_start[e], q_start[e + 1]
        n_keys = kv_len[e]
        if t1 == t0:
            continue
        k, v = gather_keys(k_pages.cpu(), v_pages.cpu(), tables[e], n_keys)
        qe = q[t0:t1].cpu().double().view(t1 - t0, q_heads, d)
        first = n_keys - (t1 - t0)
        for i in range(t1 - t0):
            pos = first + i
            lo = 0 if window <= 0 else max(0, pos - window + 1)
            for h in range(q_heads):
                kk, vv = k[h // group, lo:pos + 1], v[h // group, lo:pos + 1]
                p = torch.softmax((kk @ qe[i, h]) * scale, dim=0)
                out[t0 + i, h * d:(h + 1) * d] = p @ vv
    return out
