"""The decode attention that allocates nothing (csrc/no_alloc.h) against the entry point that takes
the caller's partial-result buffers (the same bits) and against the plain float64 attention of
tests/kernel_refs.py (so that the two cannot be wrong alike): called through ctypes, twice in a
row, the second call with a smaller input, so that what the first call left in the static array
must not matter."""

from __future__ import annotations

import ctypes

import pytest
import torch

from kernel_refs import ref_paged_attention

pytestmark = pytest.mark.gpu

BF16_TOL = 1.6e-2  # the bound of the decode attention's own kernel test


def _case(seed, requests, q_heads, kv_heads, head_dim, page, max_len, splits):
    g = torch.Generator().manual_seed(seed)
    pages = requests * (-(-max_len // page)) + 3
    k = (torch.randn(pages, kv_heads, page, head_dim, generator=g) * 0.5).to(torch.bfloat16).cuda()
    v = (torch.randn(pages, kv_heads, head_dim, page, generator=g) * 0.5).to(torch.bfloat16).cuda()
    q = torch.randn(requests, q_heads * head_dim, generator=g).to(torch.bfloat16).cuda()
    lens = torch.randint(1, max_len + 1, (requests,), generator=g, dtype=torch.int32)
    lens[0] = max_len
    width = -(-max_len // page)
    perm = torch.randperm(pages, generator=g)[:requests * width].to(torch.int32).view(requests, width)
    return dict(q=q, k=k, v=v, kv_len=lens.cuda(), tables=perm.contiguous().cuda(), q_heads=q_heads,
                kv_heads=kv_heads, head_dim=head_dim, page=page, splits=splits, requests=requests)


def _run(lib, c, static: bool):
    from dli_amd.kernels import ops

    out = torch.full((c["requests"], c["q_heads"] * c["head_dim"]), 7.0, dtype=torch.bfloat16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    scale = ctypes.c_float(c["head_dim"] ** -0.5)
    common = (c["requests"], c["q_heads"], c["kv_heads"], c["head_dim"], c["page"], scale, 0, c["splits"], stream)
    if static:
        rc = lib.dli_attention_decode_bf16_static(
            ptr(c["q"]), c["q"].stride(0), ptr(c["k"]), ptr(c["v"]), ptr(out), out.stride(0), ptr(c["kv_len"]),
            ptr(c["tables"]), c["tables"].stride(0), *common)
    else:
        slots = c["requests"] * c["q_heads"] * c["splits"]
        part_o = torch.empty(slots * c["head_dim"], dtype=torch.float32, device="cuda")
        part_ml = torch.empty(slots * 2, dtype=torch.float32, device="cuda")
        rc = lib.dli_attention_decode_bf16(
            ptr(c["q"]), c["q"].stride(0), ptr(c["k"]), ptr(c["v"]), ptr(out), out.stride(0), ptr(part_o),
            ptr(part_ml), ptr(c["kv_len"]), ptr(c["tables"]), c["tables"].stride(0), *common)
    torch.cuda.synchronize()
    return rc, out


def test_decode_attention_without_allocation_equals_the_one_with_buffers():
    from dli_amd.kernels import ops

    lib = ops.library()
    lib.dli_attention_decode_static_floats.argtypes = [ctypes.c_int] * 4
    lib.dli_attention_decode_static_floats.restype = ctypes.c_int64
    big = _case(1, requests=8, q_heads=32, kv_heads=8, head_dim=64, page=16, max_len=1500, splits=16)
    small = _case(2, requests=3, q_heads=12, kv_heads=4, head_dim=128, page=32, max_len=300, splits=4)
    one = _case(3, requests=2, q_heads=8, kv_heads=8, head_dim=32, page=16, max_len=90, splits=1)
    for c in (big, small, one, big):  # a smaller call after a larger one, then the larger again
        need = lib.dli_attention_decode_static_floats(c["requests"], c["q_heads"], c["head_dim"], c["splits"])
        slots = c["requests"] * c["q_heads"] * c["splits"]
        assert need == (0 if c["splits"] == 1 else -(-slots * c["head_dim"] // 64) * 64 + 2 * slots)
        assert need <= ops.STATIC_SCRATCH_FLOATS
        rc_ref, ref = _run(lib, c, static=False)
        before = torch.cuda.memory_allocated()
        rc, got = _run(lib, c, static=True)
        assert rc_ref == 0 and rc == 0
        assert torch.equal(got, ref), (got.float() - ref.float()).abs().max()
        plain = ref_paged_attention(c["q"].cpu(), c["k"].cpu(), c["v"].cpu(), list(range(c["requests"] + 1)),
                                    c["kv_len"].tolist(), c["tables"].tolist(), c["q_heads"], c["head_dim"] ** -0.5)
        err = (got.cpu().double() - plain).abs().max().item()
        assert err < BF16_TOL, err
        assert not torch.equal(got, torch.full_like(got, 7.0))
        del got
        assert torch.cuda.memory_allocated() <= before


def test_sizes_beyond_the_static_array_are_refused():
    from dli_amd.kernels import ops

    lib = ops.library()
    c = _case(4, requests=64, q_heads=32, kv_heads=8, head_dim=128, page=16, max_len=64, splits=16)
    rc, out = _run(lib, c, static=True)  # 64*32*16*128 floats = 4 Mi floats > 2 Mi
    assert rc == -3
    assert torch.equal(out, torch.full_like(out, 7.0)), "a refused call must not write"
    with pytest.raises(ops.KernelArgumentError, match="static scratch"):
        ops.attention_decode_static(c["q"], c["k"], c["v"], out, c["kv_len"], c["tables"], c["q_heads"],
                                    c["head_dim"] ** -0.5, splits=c["splits"])
