"""The product kernel for decode steps of 17 to 64 rows and its two finishing kernels, each alone
against float64 references, at sizes other than the engine's (features that fill no tile, k that
does not divide by the splits, rows that fill no row tile)."""

from __future__ import annotations

import math

import pytest
import torch

from kernel_refs import ref_rope

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from dli_amd.kernels import ops as o

    o.library()
    return o


def ref_norm_bf16(x, w, eps):
    """RMSNorm with the engine's rounding: cast(w * cast(x * r))."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (w * (xf * r).bfloat16().float()).bfloat16()


def make(m, n_rows, k, seed):
    torch.manual_seed(seed)
    x = (torch.randn(m, k, device="cuda") * 2).bfloat16()
    w = (torch.randn(n_rows, k, device="cuda") / math.sqrt(k)).bfloat16()
    nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
    # the sums of squares in three uneven parts, as a producer that splits its rows would leave them
    ssq = x.float().pow(2)
    cuts = [0, k // 3, k // 2, k]
    parts = torch.stack([ssq[:, a:b].sum(-1) for a, b in zip(cuts, cuts[1:])]).contiguous()
    return x, w, nw, parts


@pytest.mark.parametrize("m", [1, 16, 17, 24, 33, 48, 64])
@pytest.mark.parametrize("n,k,tiled", [(48, 128, False), (100, 384, False), (304, 640, True), (2048, 2048, True),
                                       (36, 1152, False), (576, 576, True), (100, 200, False), (64, 960, True),
                                       (48, 72, True)])
@pytest.mark.parametrize("norm", [False, True])
def test_partial_products_add_up_to_the_product(ops, m, n, k, tiled, norm):
    x, w, nw, parts = make(m, n, k, seed=m + n)
    xhat = ref_norm_bf16(x, nw, 1e-5) if norm else x
    ref = xhat.cpu().double() @ w.cpu().double().T
    bound = 2e-3 * max(1.0, ref.abs().max().item())
    # (k that is no multiple of 128: the copy in tile order has its last block filled up with zeros,
    # row by row the kernel reads on into the next row; the activations past k count as zeros)
    wt = ops.tile_weights(w, whole_blocks=False) if tiled else w
    kw = dict(norm_w=nw, eps=1e-5, ssq_in=parts) if norm else {}
    nblk = -(-k // 128)
    results = []
    shapes = list(ops.MID_SHAPES)
    plans = {(1, shapes[m % len(shapes)]), (nblk, (4, 1)), (max(1, nblk // 2), (4, 2)), (min(3, nblk), (4, 2)),
             (min(2, nblk), (4, 1)), (None, (None, None))}
    for splits, (waves, kwaves) in plans:
        out = ops.mid_gemm(x, wt, epilogue=ops.MID_PARTIAL, tiled=tiled, n=n, splits=splits, waves=waves,
                           kwaves=kwaves, **kw)
        assert out.dtype == torch.float32 and out.shape[1:] == (m, n)
        if splits is not None:
            assert out.shape[0] == splits
        total = out.cpu().double().sum(0)
        assert (total - ref).abs().max() < bound, (splits, waves, kwaves)
        results.append(total)
    # however k is split, the sums agree to 32-bit rounding
    for r in results[1:]:
        assert (r - results[0]).abs().max() < 1e-4 * max(1.0, ref.abs().max().item())


@pytest.mark.parametrize("m", [3, 17, 40, 64])
@pytest.mark.parametrize("n,k,tiled", [(40, 256, False), (160, 384, True), (8192, 2048, True), (1536, 576, True),
                                       (48, 328, False)])
def test_gated_and_stored_products(ops, m, n, k, tiled):
    x, w, nw, parts = make(m, 2 * n, k, seed=m + n + 1)
    bias = torch.randn(2 * n, device="cuda").bfloat16()
    xhat = ref_norm_bf16(x, nw, 1e-5)
    y = xhat.cpu().double() @ w.cpu().double().T + bias.cpu().double()
    g, u = y[:, :n].bfloat16().float(), y[:, n:].bfloat16().float()
    ref = (torch.nn.functional.silu(g).bfloat16().float() * u).double()
    wt = ops.tile_weights(w, whole_blocks=False) if tiled else w
    for waves, kwaves in ((2, 1), (2, 4), (2, 2), (None, None)):
        out = ops.mid_gemm(x, wt, epilogue=ops.MID_SWIGLU, tiled=tiled, n=n, bias=bias, norm_w=nw, eps=1e-5,
                           ssq_in=parts, waves=waves, kwaves=kwaves)
        assert out.dtype == torch.bfloat16 and out.shape == (m, n)
        assert (out.cpu().double() - ref).abs().max() < 2e-2 * max(1.0, ref.abs().max().item())
    # plain store with a bias, into rows that are wider than the product
    wide = torch.full((m, 2 * n + 8), 7.0, device="cuda", dtype=torch.bfloat16)
    ops.mid_gemm(x, wt, epilogue=ops.MID_STORE, tiled=tiled, n=2 * n, bias=bias, out=wide[:, :2 * n])
    ref2 = x.cpu().double() @ w.cpu().double().T + bias.cpu().double()
    assert (wide[:, :2 * n].cpu().double() - ref2).abs().max() < 1.6e-2 * max(1.0, ref2.abs().max().item())
    assert (wide[:, 2 * n:] == 7.0).all()


def test_shapes_that_the_product_refuses(ops):
    x = torch.zeros(65, 128, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(32, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(x, w, epilogue=ops.MID_PARTIAL)                       # 65 rows
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(x[:8, :100].contiguous(), w[:, :100].contiguous(), epilogue=ops.MID_PARTIAL)  # k % 8
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(x[:8], w, epilogue=ops.MID_STORE, splits=1, waves=2, kwaves=1)   # a shape of the gated product
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(x[:8], w, epilogue=ops.MID_PARTIAL, splits=2)          # one block of k only
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(x[:8], w.view(-1), epilogue=ops.MID_PARTIAL, tiled=True, n=24)  # no whole tiles
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_gemm(torch.zeros(8, 200, device="cuda", dtype=torch.bfloat16), ops.tile_weights(w),
                     epilogue=ops.MID_PARTIAL, tiled=True, n=32)   # a copy of fewer blocks of k
    assert ops.mid_gemm_supports(8, 96, torch.bfloat16)
    assert not ops.mid_gemm_supports(8, 100, torch.bfloat16) and not ops.mid_gemm_supports(8, 128, torch.float32)
    assert ops.mid_gemm_plan(2048, 8192, ops.MID_PARTIAL, 256) == (4, 2, 8)
    assert ops.mid_gemm_plan(8192, 2048, ops.MID_SWIGLU, 256, rows=32) == (2, 2, 1)
    assert ops.mid_gemm_plan(8192, 2048, ops.MID_SWIGLU, 256, rows=64) == (2, 2, 1)
    assert ops.mid_gemm_plan(8192, 3072, ops.MID_SWIGLU, 256, rows=33) == (2, 4, 1)
    assert ops.mid_gemm_plan(8192, 3072, ops.MID_SWIGLU, 256, rows=32) == (2, 2, 1)
    assert ops.mid_gemm_plan(8192, 256, ops.MID_SWIGLU, 256, rows=64) == (2, 2, 1)
    assert ops.mid_gemm_plan(48, 128, ops.MID_PARTIAL, 256) == (4, 1, 1)


@pytest.mark.parametrize("m,n,splits", [(1, 64, 1), (24, 200, 3), (64, 2048, 8), (33, 3076, 11)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_finish_of_a_residual_product(ops, m, n, splits, with_bias):
    torch.manual_seed(m + n)
    partial = torch.randn(splits, m, n, device="cuda")
    base = torch.randn(m, n + 4, device="cuda").bfloat16()
    stream = base[:, :n]                      # rows wider than the product
    before = stream.clone()
    bias = torch.randn(n, device="cuda").bfloat16() if with_bias else None
    ssq = ops.mid_finish_residual(partial, stream, bias)
    y = partial[0].clone()
    for s in range(1, splits):
        y += partial[s]                       # 32-bit, in the order of the splits
    if with_bias:
        y += bias.float()
    want = (before.float() + y.bfloat16().float()).bfloat16()
    assert torch.equal(stream, want)
    assert torch.equal(base[:, n:], base[:, n:])
    ref_ssq = want.double().pow(2).sum(-1)
    assert ssq.shape == (-(-n // 1024), m)
    assert (ssq.sum(0).cpu().double() - ref_ssq.cpu()).abs().max() < 1e-4 * ref_ssq.max().item()


@pytest.mark.parametrize("m,n,splits", [(1, 64, 1), (24, 200, 3), (64, 2048, 8), (33, 3076, 11), (17, 8192, 2), (5, 5000, 4)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_finish_of_a_residual_product_that_also_normalises(ops, m, n, splits, with_bias):
    """The same stream as the plain finish leaves, bit for bit, its whole sums of squares, and
    beside it the rows normalised as the fused norm prologues normalise (two roundings)."""
    torch.manual_seed(m + n + 1)
    partial = torch.randn(splits, m, n, device="cuda")
    base = (torch.randn(m, n + 4, device="cuda") * 3).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16() if with_bias else None
    nw = (1 + 0.1 * torch.randn(n, device="cuda")).float()
    plain = base.clone()
    parts = ops.mid_finish_residual(partial, plain[:, :n], bias)
    got = base.clone()
    wide = torch.full((m, n + 8), 7.0, device="cuda", dtype=torch.bfloat16)
    ssq = ops.mid_finish_residual(partial, got[:, :n], bias, norm_w=nw, eps=1e-5, normed_out=wide[:, :n])
    assert torch.equal(got, plain)
    assert ssq.shape == (1, m)
    ref_ssq = got[:, :n].double().pow(2).sum(-1)
    assert (ssq[0].double() - ref_ssq).abs().max() < 1e-4 * ref_ssq.max().item()
    assert (parts.sum(0).double() - ref_ssq).abs().max() < 1e-4 * ref_ssq.max().item()
    want = ref_norm_bf16(got[:, :n], nw, 1e-5)
    # rs from sums added in another order may move the inner rounding by one step of bfloat16,
    # which the outer rounding can double
    diff = (wide[:, :n].float() - want.float()).abs()
    assert (diff <= 2.0 ** -6 * want.float().abs() + 1e-6).all()
    assert (diff > 0).float().mean() < 0.02
    assert (wide[:, n:] == 7.0).all()
    with pytest.raises(ops.KernelArgumentError):
        ops.mid_finish_residual(torch.zeros(1, 2, 8196, device="cuda"), torch.zeros(2, 8196, device="cuda").bfloat16(),
                                norm_w=torch.ones(8196, device="cuda"), eps=1e-5,
                                normed_out=torch.zeros(2, 8196, device="cuda").bfloat16())


@pytest.mark.parametrize("m", [1, 17, 64])
@pytest.mark.parametrize("qh,kvh,d,k,bs", [(4, 4, 16, 128, 16), (6, 2, 32, 384, 8), (5, 1, 48, 256, 4),
                                           (32, 8, 64, 2048, 16), (3, 3, 128, 640, 16), (9, 3, 64, 576, 16)])
def test_split_qkv_product_with_its_finish(ops, m, qh, kvh, d, k, bs):
    """Product in splits, then sum, bias, rotation and cache write in the finishing kernel, against
    norm, product, rotation (kernel_refs.ref_rope) and a write by slot, each done plainly."""
    n = (qh + 2 * kvh) * d
    x, w, nw, parts = make(m, n, k, seed=m + qh + d)
    bias = torch.randn(n, device="cuda").bfloat16()
    gen = torch.Generator().manual_seed(m)
    positions = torch.randint(0, 5000, (m,), generator=gen).to(torch.int32).cuda()
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d))).cuda()
    pages = -(-m // bs) + 3
    perm = torch.randperm(pages * bs, generator=gen)[:m]
    if m > 2:
        perm[2] = -1  # not cached
    slots = perm.to(torch.int32).cuda()
    k_pages = torch.full((pages, kvh, bs, d), 7.0, device="cuda").bfloat16()
    v_pages = torch.full((pages, kvh, d, bs), 7.0, device="cuda").bfloat16()
    order = ops.qkv_rope_feature_order(qh, kvh, d).cuda()
    wt = ops.tile_weights_qkv_rope(w, qh, kvh, d)
    angles = ops.rope_angles(positions, inv_freq, torch.bfloat16)
    q_out = torch.full((m, n), 7.0, device="cuda", dtype=torch.bfloat16)
    partial = ops.mid_gemm(x, wt, epilogue=ops.MID_PARTIAL, tiled=True, n=n, norm_w=nw, eps=1e-5, ssq_in=parts,
                           splits=min(3, -(-k // 128)))
    ops.mid_finish_qkv(partial, q_out, angles, slots, k_pages, v_pages, qh, bias=bias[order].contiguous())
    xhat = ref_norm_bf16(x, nw, 1e-5)
    y = (xhat.cpu().double() @ w.cpu().double().T + bias.cpu().double()).bfloat16().view(m, qh + 2 * kvh, d)
    q_ref = ref_rope(y[:, :qh], positions.cpu(), inv_freq.cpu(), d)
    k_ref = ref_rope(y[:, qh:qh + kvh], positions.cpu(), inv_freq.cpu(), d)
    t = 3e-2 * max(1.0, y.float().abs().max().item())
    got = q_out.cpu().view(m, qh + 2 * kvh, d)
    assert (got[:, :qh].double() - q_ref).abs().max() < t
    assert (got[:, qh:] == 7.0).all()   # k and v go to the pages only
    kp, vp = k_pages.cpu(), v_pages.cpu()
    written = torch.zeros(pages * bs, dtype=torch.bool)
    for row in range(m):
        s_ = int(perm[row])
        if s_ < 0:
            continue
        written[s_] = True
        assert (kp[s_ // bs, :, s_ % bs, :].double() - k_ref[row]).abs().max() < t
        assert (vp[s_ // bs, :, :, s_ % bs].double() - y[row, qh + kvh:].double()).abs().max() < t
    for s_ in range(pages * bs):
        if not written[s_]:
            assert (kp[s_ // bs, :, s_ % bs, :] == 7.0).all() and (vp[s_ // bs, :, :, s_ % bs] == 7.0).all()
    if m <= 16 and k % 128 == 0:
        # the product for few rows that rotates in its own epilogue gives the same numbers
        q2 = torch.empty_like(q_out)
        k2, v2 = torch.zeros_like(k_pages), torch.zeros_like(v_pages)
        ops.skinny_gemm_qkv_rope(x, wt, q2, angles, slots, k2, v2, qh, bias=bias[order].contiguous(), norm_w=nw,
                                 eps=1e-5, ssq_in=parts)
        assert (q2[:, :qh * d].float() - q_out[:, :qh * d].float()).abs().max() <= t
