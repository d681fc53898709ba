"""Each HIP kernel alone against a plain float64 reference, at sizes other than the engine's."""

from __future__ import annotations

import math

import pytest
import torch

from kernel_refs import ref_paged_attention, ref_rms_norm, ref_rope

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 1.6e-2


@pytest.fixture(scope="module")
def ops():
    from dli_amd.kernels import ops as o

    o.library()
    return o


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_gather_rows(ops, dtype):
    torch.manual_seed(0)
    table = torch.randn(37, 50, device="cuda").to(dtype)
    ids = torch.tensor([3, 36, 0, 3, 17], dtype=torch.int32, device="cuda")
    out = torch.empty(5, 50, device="cuda", dtype=dtype)
    ops.embedding(table, ids, out)
    assert torch.equal(out.cpu(), table.cpu()[ids.cpu().long()])
    out2 = torch.empty(5, 50, device="cuda", dtype=dtype)
    ops.gather_rows(table, ids, out2)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,eps", [(64, 1e-5), (192, 1e-6), (2048, 1e-5), (2050, 1e-5), (4104, 1e-5), (7, 1e-2)])
def test_rms_norm(ops, dtype, width, eps):
    torch.manual_seed(1)
    x = (torch.randn(9, width, device="cuda") * 3).to(dtype)
    x[2] = x[2] * 1e-3  # a small row: eps matters here
    w = (1 + 0.1 * torch.randn(width, device="cuda")).float()
    out = torch.empty_like(x)
    ops.rms_norm(x, w, eps, out)
    ref = ref_rms_norm(x.cpu(), w.cpu(), eps)
    assert (out.cpu().double() - ref).abs().max() < tol(dtype) * 4
    # fused residual: x + delta first
    delta = torch.randn_like(x)
    summed = torch.empty_like(x)
    ops.rms_norm(x, w, eps, out, delta=delta, sum_out=summed)
    s_ref = (x.float() + delta.float()).to(dtype)
    assert torch.equal(summed, s_ref)
    ref2 = ref_rms_norm(s_ref.cpu(), w.cpu(), eps)
    assert (out.cpu().double() - ref2).abs().max() < tol(dtype) * 4


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_and_add(ops, dtype):
    torch.manual_seed(2)
    gu = (torch.randn(5, 2 * 23, device="cuda") * 4).to(dtype)
    gu[0, 0] = 0.0
    gu[0, 1] = 30.0
    out = torch.empty(5, 23, device="cuda", dtype=dtype)
    ops.silu_mul(gu, out)
    g, u = gu.cpu().double()[:, :23], gu.cpu().double()[:, 23:]
    ref = g * torch.sigmoid(g) * u
    assert (out.cpu().double() - ref).abs().max() <= tol(dtype) * ref.abs().max()
    assert out[0, 0].item() == 0.0
    a, b = torch.randn(4, 10, device="cuda").to(dtype), torch.randn(4, 10, device="cuda").to(dtype)
    bias = torch.randn(10, device="cuda").to(dtype)
    o = torch.empty_like(a)
    ops.add(a, b, o, bias=bias)
    ref = a.cpu().double() + bias.cpu().double() + b.cpu().double()
    assert (o.cpu().double() - ref).abs().max() < tol(dtype) * 4


@pytest.mark.parametrize("m,n,k", [(1, 5, 7), (3, 64, 64), (65, 130, 100), (200, 97, 258), (17, 384, 192)])
def test_gemm_f32(ops, m, n, k):
    torch.manual_seed(3)
    a = torch.randn(m, k, device="cuda")
    w = torch.randn(n, k, device="cuda")
    bias = torch.randn(n, device="cuda")
    res = torch.randn(m, n, device="cuda")
    out = torch.empty(m, n, device="cuda")
    ops.gemm_f32(a, w, out, bias=bias, residual=res)
    ref = a.cpu().double() @ w.cpu().double().T + bias.cpu().double() + res.cpu().double()
    assert (out.cpu().double() - ref).abs().max() < 1e-5 * math.sqrt(k) * 4
    # a row's result does not depend on the other rows of the batch
    out1 = torch.empty(1, n, device="cuda")
    ops.gemm_f32(a[m - 1:m].contiguous(), w, out1, bias=bias, residual=res[m - 1:m].contiguous())
    assert torch.equal(out1[0], out[m - 1])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("qh,kvh,d,rd,bs", [(4, 4, 16, 16, 16), (6, 2, 32, 32, 8), (3, 1, 48, 32, 4), (2, 2, 80, 80, 16)])
# up to 512 tokens: one item per thread; more: a workgroup per 8 tokens, which writes v in runs where
# the slots are consecutive and aligned in a page (and element by element where they are not)
@pytest.mark.parametrize("n,slots_as", [(11, "scattered"), (70, "scattered"), (203, "consecutive"), (150, "offset"),
                                        (512, "offset"), (530, "scattered"), (707, "consecutive"), (650, "offset")])
def test_rope_kv_write(ops, dtype, qh, kvh, d, rd, bs, n, slots_as):
    torch.manual_seed(4)
    pages = max(9, -(-n // bs) + 3)
    qkv = torch.randn(n, (qh + 2 * kvh) * d, device="cuda").to(dtype)
    orig = qkv.clone()
    positions = torch.tensor([0, 1, 2, 3, 500, 4095, 7, 8, 9, 10, 11] + list(range(100, 100 + n - 11)),
                             dtype=torch.int32, device="cuda")
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, rd, 2).float() / rd))).cuda()
    if slots_as == "scattered":
        perm = torch.randperm(pages * bs)[:n]
    else:  # a prompt's portion: consecutive slots, from a page's start or from inside a page
        first = bs if slots_as == "consecutive" else bs + 3
        perm = torch.arange(first, first + n)
    perm[5] = -1  # not cached
    slots = perm.to(torch.int32).cuda()
    k_pages = torch.full((pages, kvh, bs, d), 7.0, device="cuda").to(dtype)
    v_pages = torch.full((pages, kvh, d, bs), 7.0, device="cuda").to(dtype)
    ops.rope_kv_write(qkv, positions, inv_freq, rd, slots, k_pages, v_pages, qh, kvh, d)
    o = orig.cpu().view(n, qh + 2 * kvh, d)
    q_ref = ref_rope(o[:, :qh], positions.cpu(), inv_freq.cpu(), rd)
    k_ref = ref_rope(o[:, qh:qh + kvh], positions.cpu(), inv_freq.cpu(), rd)
    got = qkv.cpu().view(n, qh + 2 * kvh, d)
    t = tol(dtype) * 4
    assert (got[:, :qh].double() - q_ref).abs().max() < t
    assert torch.equal(got[:, qh:], o[:, qh:])  # k and v columns of the input are left alone
    kp, vp = k_pages.cpu(), v_pages.cpu()
    written = torch.zeros(pages * bs, dtype=torch.bool)
    for tkn in range(n):
        s = int(perm[tkn])
        if s < 0:
            continue
        written[s] = True
        assert (kp[s // bs, :, s % bs, :].double() - k_ref[tkn]).abs().max() < t
        assert torch.equal(vp[s // bs, :, :, s % bs], o[tkn, qh + kvh:])
    for s in range(pages * bs):  # nothing else was touched
        if not written[s]:
            assert (kp[s // bs, :, s % bs, :] == 7.0).all() and (vp[s // bs, :, :, s % bs] == 7.0).all()
    # position 0 is the identity
    assert torch.equal(got[0, :qh], o[0, :qh])


def _paged_case(dtype, qh, kvh, d, bs, lens, seed=0, poison=True):
    """Random pools, scattered tables wider than needed whose spare entries name a poisoned page."""
    g = torch.Generator().manual_seed(seed)
    need = sum(-(-kv // bs) for _, kv in lens)
    pages = need + 3
    k_pages = torch.randn(pages, kvh, bs, d, generator=g)
    v_pages = torch.randn(pages, kvh, d, bs, generator=g)
    poison_page = pages - 1
    if poison:
        k_pages[poison_page] = float("nan")
        v_pages[poison_page] = float("nan")
    order = torch.randperm(pages - 1, generator=g).tolist()
    width = max(-(-kv // bs) for _, kv in lens) + 2
    tables, q_start, kv_len = [], [0], []
    for q_len, kv in lens:
        nb = -(-kv // bs)
        row = [order.pop() for _ in range(nb)]
        tables.append(row + [poison_page] * (width - nb))
        q_start.append(q_start[-1] + q_len)
        kv_len.append(kv)
    q = torch.randn(q_start[-1], qh * d, generator=g)
    return q.to(dtype), k_pages.to(dtype), v_pages.to(dtype), q_start, kv_len, tables


def _tiles(q_start, bm):
    te, tq = [], []
    for e in range(len(q_start) - 1):
        for q0 in range(0, q_start[e + 1] - q_start[e], bm):
            te.append(e)
            tq.append(q0)
    return te, tq


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("qh,kvh,d,bs,window", [
    (4, 4, 16, 16, 0), (6, 2, 32, 8, 0), (3, 3, 64, 4, 0), (8, 2, 128, 16, 0), (2, 1, 80, 16, 0),
    (2, 2, 256, 32, 0), (5, 1, 48, 1, 0), (4, 2, 32, 8, 5), (4, 2, 64, 16, 37),
])
def test_attention_generic(ops, dtype, qh, kvh, d, bs, window):
    # (query tokens now, keys after this step): decode rows, fresh prompts, portions on a prefix
    lens = [(1, 1), (1, bs), (1, bs + 1), (1, 3 * bs - 1), (7, 7), (33, 33), (5, 40), (2, 131), (70, 70), (1, 300)]
    q, kp, vp, q_start, kv_len, tables = _paged_case(dtype, qh, kvh, d, bs, lens, seed=d + bs)
    bm = ops.attention_generic_tile_rows(d)
    te, tq = _tiles(q_start, bm)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    out = torch.full(q.shape, 9.0, dtype=dtype, device="cuda")
    scale = 1.0 / math.sqrt(d)
    ops.attention_generic(q.cuda(), kp.cuda(), vp.cuda(), out, dev(q_start), dev(kv_len), dev(tables),
                          dev(te), dev(tq), qh, scale, window)
    ref = ref_paged_attention(q, kp, vp, q_start, kv_len, tables, qh, scale, window)
    err = (out.cpu().double() - ref).abs().max().item()
    assert err < tol(dtype), err


MFMA_SHAPES = [(4, 4, 16, 16), (6, 2, 32, 16), (32, 8, 64, 16), (14, 2, 64, 32), (8, 8, 128, 16), (5, 1, 80, 16),
               (3, 3, 48, 64), (40, 2, 64, 16), (7, 7, 112, 16), (12, 2, 96, 16), (9, 3, 64, 48), (16, 2, 128, 64)]


@pytest.mark.parametrize("qh,kvh,d,bs", MFMA_SHAPES)
@pytest.mark.parametrize("splits", [1, 4, 16])
@pytest.mark.parametrize("window", [0, 45])
def test_attention_decode_mfma(ops, qh, kvh, d, bs, splits, window):
    """One query per request against scattered, over-wide tables whose spare entries name a
    poisoned page; lengths at the page's edges; every split factor gives the same result."""
    rng = torch.Generator().manual_seed(d * 7 + bs)
    rand = [int(x) for x in torch.randint(1, 40 * bs, (6,), generator=rng)]
    lens = [(1, n) for n in [1, bs, bs + 1, 3 * bs - 1, 15, 16, 17] + rand]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=d + bs + splits)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    out = torch.full(q.shape, 9.0, dtype=torch.bfloat16, device="cuda")
    scale = 1.0 / math.sqrt(d)
    n = len(lens)
    part_o = torch.full((n * qh * splits * d,), float("nan"), device="cuda")
    part_ml = torch.full((n * qh * splits * 2,), float("nan"), device="cuda")
    ops.attention_decode(q.cuda(), kp.cuda(), vp.cuda(), out, dev(kv_len), dev(tables), qh, scale, window, splits,
                         part_o, part_ml)
    ref = ref_paged_attention(q, kp, vp, q_start, kv_len, tables, qh, scale, window)
    err = (out.cpu().double() - ref).abs().max().item()
    assert err < tol(torch.bfloat16), err


@pytest.mark.parametrize("qh,kvh,d,bs", MFMA_SHAPES)
@pytest.mark.parametrize("splits", [2, 5, 16, 17])
@pytest.mark.parametrize("window", [0, 45])
def test_attention_decode_that_merges_in_its_last_workgroup(ops, qh, kvh, d, bs, splits, window):
    """With arrival counters the launch merges its runs of keys by itself: the same bits as with the
    merge kernel, launch after launch on the same counters (each leaves them zero), also after a
    launch with other lengths; 17 runs are more than it takes, then the merge kernel runs."""
    rng = torch.Generator().manual_seed(d * 5 + bs + splits)
    rand = [int(x) for x in torch.randint(1, 40 * bs, (5,), generator=rng)]
    lens = [(1, n) for n in [1, bs, bs + 1, 3 * bs - 1, 15, 17] + rand]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=d + bs + splits)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    q, kp, vp, kv_len, tables = q.cuda(), kp.cuda(), vp.cuda(), dev(kv_len), dev(tables)
    scale = 1.0 / math.sqrt(d)
    n = len(lens)
    counters = torch.zeros(n * kvh * (-(-(qh // kvh) // 16)) + 3, dtype=torch.int32, device="cuda")

    def run(rows, arrivals):
        part_o = torch.full((rows * qh * splits * d,), float("nan"), device="cuda")
        part_ml = torch.full((rows * qh * splits * 2,), float("nan"), device="cuda")
        out = torch.full((rows, qh * d), 9.0, dtype=torch.bfloat16, device="cuda")
        ops.attention_decode(q[:rows], kp, vp, out, kv_len, tables, qh, scale, window, splits, part_o, part_ml,
                             arrivals=arrivals)
        return out

    want = run(n, None)
    for rows in (n, 3, n):
        got = run(rows, counters)
        assert torch.equal(got, want[:rows]), rows
        assert int(counters.abs().sum()) == 0
    with pytest.raises(ops.KernelArgumentError):
        run(n, counters[:2])


@pytest.mark.parametrize("rows", [1, 2, 3, 4])
@pytest.mark.parametrize("qh,kvh,d,n,splits", [(32, 8, 64, 2048, 16), (32, 8, 64, 2048, 8), (8, 2, 48, 304, 3),
                                               (24, 8, 128, 3072, 16), (2, 1, 64, 48, 2), (16, 16, 16, 512, 5)])
@pytest.mark.parametrize("window", [0, 45])
def test_o_projection_that_merges_the_split_key_results_itself(ops, rows, qh, kvh, d, n, splits, window):
    """Attention without its merge kernel, then the o projection that merges while it loads,
    against attention with the merge kernel and the plain residual product: the same bits, since
    both add in the same order. Lengths (and a window) make some runs of keys empty; a bias; rows
    of the stream wider than the product."""
    bs = 16
    lens = [(1, kv) for kv in [700, 33, 1, 255][:rows]]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=rows + d + splits)
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    q, kp, vp, kv_len, tables = q.cuda(), kp.cuda(), vp.cuda(), dev(kv_len), dev(tables)
    scale = 1.0 / math.sqrt(d)
    k = qh * d
    gen = torch.Generator().manual_seed(n + rows)
    w = (torch.randn(n, k, generator=gen) / math.sqrt(k)).bfloat16().cuda()
    bias = torch.randn(n, generator=gen).bfloat16().cuda()
    wt = ops.tile_weights(w)
    base = torch.randn(rows, n + 8, generator=gen).bfloat16().cuda()
    assert ops.skinny_gemm_merged_supports(rows, n, qh, d, splits, q.device)

    def partials():
        return (torch.full((rows * qh * splits * d,), float("nan"), device="cuda"),
                torch.full((rows * qh * splits * 2,), float("nan"), device="cuda"))

    po, pm = partials()
    out = torch.empty_like(q)
    ops.attention_decode(q, kp, vp, out, kv_len, tables, qh, scale, window, splits, po, pm)
    want = base.clone()
    ssq_want = ops.skinny_gemm(out, w, w_tiled=wt, epilogue=ops.SKINNY_RESIDUAL, stream=want[:, :n], bias=bias)

    po, pm = partials()
    ops.attention_decode(q, kp, vp, None, kv_len, tables, qh, scale, window, splits, po, pm, merge=False)
    got = base.clone()
    ssq_got = ops.skinny_gemm_merged(po, pm, splits, qh, d, wt, got[:, :n], bias=bias)
    assert torch.equal(got, want)
    assert torch.equal(ssq_got, ssq_want)
    # and both are the product of the attention's output (64-bit reference)
    ref = base[:, :n].cpu().double() + (out.cpu().double() @ w.cpu().double().T + bias.cpu().double())
    assert (got[:, :n].cpu().double() - ref).abs().max() < 3e-2 * max(1.0, ref.abs().max().item())


def test_the_merging_o_projection_refuses_what_it_does_not_take(ops):
    dev = torch.device("cuda")
    assert not ops.skinny_gemm_merged_supports(5, 2048, 32, 64, 8, dev)       # rows
    assert not ops.skinny_gemm_merged_supports(1, 2048, 32, 64, 17, dev)      # runs of keys
    assert not ops.skinny_gemm_merged_supports(1, 2048, 32, 64, 1, dev)       # nothing to merge
    assert not ops.skinny_gemm_merged_supports(1, 2048, 6, 32, 4, dev)        # k % 128
    assert not ops.skinny_gemm_merged_supports(1, 2048, 64, 128, 4, dev)      # a wave's run of k too long
    stream = torch.zeros(1, 2048, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ops.KernelArgumentError):
        ops.skinny_gemm_merged(torch.zeros(8, device="cuda"), torch.zeros(8, device="cuda"), 17, 32, 64,
                               torch.zeros(2048 * 2048, device="cuda", dtype=torch.bfloat16), stream)
    q = torch.zeros(1, 2048, device="cuda", dtype=torch.bfloat16)
    pages = torch.zeros(2, 8, 16, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ops.KernelArgumentError):
        ops.attention_decode(q, pages, pages.view(2, 8, 64, 16), None, torch.ones(1, dtype=torch.int32, device="cuda"),
                             torch.zeros(1, 1, dtype=torch.int32, device="cuda"), 32, 1.0, 0, 1, merge=False)


@pytest.mark.parametrize("qh,kvh,d,bs", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 37])
def test_attention_prefill_mfma(ops, qh, kvh, d, bs, window):
    """Portions of every shape against their caches (odd and even numbers of tiles, one tile only,
    half-filled last tiles)."""
    lens = [(2, 2), (7, 7), (33, 33), (5, 40), (2, 131), (129, 129), (16, 16), (31, 300), (140, 333), (1, 50),
            (257, 257), (200, 420)]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=d + bs)
    te, tq = _tiles(q_start, ops.attention_prefill_tile_rows(d, qh, kvh))
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    out = torch.full(q.shape, 9.0, dtype=torch.bfloat16, device="cuda")
    scale = 1.0 / math.sqrt(d)
    ops.attention_prefill(q.cuda(), kp.cuda(), vp.cuda(), out, dev(q_start), dev(kv_len), dev(tables),
                          dev(te), dev(tq), qh, scale, window)
    ref = ref_paged_attention(q, kp, vp, q_start, kv_len, tables, qh, scale, window)
    err = (out.cpu().double() - ref).abs().max().item()
    assert err < tol(torch.bfloat16), err


@pytest.mark.parametrize("qh,kvh,d", [(16, 16, 64), (8, 4, 32), (12, 4, 128), (16, 4, 64), (9, 3, 64), (8, 2, 96),
                                      (8, 2, 80), (6, 3, 48), (7, 1, 112), (10, 2, 80)])
def test_attention_prefill_of_a_launch_of_one_and_a_half_workgroups_a_unit(ops, qh, kvh, d):
    """A launch in which compute units work on two tiles of different lengths at a time (and, with
    many heads, in which the order of the workgroups differs from the grid's), listed as the engine
    lists it: one prompt whose length puts the launch there, on top of 24 cached keys, and a short
    one beside it. Once with every tile whole and once with the keys of the longest tiles cut
    into runs that as many workgroups share (twice on the same counters and buffers, with a launch
    for other queries in between: each launch leaves the counters zero, and the two give the same
    bits): whole and cut agree, and rows of both requests agree with a 32-bit softmax over their keys. The same again for a portion of 100 tokens on top of
    3,000 cached keys, whose few tiles are cut into many runs, and for 40 tokens on top of 8,960,
    whose two tiles get as many runs as the kernel takes."""
    units = ops.compute_units(torch.device("cuda"))
    rows = ops.attention_prefill_tile_rows(d, qh, kvh)
    per_tile = qh // (4 * 32 // rows)             # workgroups that a tile of the list becomes
    tiles = -(-units * 3 // (2 * per_tile))        # 1.5 workgroups a unit
    bs = 16
    long_q = tiles * rows - 40 - rows
    for lens, most_runs in (([(long_q, long_q + 24), (40, 77)], 2), ([(100, 3100), (40, 77)], 3),
                            ([(40, 9000), (40, 77)], ops.attention_prefill_max_cuts())):
        _check_cut_and_whole(ops, qh, kvh, d, bs, lens, rows, per_tile, units, most_runs)


def _check_cut_and_whole(ops, qh, kvh, d, bs, lens, rows, per_tile, units, most_runs):
    import numpy as np
    from dli_amd.parts.attention_kernels import list_tiles

    long_q = lens[0][0]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=qh + d)
    dev = lambda x: torch.tensor(np.asarray(x), dtype=torch.int32, device="cuda")
    scale = 1.0 / math.sqrt(d)
    q_len = np.asarray([n for n, _ in lens], np.int64)
    outs = []
    for may_cut in (False, True):
        te, tq, code, n_cut, room = list_tiles(q_len, np.asarray(kv_len, np.int64), 0, rows, per_tile, units, may_cut)
        assert (code is not None) == may_cut
        extra = {}
        if may_cut:
            assert n_cut > 0 and room >= most_runs
            extra = dict(tile_cut=dev(code), cut_tiles=n_cut, cut_room=room,
                         cut_buf=torch.full((n_cut * room * ops.attention_prefill_cut_floats(d, qh, kvh),), float("nan"),
                                            device="cuda"),
                         cut_count=torch.zeros(n_cut * qh, dtype=torch.int32, device="cuda"))
        for again in range(2 if may_cut else 1):
            if again:   # other queries through the same buffers in between: nothing of them may be left behind
                ops.attention_prefill(-q.cuda(), kp.cuda(), vp.cuda(), torch.empty_like(out), dev(q_start), dev(kv_len),
                                      dev(tables), dev(te), dev(tq), qh, scale, 0, **extra)
            out = torch.full(q.shape, 9.0, dtype=torch.bfloat16, device="cuda")
            ops.attention_prefill(q.cuda(), kp.cuda(), vp.cuda(), out, dev(q_start), dev(kv_len), dev(tables), dev(te),
                                  dev(tq), qh, scale, 0, **extra)
            assert torch.isfinite(out.float()).all() and (out.float().abs() < 8).all()   # every row was written
            outs.append(out)
        if may_cut:
            assert int(extra["cut_count"].abs().sum()) == 0
    assert torch.equal(outs[1], outs[2])
    assert (outs[0].float() - outs[1].float()).abs().max().item() < tol(torch.bfloat16)
    # rows of the long request and the short one's last, from their keys gathered out of the pages
    kd, vd = kp.cuda().float(), vp.cuda().float()
    for e, row in ((0, 0), (0, 31), (0, 32), (0, min(127, long_q - 2)), (0, min(128, long_q - 2)), (0, long_q // 2 + 3),
                   (0, long_q - 1), (1, 39)):
        n_keys = kv_len[e] - (q_start[e + 1] - q_start[e]) + row + 1
        pages = torch.tensor(tables[e][:-(-n_keys // bs)], device="cuda")
        keys = kd[pages].permute(1, 0, 2, 3).reshape(kvh, -1, d)[:, :n_keys]         # [kvh, keys, d]
        vals = vd[pages].permute(1, 2, 0, 3).reshape(kvh, d, -1)[:, :, :n_keys]      # [kvh, d, keys]
        qrow = q[q_start[e] + row].cuda().float().view(kvh, qh // kvh, d)
        p = torch.softmax(torch.einsum("hgd,hkd->hgk", qrow, keys) * scale, dim=-1)
        ref = torch.einsum("hgk,hdk->hgd", p, vals).reshape(-1)
        for out in outs[:2]:
            assert (out[q_start[e] + row].float() - ref).abs().max().item() < tol(torch.bfloat16), (e, row)


def test_attention_finds_one_far_key_among_hundreds(ops):
    """One key far back is made to dominate (its q.k is scaled up); the output must be its value.
    A kernel that drops, misplaces or mis-masks a page cannot pass."""
    qh, kvh, d, bs = 8, 2, 64, 16
    lens = [(1, 700), (3, 700)]
    q, kp, vp, q_start, kv_len, tables = _paged_case(torch.bfloat16, qh, kvh, d, bs, lens, seed=3, poison=False)
    kp, vp, q = kp.float(), vp.float(), q.float() * 0.05
    far = 37
    for e in range(2):
        page, off = tables[e][far // bs], far % bs
        kp[page, :, off, :] = 1.0
        for row in range(q_start[e], q_start[e + 1]):
            q[row] = q[row] + 4.0  # q.k of that key: 4*64 = 256 before scaling, 32 after
    q, kp, vp = q.bfloat16(), kp.bfloat16(), vp.bfloat16()
    dev = lambda x: torch.tensor(x, dtype=torch.int32, device="cuda")
    scale = 1.0 / math.sqrt(d)
    out = torch.zeros(q.shape, dtype=torch.bfloat16, device="cuda")
    ops.attention_decode(q[:1].cuda(), kp.cuda(), vp.cuda(), out[:1], dev(kv_len), dev(tables), qh, scale, 0, 4,
                         torch.empty(qh * 4 * d, device="cuda"), torch.empty(qh * 4 * 2, device="cuda"))
    te, tq = _tiles(q_start, ops.attention_prefill_tile_rows(d, qh, kvh))
    te, tq = [t for t in te if t == 1], [q0 for t, q0 in zip(te, tq) if t == 1]
    ops.attention_prefill(q.cuda(), kp.cuda(), vp.cuda(), out, dev(q_start), dev(kv_len), dev(tables),
                          dev(te), dev(tq), qh, scale, 0)
    for e in range(2):
        page, off = tables[e][far // bs], far % bs
        for row in range(q_start[e], q_start[e + 1]):
            got = out[row].float().cpu().view(qh, d)
            for h in range(qh):
                want = vp[page, h // (qh // kvh), :, off].float()
                assert (got[h] - want).abs().max() < 0.05, (e, row, h)


@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n,k", [(48, 1024), (3088, 2048), (1008, 3072), (272, 4096)])
@pytest.mark.parametrize("norm", [False, True])
def test_logits_kernel_whose_workgroups_stay(ops, m, n, k, norm):
    """The product for a vocabulary of rows (workgroups that walk the tiles in turn, activations
    kept in registers): the same bits as the tile-by-tile kernel with 4 k-waves on two tiles,
    whatever the number of workgroups (fewer than pairs of tiles, one, an odd number of tiles at
    the end); against a 64-bit product; rows of the output wider than the product."""
    torch.manual_seed(m + n + k)
    x = (torch.randn(m, k, device="cuda") * 2).bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    wt = ops.tile_weights(w)
    kw = {}
    xhat = x
    if norm:
        nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
        ssq = x.float().pow(2)
        parts = torch.stack([ssq[:, :k // 3].sum(-1), ssq[:, k // 3:].sum(-1)]).contiguous()
        kw = dict(norm_w=nw, eps=1e-5, ssq_in=parts)
        xf = x.float()
        r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)
        xhat = (nw * (xf * r).bfloat16().float()).bfloat16()
    assert ops.head_gemm_supports(m, n, k, torch.bfloat16)
    want = torch.empty(m, n, device="cuda", dtype=torch.float32)
    ops.skinny_gemm(x, w, w_tiled=wt, epilogue=ops.SKINNY_F32, out=want, shape=4, **kw)
    for workgroups in (0, 1, 5, n // 32 + 3):
        wide = torch.full((m, n + 4), 7.0, device="cuda", dtype=torch.float32)
        ops.head_gemm(x, wt, wide[:, :n], workgroups=workgroups, **kw)
        assert torch.equal(wide[:, :n], want), workgroups
        assert (wide[:, n:] == 7.0).all()
    ref = xhat.cpu().double() @ w.cpu().double().T
    assert (want.cpu().double() - ref).abs().max() < 2e-3 * max(1.0, ref.abs().max().item())
    assert not ops.head_gemm_supports(17, n, k, torch.bfloat16) and not ops.head_gemm_supports(m, n, 1536, torch.bfloat16)
    assert not ops.head_gemm_supports(m, n + 8, k, torch.bfloat16) and not ops.head_gemm_supports(m, n, k, torch.float32)
    with pytest.raises(ops.KernelArgumentError):
        ops.head_gemm(x[:, :512].contiguous(), wt, wide[:, :n])


@pytest.mark.parametrize("m,n,k", [(17, 48, 64), (100, 301, 160), (512, 2048, 2048), (70, 1000, 96), (2048, 96, 4104)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_library_product_called_directly(ops, m, n, k, with_bias):
    """The vendor library's bfloat16 product behind the engine's own binding (descriptors and the
    chosen kernel cached per shape): against a float64 product, with the bias inside, with row
    strides larger than the widths, and the second call of a shape like the first."""
    torch.manual_seed(m + n + k)
    xb = torch.randn(m, k + 8, device="cuda").bfloat16()
    x = xb[:, :k]                     # rows contiguous, stride k + 8
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16() if with_bias else None
    outb = torch.full((m, n + 16), 7.0, device="cuda", dtype=torch.bfloat16)
    out = outb[:, :n]
    if not ops.gemm_bf16(x, w, out, bias):
        pytest.skip("the library offers no kernel for this shape: the engine then goes through torch.mm")
    ref = x.cpu().double() @ w.cpu().double().T + (bias.cpu().double() if with_bias else 0.0)
    bound = 2.0 ** -8 * ref.abs().max().item() + 1e-2
    assert (out.cpu().double() - ref).abs().max() < bound
    assert (outb[:, n:] == 7.0).all()   # nothing beyond the row's width is touched
    again = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    assert ops.gemm_bf16(x, w, again, bias)
    assert torch.equal(again, out)
    # the 32-bit sums themselves (the logits of many rows): far closer to the 64-bit product, and
    # rounding them gives the bfloat16 result
    wide = torch.full((m, n + 4), 7.0, device="cuda", dtype=torch.float32)
    if ops.gemm_bf16(x, w, wide[:, :n], bias):
        assert (wide[:, :n].cpu().double() - ref).abs().max() < 1e-4 * max(1.0, ref.abs().max().item())
        assert (wide[:, n:] == 7.0).all()
        assert ((wide[:, :n].bfloat16().float() - out.float()).abs() <= 2.0 ** -7 * out.float().abs() + 1e-6).all()


@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_where_the_direct_library_call_finds_no_kernel(ops, monkeypatch, with_bias):
    """``parts.linear`` goes through ``torch.mm`` (and the engine's bias kernel) for a shape that
    the direct call refuses; the refusal is forced here so that this branch runs on every box."""
    from dli_amd.parts import linear as L
    from dli_amd.parts.base import Runtime

    calls = []
    monkeypatch.setattr(L.ops, "gemm_bf16", lambda *a: calls.append(1) and False)
    torch.manual_seed(5)
    m, n, k = 37, 200, 136
    x = torch.randn(m, k, device="cuda").bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16() if with_bias else None
    rt = Runtime(device=torch.device("cuda"), dtype=torch.bfloat16)
    out = L.linear(rt, x, w, bias)
    assert calls == [1] and out.dtype == torch.bfloat16
    ref = x.cpu().double() @ w.cpu().double().T + (bias.cpu().double() if with_bias else 0.0)
    assert (out.cpu().double() - ref).abs().max() < 2.0 ** -7 * ref.abs().max().item() + 1e-2


def _ref_norm_bf16(x, w, eps):
    """RMSNorm with the engine's rounding: cast(w * cast(x * r))."""
    xf = x.float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (w * (xf * r).bfloat16().float()).bfloat16()


@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("n,k,shape", [(48, 64, 0), (100, 192, 2), (301, 160, 1), (512, 2048, 1), (64, 416, 3),
                                       (1000, 96, 2), (2048, 8192, 1), (1000, 416, 4)])
def test_skinny_gemm_epilogues(ops, m, n, k, shape):
    torch.manual_seed(m * 1000 + n)
    x = torch.randn(m, k, device="cuda").bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16()
    ref = x.cpu().double() @ w.cpu().double().T + bias.cpu().double()
    out = torch.full((m, n), 7.0, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_STORE, out=out, bias=bias, shape=shape)
    assert (out.cpu().double() - ref).abs().max() < 3e-2
    out32 = torch.empty(m, n, device="cuda")
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_F32, out=out32, shape=shape)
    assert (out32.cpu().double() - (ref - bias.cpu().double())).abs().max() < 1e-4 * math.sqrt(k)
    # a row's result does not depend on the other rows
    one = torch.empty(1, n, device="cuda")
    ops.skinny_gemm(x[m - 1:m].contiguous(), w, epilogue=ops.SKINNY_F32, out=one, shape=shape)
    assert torch.equal(one[0], out32[m - 1])
    # residual: stream += y, with the parts of its row sums of squares
    stream = torch.randn(m, n, device="cuda").bfloat16()
    before = stream.clone()
    ssq = torch.full((-(-n // 16), m), float("nan"), device="cuda")
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_RESIDUAL, stream=stream, ssq_out=ssq, bias=bias, shape=shape)
    want = (before.float() + out.float()).bfloat16()
    assert torch.equal(stream, want)
    assert torch.allclose(ssq.sum(0), stream.float().pow(2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("m", [1, 8, 33])
@pytest.mark.parametrize("shape", [0, 2, 3])
@pytest.mark.parametrize("inter,k,parts", [(160, 64, 1), (512, 192, 5), (8192, 2048, 128), (160, 128, 600)])
def test_skinny_gemm_norm_and_swiglu(ops, m, inter, k, shape, parts):
    torch.manual_seed(m + inter)
    x = (torch.randn(m, k, device="cuda") * 2).bfloat16()
    nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
    w = (torch.randn(2 * inter, k, device="cuda") / math.sqrt(k)).bfloat16()
    xs = x.float().pow(2)
    cut = torch.linspace(0, k, parts + 1).long().tolist()
    ssq = torch.stack([xs[:, a:b].sum(-1) for a, b in zip(cut[:-1], cut[1:])]).contiguous()
    eps = 1e-5
    xhat = _ref_norm_bf16(x, nw, eps)
    gu = (xhat.cpu().double() @ w.cpu().double().T)
    g, u = gu[:, :inter].bfloat16().double(), gu[:, inter:].bfloat16().double()
    ref = (g * torch.sigmoid(g)).bfloat16().double() * u
    out = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_SWIGLU, out=out, norm_w=nw, eps=eps, ssq_in=ssq, shape=shape)
    assert (out.cpu().double() - ref).abs().max() < 2e-2 * max(1.0, ref.abs().max().item())
    y = torch.empty(m, 2 * inter, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_STORE, out=y, norm_w=nw, eps=eps, ssq_in=ssq, shape=shape)
    assert (y.cpu().double() - gu).abs().max() < 3e-2 * max(1.0, gu.abs().max().item())


@pytest.mark.parametrize("m", [1, 5, 8, 16])
@pytest.mark.parametrize("shape", [None, 0, 1, 2, 3, 4])
@pytest.mark.parametrize("n,k", [(96, 128), (112, 384), (2048, 2048), (1008, 640)])
def test_skinny_gemm_with_weights_in_tile_order(ops, m, n, k, shape):
    """The second copy of the weights, tile by tile, gives what the row-major weights give (the
    same products; only the split of k over the waves may differ), for every epilogue."""
    torch.manual_seed(m + n + k)
    x = torch.randn(m, k, device="cuda").bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    wt = ops.tile_weights(w)
    assert wt.numel() == w.numel() and not torch.equal(wt.view(n, k), w)
    # element (feature 16*tile + c, k 128*block + 32*g + 8*q + i) sits at [tile][block][q][g][c][i]
    assert wt.view(n // 16, k // 128, 4, 4, 16, 8)[1, 0, 2, 3, 5, 6] == w[16 + 5, 32 * 3 + 8 * 2 + 6]
    bias = torch.randn(n, device="cuda").bfloat16()
    ref = x.cpu().double() @ w.cpu().double().T
    kw = {} if shape is None else {"shape": shape}
    plain32, tiled32 = torch.empty(m, n, device="cuda"), torch.empty(m, n, device="cuda")
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_F32, out=plain32, **kw)
    ops.skinny_gemm(x, w, w_tiled=wt, epilogue=ops.SKINNY_F32, out=tiled32, **kw)
    assert (tiled32.cpu().double() - ref).abs().max() < 1e-4 * math.sqrt(k)
    assert (tiled32 - plain32).abs().max() < 1e-5 * math.sqrt(k)
    # residual with bias and the parts of the sums of squares
    stream = torch.randn(m, n, device="cuda").bfloat16()
    before = stream.clone()
    ssq = ops.skinny_gemm(x, w, w_tiled=wt, epilogue=ops.SKINNY_RESIDUAL, stream=stream, bias=bias, **kw)
    y = (tiled32 + bias.float()).bfloat16()
    assert torch.equal(stream, (before.float() + y.float()).bfloat16())
    assert torch.allclose(ssq.sum(0), stream.float().pow(2).sum(-1), rtol=1e-5)
    # norm prologue and SwiGLU epilogue: gate rows then up rows, both halves whole tiles
    if n % 32 == 0:
        nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
        ssq_in = x.float().pow(2).sum(-1)[None].contiguous()
        a = torch.empty(m, n // 2, device="cuda", dtype=torch.bfloat16)
        b = torch.empty(m, n // 2, device="cuda", dtype=torch.bfloat16)
        ops.skinny_gemm(x, w, epilogue=ops.SKINNY_SWIGLU, out=a, norm_w=nw, eps=1e-5, ssq_in=ssq_in, **kw)
        ops.skinny_gemm(x, w, w_tiled=wt, epilogue=ops.SKINNY_SWIGLU, out=b, norm_w=nw, eps=1e-5, ssq_in=ssq_in, **kw)
        assert (a.float() - b.float()).abs().max() <= 2e-2 * max(1.0, a.float().abs().max().item())
        xhat = _ref_norm_bf16(x, nw, 1e-5)
        gu = xhat.cpu().double() @ w.cpu().double().T
        g, u = gu[:, :n // 2].bfloat16().double(), gu[:, n // 2:].bfloat16().double()
        want = (g * torch.sigmoid(g)).bfloat16().double() * u
        assert (b.cpu().double() - want).abs().max() < 2e-2 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("m", [1, 5, 8, 16])
@pytest.mark.parametrize("qh,kvh,d,k,bs,shape", [(4, 4, 16, 128, 16, None), (6, 2, 32, 384, 8, 0), (5, 1, 48, 256, 4, 4),
                                                 (32, 8, 64, 2048, 16, None), (3, 3, 128, 640, 16, 3)])
def test_skinny_gemm_qkv_with_rotation_and_cache_write(ops, m, qh, kvh, d, k, bs, shape):
    """The fused projection that rotates q and k and writes the cache itself against: norm,
    product, rotation (kernel_refs.ref_rope) and a write by slot, each done plainly."""
    torch.manual_seed(m + qh + d)
    n = (qh + 2 * kvh) * d
    x = (torch.randn(m, k, device="cuda") * 2).bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16()
    nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
    ssq = x.float().pow(2).sum(-1)[None].contiguous()
    positions = torch.tensor([0, 1, 4095, 77, 500, 3, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18][:m], dtype=torch.int32, device="cuda")
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d))).cuda()
    pages = 6
    perm = torch.randperm(pages * bs)[:m]
    if m > 2:
        perm[2] = -1  # not cached
    slots = perm.to(torch.int32).cuda()
    k_pages = torch.full((pages, kvh, bs, d), 7.0, device="cuda").bfloat16()
    v_pages = torch.full((pages, kvh, d, bs), 7.0, device="cuda").bfloat16()
    order = ops.qkv_rope_feature_order(qh, kvh, d)
    assert sorted(order.tolist()) == list(range(n))
    wt = ops.tile_weights_qkv_rope(w, qh, kvh, d)
    q_out = torch.full((m, n), 7.0, device="cuda", dtype=torch.bfloat16)
    angles = ops.rope_angles(positions, inv_freq, torch.bfloat16)
    ops.skinny_gemm_qkv_rope(x, wt, q_out, angles, slots, k_pages, v_pages, qh, bias=bias[order.cuda()].contiguous(),
                             norm_w=nw, eps=1e-5, ssq_in=ssq, shape=shape)
    xhat = _ref_norm_bf16(x, nw, 1e-5)
    y = (xhat.cpu().double() @ w.cpu().double().T + bias.cpu().double()).bfloat16().view(m, qh + 2 * kvh, d)
    q_ref = ref_rope(y[:, :qh], positions.cpu(), inv_freq.cpu(), d)
    k_ref = ref_rope(y[:, qh:qh + kvh], positions.cpu(), inv_freq.cpu(), d)
    scale = max(1.0, y.float().abs().max().item())
    t = 3e-2 * scale
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
    # the same numbers as the separate kernels give: product, then rotation and cache write
    qkv = torch.empty(m, n, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_STORE, out=qkv, bias=bias, norm_w=nw, eps=1e-5, ssq_in=ssq, shape=0)
    k2, v2 = torch.zeros_like(k_pages), torch.zeros_like(v_pages)
    ops.rope_kv_write(qkv, positions, inv_freq, d, slots, k2, v2, qh, kvh, d)
    assert (qkv[:, :qh * d].float() - q_out[:, :qh * d].float()).abs().max() <= 2e-2 * scale


def test_tiled_weights_are_refused_where_they_do_not_fit(ops):
    w = torch.zeros(40, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(ops.KernelArgumentError):
        ops.tile_weights(w)                       # 40 features: no whole tiles
    with pytest.raises(ops.KernelArgumentError):
        ops.tile_weights(torch.zeros(48, 96, device="cuda", dtype=torch.bfloat16))  # k % 128 != 0
    assert not ops.tiled_weights_help(40, 128, ops.SKINNY_STORE, w.device)
    assert not ops.tiled_weights_help(48, 96, ops.SKINNY_STORE, w.device)
    assert not ops.tiled_weights_help(48, 128, ops.SKINNY_SWIGLU, w.device)   # halves of 24 features
    assert ops.tiled_weights_help(2048, 2048, ops.SKINNY_RESIDUAL, w.device)
    assert not ops.tiled_weights_help(2048, 8192, ops.SKINNY_RESIDUAL, w.device)  # the block kernel's at every size
    assert ops.tiled_weights_help(3072, 8192, ops.SKINNY_RESIDUAL, w.device)      # enough tiles for the tile kernel


@pytest.mark.parametrize("m", [1, 3, 4, 5, 8, 9, 16])
@pytest.mark.parametrize("n,k", [(48, 64), (100, 192), (301, 160), (512, 2048), (64, 416), (1000, 96), (2048, 8192)])
@pytest.mark.parametrize("blocks4", [0, 1, 2])
def test_skinny4_gemm_epilogues(ops, m, n, k, blocks4):
    """The 4x4-block product: store, float32 and residual epilogues at sizes that are no multiples
    of its tiles and chunks, in every workgroup shape."""
    torch.manual_seed(m * 1000 + n)
    x = torch.randn(m, k, device="cuda").bfloat16()
    w = (torch.randn(n, k, device="cuda") / math.sqrt(k)).bfloat16()
    bias = torch.randn(n, device="cuda").bfloat16()
    ref = x.cpu().double() @ w.cpu().double().T + bias.cpu().double()
    kw = dict(blocks4=blocks4)
    for _ in range(1):
        out = torch.full((m, n), 7.0, device="cuda", dtype=torch.bfloat16)
        ops.skinny_gemm(x, w, epilogue=ops.SKINNY_STORE, out=out, bias=bias, **kw)
        assert (out.cpu().double() - ref).abs().max() < 3e-2
    out32 = torch.empty(m, n, device="cuda")
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_F32, out=out32, **kw)
    assert (out32.cpu().double() - (ref - bias.cpu().double())).abs().max() < 1e-4 * math.sqrt(k)
    # a row's result does not depend on the other rows (same row group size: same kernel)
    again = torch.empty(m, n, device="cuda")
    x2 = x.clone()
    x2[: m - 1] = torch.randn(m - 1, k, device="cuda").bfloat16()
    ops.skinny_gemm(x2, w, epilogue=ops.SKINNY_F32, out=again, **kw)
    assert torch.equal(again[m - 1], out32[m - 1])
    # residual: stream += y, with the parts of its row sums of squares
    stream = torch.randn(m, n, device="cuda").bfloat16()
    before = stream.clone()
    ssq = ops.skinny_gemm(x, w, epilogue=ops.SKINNY_RESIDUAL, stream=stream, bias=bias, **kw)
    want = (before.float() + out.float()).bfloat16()
    assert torch.equal(stream, want)
    assert ssq.shape[1] == m and torch.allclose(ssq.sum(0), stream.float().pow(2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("m", [1, 8, 13])
@pytest.mark.parametrize("blocks4", [0, 1, 2])
@pytest.mark.parametrize("inter,k,parts", [(160, 64, 1), (500, 192, 5), (8192, 2048, 128), (160, 128, 2100)])
def test_skinny4_gemm_norm_and_swiglu(ops, m, inter, k, parts, blocks4):
    torch.manual_seed(m + inter)
    x = (torch.randn(m, k, device="cuda") * 2).bfloat16()
    nw = (1 + 0.1 * torch.randn(k, device="cuda")).float()
    w = (torch.randn(2 * inter, k, device="cuda") / math.sqrt(k)).bfloat16()
    xs = x.float().pow(2)
    cut = torch.linspace(0, k, parts + 1).long().tolist()
    ssq = torch.stack([xs[:, a:b].sum(-1) for a, b in zip(cut[:-1], cut[1:])]).contiguous()
    eps = 1e-5
    xhat = _ref_norm_bf16(x, nw, eps)
    gu = (xhat.cpu().double() @ w.cpu().double().T)
    g, u = gu[:, :inter].bfloat16().double(), gu[:, inter:].bfloat16().double()
    ref = (g * torch.sigmoid(g)).bfloat16().double() * u
    out = torch.empty(m, inter, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_SWIGLU, out=out, norm_w=nw, eps=eps, ssq_in=ssq, blocks4=blocks4)
    assert (out.cpu().double() - ref).abs().max() < 2e-2 * max(1.0, ref.abs().max().item())
    y = torch.empty(m, 2 * inter, device="cuda", dtype=torch.bfloat16)
    ops.skinny_gemm(x, w, epilogue=ops.SKINNY_STORE, out=y, norm_w=nw, eps=eps, ssq_in=ssq, blocks4=blocks4)
    assert (y.cpu().double() - gu).abs().max() < 3e-2 * max(1.0, gu.abs().max().item())


def test_embedding_with_sum_of_squares(ops):
    table = torch.randn(50, 96, device="cuda").bfloat16()
    ids = torch.tensor([4, 49, 0, 4], dtype=torch.int32, device="cuda")
    out = torch.empty(4, 96, device="cuda", dtype=torch.bfloat16)
    ssq = torch.empty(1, 4, device="cuda")
    ops.embedding_ssq(table, ids, out, ssq)
    assert torch.equal(out, table[ids.long()])
    assert torch.allclose(ssq[0], out.float().pow(2).sum(-1), rtol=1e-5)
