"""Each HIP kernel alone against a plain float64 reference of the same op,
at sizes other than the engine tests': widths that are no power of two, odd
head groups, head sizes from 16 to 256, pages in shuffled order."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"


def ops():
    from vt_transformer_amd.kernels import ops as o
    return o


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    ref = ref.double().cpu()
    got = got.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(torch.float64)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vocab,hidden,n", [(203, 80, 7), (1000, 3584, 33)])
def test_embed(dtype, vocab, hidden, n):
    g = torch.Generator().manual_seed(1)
    table = torch.randn(vocab, hidden, generator=g).to(dtype)
    ids = torch.randint(0, vocab, (n,), generator=g, dtype=torch.int32)
    ids[0], ids[-1] = vocab - 1, 0
    out = torch.empty(n, hidden, dtype=torch.float32, device=DEV)
    ops().embed(table.to(DEV), ids.to(DEV), out)
    assert torch.equal(out.cpu(), table.float()[ids.long()])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("delta_dtype", [None, torch.float32, "out"])
@pytest.mark.parametrize("n,hidden,eps", [(5, 80, 1e-5), (3, 3584, 1e-6), (2, 1000, 1e-2)])
def test_rmsnorm_with_residual(out_dtype, delta_dtype, n, hidden, eps):
    g = torch.Generator().manual_seed(2)
    h = torch.randn(n, hidden, generator=g) * 3
    gain = 1 + 0.1 * torch.randn(hidden, generator=g)
    if delta_dtype == "out":        # a 16-bit delta is of the build's 16-bit type, like the output
        delta_dtype = torch.bfloat16 if out_dtype == torch.float32 else out_dtype
    delta = None if delta_dtype is None else torch.randn(n, hidden, generator=g).to(delta_dtype)
    x = h.double() + (delta.double() if delta is not None else 0)
    ref = gain.double() * x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    hd = h.to(DEV)
    out = torch.empty(n, hidden, dtype=out_dtype, device=DEV)
    ops().rmsnorm(hd, delta.to(DEV) if delta is not None else None, gain.to(DEV), out, eps)
    tol = 1e-5 if out_dtype == torch.float32 else 5e-3
    assert rel_err(out, ref) < tol
    # the sum went back into the residual stream, in fp32
    assert rel_err(hd, x) < 1e-6
    # eps sits inside the root: a large eps must show
    if eps == 1e-2:
        wrong = gain.double() * x / (torch.sqrt((x * x).mean(-1, keepdim=True)) + eps)
        assert rel_err(out, wrong) > 10 * tol or out_dtype != torch.float32


def test_rmsnorm_rows_gather():
    g = torch.Generator().manual_seed(3)
    h = torch.randn(9, 96, generator=g)
    delta = torch.randn(9, 96, generator=g)
    gain = torch.randn(96, generator=g)
    rows = torch.tensor([8, 0, 3], dtype=torch.int32)
    x = (h + delta).double()[rows.long()]
    ref = gain.double() * x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    hd = h.to(DEV)
    out = torch.empty(3, 96, dtype=torch.float32, device=DEV)
    ops().rmsnorm(hd, delta.to(DEV), gain.to(DEV), out, 1e-6, rows=rows.to(DEV))
    assert rel_err(out, ref) < 1e-5
    assert torch.equal(hd.cpu(), h)  # a row list never writes the residual


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,inter", [(5, 200), (3, 204), (2, 203), (300, 1184)])   # widths in steps of 8, of 4, odd
def test_silu_mul(dtype, n, inter):
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(n, 2 * inter, generator=g) * 4).to(dtype)
    gate, up = gu[:, :inter].double(), gu[:, inter:].double()
    ref = gate / (1 + torch.exp(-gate)) * up
    out = torch.empty(n, inter, dtype=dtype, device=DEV)
    ops().silu_mul(gu.to(DEV), out)
    assert rel_err(out, ref) < (1e-6 if dtype == torch.float32 else 5e-3)
    # gate = 0 gives 0 whatever the up value
    z = torch.zeros(1, 2 * inter, dtype=dtype)
    z[:, inter:] = 7
    out1 = torch.empty(1, inter, dtype=dtype, device=DEV)
    ops().silu_mul(z.to(DEV), out1)
    assert float(out1.abs().max()) == 0.0


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n,m,k", [(1, 200, 96), (7, 320, 200), (16, 64, 64), (17, 130, 50), (70, 257, 333)])
def test_linear_f32(n, m, k):
    g = torch.Generator().manual_seed(5)
    x, w, b = torch.randn(n, k, generator=g), torch.randn(m, k, generator=g), torch.randn(m, generator=g)
    out = torch.empty(n, m, dtype=torch.float32, device=DEV)
    ops().linear_f32(x.to(DEV), w.to(DEV), b.to(DEV), out)
    assert rel_err(out, x.double() @ w.double().t() + b.double()) < 2e-6
    out2 = torch.empty(n, m, dtype=torch.float32, device=DEV)
    ops().linear_f32(x.to(DEV), w.to(DEV), None, out2)
    assert rel_err(out2, x.double() @ w.double().t()) < 2e-6


def test_linear_f32_is_true_fp32_and_batch_invariant():
    """Values that a reduced-precision matrix mode would lose; and a row's result must not depend on the batch."""
    g = torch.Generator().manual_seed(6)
    k, m = 512, 96
    x = torch.randn(40, k, generator=g) * (1 + 2.0 ** -12)
    w = torch.randn(m, k, generator=g)
    big = torch.empty(40, m, dtype=torch.float32, device=DEV)
    ops().linear_f32(x.to(DEV), w.to(DEV), None, big)
    assert rel_err(big, x.double() @ w.double().t()) < 2e-6  # tf32/bf16 products would be near 1e-3
    one = torch.empty(1, m, dtype=torch.float32, device=DEV)
    ops().linear_f32(x[11:12].to(DEV).contiguous(), w.to(DEV), None, one)
    assert torch.equal(one[0], big[11])


@pytest.mark.parametrize("n", [1, 3, 16, 17, 33, 64, 100, 300])
@pytest.mark.parametrize("m,k", [(320, 96), (200, 200), (1030, 3584), (96, 18944 // 8)])
@pytest.mark.parametrize("out_dtype", [torch.float32, "lowp"])
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_linear_bf16(n, m, k, out_dtype, lp):
    g = torch.Generator().manual_seed(7)
    out_dtype = lp if out_dtype == "lowp" else out_dtype
    x = torch.randn(n, k, generator=g).to(lp)
    w = (torch.randn(m, k, generator=g) * 0.05).to(lp)
    b = torch.randn(m, generator=g)
    ref = x.double() @ w.double().t() + b.double()
    out = torch.empty(n, m, dtype=out_dtype, device=DEV)
    ops().linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), out, work_for(n, m, k))
    assert rel_err(out, ref) < (2e-5 if out_dtype == torch.float32 else 5e-3)


def work_for(n, m, k):
    need = ops().linear_bf16_workspace(n, m, k) if n > 16 else 0
    return torch.full((need,), float("nan"), device=DEV) if need else None


def test_linear_bf16_split_k_needs_and_uses_a_workspace():
    o = ops()
    g = torch.Generator().manual_seed(81)
    n, m, k = 100, 256, 4096           # few rows of W, long k, more than 64 tokens: the k range is split over blocks
    assert o.linear_bf16_workspace(n, m, k) >= 2 * n * m
    assert o.linear_bf16_workspace(8, m, k) == 0 and o.linear_bf16_workspace(24, m, k) == 0   # whole k in a block
    x = torch.randn(n, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(m, k, generator=g) * 0.05).to(torch.bfloat16)
    b = torch.randn(m, generator=g)
    out = torch.empty(n, m, dtype=torch.float32, device=DEV)
    with pytest.raises(o.KernelError, match="workspace"):
        o.linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), out)
    o.linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), out, work_for(n, m, k))
    assert rel_err(out, x.double() @ w.double().t() + b.double()) < 2e-5


@pytest.mark.parametrize("n", [17, 31, 32, 33, 50, 64])
@pytest.mark.parametrize("m,k", [(200, 200), (1030, 3584), (96, 18944 // 4), (3584, 512), (4608, 256), (4100, 128)])
def test_linear_bf16_adds_to_a_residual_up_to_64_rows(n, m, k):
    """17 to 64 rows: whole k in a block (two or four token tiles, one or two tile rows of W; 4,100 rows leave the
    last block's second tile row beyond the matrix), the result added to a residual in place; shapes for which the
    kernel that splits k over blocks is the faster one add the residual in the launch that adds the partial sums."""
    g = torch.Generator().manual_seed(83)
    x = torch.randn(n, k, generator=g).to(torch.bfloat16)
    w = (torch.randn(m, k, generator=g) * 0.05).to(torch.bfloat16)
    b = torch.randn(m, generator=g)
    res = torch.randn(n, m, generator=g)
    h = res.to(DEV)
    if not ops().linear_bf16_adds_residual(n, m, k):
        assert n > 32 and k > 3000 and m % 4         # k split over blocks, and rows that the adding launch cannot take by fours
        with pytest.raises(ops().KernelError, match="residual"):
            ops().linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), h, residual=h)
        return
    need = ops().linear_bf16_workspace(n, m, k)
    work = torch.full((need,), float("nan"), device=DEV) if need else None
    if need:
        with pytest.raises(ops().KernelError, match="workspace"):
            ops().linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), h, residual=h)
    out = ops().linear_bf16(x.to(DEV), w.to(DEV), b.to(DEV), h, work, residual=h)
    assert out is h
    assert rel_err(h, res.double() + x.double() @ w.double().t() + b.double()) < 2e-5
    with pytest.raises(ops().KernelError, match="residual"):
        big = torch.zeros(65, m, device=DEV)
        ops().linear_bf16(torch.zeros(65, k, dtype=torch.bfloat16, device=DEV), w.to(DEV), None, big, residual=big)


def test_linear_bf16_says_which_shapes_take_a_residual():
    o = ops()
    assert o.linear_bf16_adds_residual(16, 3584, 18944) and o.linear_bf16_adds_residual(1, 50, 64)
    assert not o.linear_bf16_adds_residual(8, 50, 53)            # k no multiple of 8: the any-shape kernel
    assert o.linear_bf16_adds_residual(64, 3584, 3584)           # 224 tile rows: one block each, whole k
    assert o.linear_bf16_adds_residual(64, 4608, 3584)           # 288 tile rows: two per block
    assert o.linear_bf16_adds_residual(64, 3584, 18944)          # a long k at 64 rows: split over blocks, and the launch that adds up adds the residual
    assert not o.linear_bf16_adds_residual(64, 152064, 3584)     # many rows: nothing to split
    assert not o.linear_bf16_adds_residual(65, 3584, 3584)


@pytest.mark.parametrize("m,k,halves", [(16, 128, 1), (70, 53, 1), (1030, 3584, 1), (200, 96, 2), (37, 264, 2)])
def test_unpack_gives_back_what_was_packed(m, k, halves):
    g = torch.Generator().manual_seed(84)
    w = torch.randn(halves * m, k, generator=g).to(torch.bfloat16).to(DEV)
    packed = ops().pack_matrix_bf16(w, halves)
    out = torch.full_like(w, float("nan"))
    assert torch.equal(ops().unpack_matrix_bf16(packed, out), w)


def test_linear_bf16_odd_k_uses_plain_kernel():
    g = torch.Generator().manual_seed(8)
    n, m, k = 5, 70, 53
    x = torch.randn(n, k, generator=g).to(torch.bfloat16)
    w = torch.randn(m, k, generator=g).to(torch.bfloat16)
    out = torch.empty(n, m, dtype=torch.float32, device=DEV)
    ops().linear_bf16(x.to(DEV), w.to(DEV), None, out)
    assert rel_err(out, x.double() @ w.double().t()) < 2e-5


def test_linear_bf16_batch_invariant():
    g = torch.Generator().manual_seed(9)
    m, k = 640, 1536
    x = torch.randn(64, k, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(m, k, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    # up to 16 rows one kernel, above it another: within each, a row's result does not depend on the batch
    full = torch.empty(64, m, dtype=torch.float32, device=DEV)
    ops().linear_bf16(x, w, None, full, work_for(64, m, k))
    for rows in (list(range(20, 37)), list(range(3, 50))):
        sub = torch.empty(len(rows), m, dtype=torch.float32, device=DEV)
        ops().linear_bf16(x[rows].contiguous(), w, None, sub, work_for(len(rows), m, k))
        assert torch.equal(sub, full[rows]), rows
    small = torch.empty(16, m, dtype=torch.float32, device=DEV)
    ops().linear_bf16(x[:16].contiguous(), w, None, small)
    for rows in ([5], [0, 15], list(range(2, 11))):
        sub = torch.empty(len(rows), m, dtype=torch.float32, device=DEV)
        ops().linear_bf16(x[rows].contiguous(), w, None, sub)
        assert torch.equal(sub, small[rows]), rows
    assert rel_err(small, full[:16]) < 1e-5


@pytest.mark.parametrize("n", [1, 9, 40, 64, 100, 128, 300])
@pytest.mark.parametrize("inter,k", [(200, 96), (128, 64), (1184, 3584), (18944, 40), (22016, 32), (29568, 24)])
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_gated_linear_bf16(n, inter, k, lp):
    # the three wide ones make the 64-token kernel take 5, 6 and 8 waves a block; from 65 rows on a block takes 128 tokens
    g = torch.Generator().manual_seed(10)
    x = torch.randn(n, k, generator=g).to(lp)
    w = (torch.randn(2 * inter, k, generator=g) * 0.05).to(lp)
    gate = x.double() @ w[:inter].double().t()
    up = x.double() @ w[inter:].double().t()
    ref = gate / (1 + torch.exp(-gate)) * up
    out = torch.empty(n, inter, dtype=lp, device=DEV)
    ops().gated_linear_bf16(x.to(DEV), w.to(DEV), out)
    assert rel_err(out, ref) < 6e-3
    out32 = torch.empty(n, inter, dtype=torch.float32, device=DEV)
    ops().gated_linear_bf16(x.to(DEV), w.to(DEV), out32)
    assert rel_err(out32, ref) < 3e-5


# ---------------------------------------------------------------------------
# paged cache helpers
# ---------------------------------------------------------------------------
def make_pages(k, v, lens, page_size, dtype, seed, extra_pages=3, free_before=None):
    """k, v: lists of [T_e, KVH, D] per entry.  Pages in shuffled order.  Returns k_pages, v_pages, block_table.
    free_before[e]: pages that lie wholly before this key have been given back (a window has passed them): the
    table holds -1 there, as the cache manager leaves it."""
    kvh, d = k[0].shape[1], k[0].shape[2]
    n_blocks = [-(-t // page_size) for t in lens]
    total = sum(n_blocks) + extra_pages
    perm = np.random.RandomState(seed).permutation(total)
    kp = torch.full((total, kvh, page_size, d), 1e4, dtype=torch.float32)   # unwritten slots hold a large finite value
    vp = torch.full((total, kvh, d, page_size), -1e4, dtype=torch.float32)
    bt = torch.full((len(lens), max(n_blocks) + 2), -1, dtype=torch.int32)
    nxt = 0
    for e, t in enumerate(lens):
        for b in range(n_blocks[e]):
            if free_before is not None and (b + 1) * page_size <= free_before[e]:
                continue
            pg = int(perm[nxt]); nxt += 1
            bt[e, b] = pg
            lo, hi = b * page_size, min(t, (b + 1) * page_size)
            kp[pg, :, : hi - lo, :] = k[e][lo:hi].permute(1, 0, 2)
            vp[pg, :, :, : hi - lo] = v[e][lo:hi].permute(1, 2, 0)
    return kp.to(dtype), vp.to(dtype), bt


def ref_attention(q, k, v, pos, window, scale):
    """q [NH, D] at position pos against k, v [T, KVH, D]; float64."""
    nh, d = q.shape
    kvh = k.shape[1]
    out = torch.zeros(nh, d, dtype=torch.float64)
    lo = max(0, pos - window + 1) if window > 0 else 0
    for h in range(nh):
        kk, vv = k[lo:pos + 1, h // (nh // kvh)].double(), v[lo:pos + 1, h // (nh // kvh)].double()
        s = (kk @ q[h].double()) * scale
        p = torch.softmax(s, dim=0)
        out[h] = p @ vv
    return out


def attention_case(dtype, nh, kvh, d, page_size, window, entries, seed, spike=False):
    """entries: list of (cached tokens, new tokens).  Returns (got, ref) as [N, NH*D]."""
    o = ops()
    g = torch.Generator().manual_seed(seed)
    lens = [c + n for c, n in entries]
    ks = [torch.randn(t, kvh, d, generator=g) for t in lens]
    vs = [torch.randn(t, kvh, d, generator=g) for t in lens]
    qs = [torch.randn(n, nh, d, generator=g) for _, n in entries]
    if spike:
        # one far key that the query must find: its score stands out among hundreds
        for e, (c, n) in enumerate(entries):
            far = 3 if window == 0 else max(0, lens[e] - window)  # the oldest key the last token may still see
            ks[e][far] *= 0
            ks[e][far, :, 0] = 30.0
            qs[e][-1] *= 0
            qs[e][-1, :, 0] = 30.0 * math.sqrt(d) / 30.0 * 2.0
            vs[e][far] = 5.0
    if dtype != torch.float32:
        ks, vs, qs = ([t.to(dtype).float() for t in x] for x in (ks, vs, qs))
    # with a window: the pages that the entry's first new token no longer sees are gone
    free_before = [max(0, c - window + 1) for c, _ in entries] if window > 0 else None
    kp, vp, bt = make_pages(ks, vs, lens, page_size, dtype, seed, free_before=free_before)
    n_tok = sum(n for _, n in entries)
    q = torch.cat(qs).reshape(n_tok, nh * d).to(dtype).to(DEV)
    positions = torch.tensor([c + i for c, n in entries for i in range(n)], dtype=torch.int32)
    tok_entry = torch.tensor([e for e, (c, n) in enumerate(entries) for _ in range(n)], dtype=torch.int32)
    out = torch.empty(n_tok, nh * d, dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(d)
    if dtype == torch.float32:
        o.attention_f32(q, kp.to(DEV), vp.to(DEV), positions.to(DEV), tok_entry.to(DEV), bt.to(DEV), out, nh, kvh, d,
                        window, scale)
    else:
        from vt_transformer_amd.parts.attention_plan import plan_attention_items
        start = np.cumsum([0] + [n for _, n in entries]).astype(np.int32)
        pos0 = np.array([c for c, _ in entries], dtype=np.int32)
        from vt_transformer_amd.parts.attention_plan import plan_tile_items
        first = None
        kpd, vpd, btd = kp.to(DEV), vp.to(DEV), bt.to(DEV)
        # 16-row items with keys unsplit and split, one and two row tiles; then the LDS-tiled kernel on all entries
        for target, rt in ((0, 1), (10 ** 9, 1), (0, 2), (10 ** 9, 2)):
            if rt == 2 and d > 128:
                continue            # two row tiles per wave do not fit the registers with heads above 128
            items, citems, n_parts = plan_attention_items(start, pos0, nh // kvh, window, kvh, target_waves=target,
                                                          min_chunk=16, rt=rt)
            part_o = torch.full((max(1, n_parts) * rt * kvh * 16 * d,), float("nan"), device=DEV)
            part_ml = torch.full((max(1, n_parts) * rt * kvh * 32,), float("nan"), device=DEV)
            out.fill_(float("nan"))
            o.attention_bf16(q, kpd, vpd, btd, torch.from_numpy(items).to(DEV).reshape(-1),
                             items.shape[0], torch.from_numpy(citems).to(DEV).reshape(-1) if len(citems) else None,
                             len(citems), out, part_o, part_ml, nh, kvh, d, window, scale, max_part=n_parts, rt=rt)
            if first is None:
                first = out.clone()
            assert bool(torch.isfinite(out).all()), (target, rt)
            assert rel_err(out, first) < 1e-2, (target, rt)  # every way of cutting the work agrees to rounding
        # ... whole key ranges per item, and the longest items' keys cut into ranges that are merged afterwards
        for rt, split in ((1, 0.), (2, 0.), (1, 0.3), (2, 0.3)):
            items, _, citems, n_parts = plan_tile_items(start, pos0, nh // kvh, window, kvh, np.arange(len(entries)),
                                                        rt=rt, split=split, head_dim=d)
            part_o = torch.full((max(1, n_parts) * 4 * rt * kvh * 16 * d,), float("nan"), device=DEV)
            part_ml = torch.full((max(1, n_parts) * 4 * rt * kvh * 32,), float("nan"), device=DEV)
            out.fill_(float("nan"))
            o.attention_bf16_tiles(q, kpd, vpd, btd, torch.from_numpy(items).to(DEV).reshape(-1), items.shape[0], out,
                                   nh, kvh, d, window, scale, rt=rt,
                                   citems=torch.from_numpy(citems).to(DEV).reshape(-1) if len(citems) else None,
                                   n_citems=len(citems), part_o=part_o, part_ml=part_ml, n_parts=n_parts)
            assert bool(torch.isfinite(out).all()), ("tiles", rt, split)
            assert rel_err(out, first) < 1e-2, ("tiles", rt, split)
    ref = torch.cat([ref_attention(qs[e][i], ks[e], vs[e], c + i, window, scale).reshape(1, -1)
                     for e, (c, n) in enumerate(entries) for i in range(n)])
    return out, ref


ATT_TOL = {torch.float32: 1e-5, torch.bfloat16: 1.5e-2, torch.float16: 2e-3}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nh,kvh,d", [(4, 2, 16), (3, 3, 32), (5, 1, 48), (14, 2, 64), (7, 7, 80), (28, 4, 128), (6, 2, 144),
                                      (2, 1, 256)])
def test_attention_mixed_batch(dtype, nh, kvh, d):
    # a whole prompt, a decoded token with a long cache, a portion in the middle of a prompt, a first token
    entries = [(0, 37), (300, 1), (45, 19), (0, 1), (16, 2)]
    got, ref = attention_case(dtype, nh, kvh, d, 16, 0, entries, seed=nh * 100 + d)
    assert rel_err(got, ref) < ATT_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page_size", [16, 32, 64])
def test_attention_page_sizes_and_edges(dtype, page_size):
    # lengths that end exactly on, one before and one after a page's edge
    entries = [(page_size - 1, 1), (page_size, 1), (page_size + 1, 1), (2 * page_size - 1, 3), (0, 2 * page_size)]
    got, ref = attention_case(dtype, 6, 2, 32, page_size, 0, entries, seed=page_size)
    assert rel_err(got, ref) < ATT_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page_size,window", [(32, 0), (48, 100), (64, 0), (128, 33)])
def test_attention_head_128_page_sizes(dtype, page_size, window):
    """Head size 128: the tiled kernel's waves bring one group of 16 keys each from the pages straight into LDS, and
    walk on by 64 keys without a division.  Pages that hold two, three, four and eight such groups; portions that
    begin in the middle of a page and of a group; a window that frees the pages behind it."""
    entries = [(0, 3 * page_size + 5), (page_size + 7, 300), (523, 90), (2 * page_size - 1, 1)]
    got, ref = attention_case(dtype, 14, 2, 128, page_size, window, entries, seed=page_size + window, spike=window > 0)
    assert rel_err(got, ref) < ATT_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("window", [1, 5, 16, 40])
def test_attention_window_edge(dtype, window):
    entries = [(0, 70), (130, 1), (window, 1), (window - 1, 1) if window > 1 else (0, 1), (20, 30)]
    got, ref = attention_case(dtype, 4, 2, 32, 16, window, entries, seed=window, spike=True)
    assert rel_err(got, ref) < ATT_TOL[dtype]


def test_attention_long_portion_bf16():
    """A portion of 700 tokens after 4,500 cached ones: more pages than the tiled kernel keeps ids for at a time."""
    entries = [(4500, 700), (0, 300)]
    got, ref = attention_case(torch.bfloat16, 4, 2, 32, 16, 0, entries, seed=5)
    assert rel_err(got, ref) < ATT_TOL[torch.bfloat16]
    got, ref = attention_case(torch.bfloat16, 2, 1, 64, 16, 600, [(3000, 400)], seed=6, spike=True)
    assert rel_err(got, ref) < ATT_TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_attention_far_key_among_hundreds(dtype):
    entries = [(700, 1), (0, 600), (513, 7)]
    got, ref = attention_case(dtype, 8, 2, 64, 16, 0, entries, seed=77, spike=True)
    assert rel_err(got, ref) < ATT_TOL[dtype]
    # the spiked key carries almost all the weight: output of the last token of entry 0 is its value
    assert abs(float(got[0, 0]) - 5.0) < 0.1


def test_attention_fp32_one_key_is_value_row_and_zero_query_is_mean():
    o = ops()
    g = torch.Generator().manual_seed(11)
    nh, kvh, d, t = 2, 1, 16, 9
    k = [torch.randn(t, kvh, d, generator=g)]
    v = [torch.randn(t, kvh, d, generator=g)]
    kp, vp, bt = make_pages(k, v, [t], 16, torch.float32, 5)
    q = torch.zeros(t, nh * d, device=DEV)
    out = torch.empty(t, nh * d, device=DEV)
    pos = torch.arange(t, dtype=torch.int32, device=DEV)
    o.attention_f32(q, kp.to(DEV), vp.to(DEV), pos, torch.zeros(t, dtype=torch.int32, device=DEV), bt.to(DEV), out, nh,
                    kvh, d, 0, 0.25)
    out = out.cpu().reshape(t, nh, d)
    assert torch.allclose(out[0, 0], v[0][0, 0], atol=1e-6)             # one key: the value row itself
    assert torch.allclose(out[5, 1], v[0][:6, 0].mean(0), atol=1e-6)    # zero query: mean of the allowed values


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nh,kvh,d,page_size", [(4, 2, 16, 16), (5, 1, 48, 32), (28, 4, 128, 16), (64, 8, 128, 16)])
@pytest.mark.parametrize("many", [False, True])
def test_rope_store(dtype, nh, kvh, d, page_size, many):
    """many: enough tokens for the kernel that takes sixteen tokens to a block and writes the values' page rows
    through LDS; portions that start at a page's edge (whole rows in one store) and in the middle of a page, a single
    token, a portion that ends in the middle of a group of sixteen."""
    from vt_transformer_amd.parts.rotary import rotary_table
    o = ops()
    g = torch.Generator().manual_seed(12)
    theta = 10000.0
    entries = [(0, 20), (33, 1), (page_size - 1, 3)]
    if many:
        entries = [(5, 70), (0, 48), (page_size - 3, 37), (64, 1), (2 * page_size, 21)]
    n = sum(x[1] for x in entries)
    width = (nh + 2 * kvh) * d
    qkv = torch.randn(n, width, generator=g)
    positions = torch.tensor([c + i for c, m in entries for i in range(m)], dtype=torch.int32)
    tok_entry = torch.tensor([e for e, (c, m) in enumerate(entries) for _ in range(m)], dtype=torch.int32)
    lens = [c + m for c, m in entries]
    n_pages = sum(-(-t // page_size) for t in lens) + 2
    perm = np.random.RandomState(3).permutation(n_pages)
    bt = torch.full((len(entries), 8), -1, dtype=torch.int32)
    nxt = 0
    for e, t in enumerate(lens):
        for b in range(-(-t // page_size)):
            bt[e, b] = int(perm[nxt]); nxt += 1
    cos, sin = rotary_table(256, d, theta)
    kp = torch.zeros(n_pages, kvh, page_size, d, dtype=dtype, device=DEV)
    vp = torch.zeros(n_pages, kvh, d, page_size, dtype=dtype, device=DEV)
    q_out = torch.empty(n, nh * d, dtype=dtype, device=DEV)
    o.rope_store(qkv.to(DEV), torch.from_numpy(cos).to(DEV), torch.from_numpy(sin).to(DEV), positions.to(DEV),
                 tok_entry.to(DEV), bt.to(DEV), q_out, kp, vp, nh, kvh, d)
    # reference: rotate-half pairs (i, i + d/2), float64 angles
    i = torch.arange(0, d, 2, dtype=torch.float64)
    ang = positions.double()[:, None] / torch.pow(torch.tensor(theta, dtype=torch.float64), i / d)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rot(x):
        x1, x2 = x[..., : d // 2].double(), x[..., d // 2:].double()
        return torch.cat([c * x1 - s * x2, c * x2 + s * x1], -1)
    q_ref = rot(qkv[:, : nh * d].reshape(n, nh, d)).reshape(n, nh * d)
    k_ref = rot(qkv[:, nh * d:(nh + kvh) * d].reshape(n, kvh, d))
    v_ref = qkv[:, (nh + kvh) * d:].reshape(n, kvh, d).double()
    tol = 2e-6 if dtype == torch.float32 else 5e-3
    assert rel_err(q_out, q_ref) < tol
    kp, vp = kp.cpu().double(), vp.cpu().double()
    for t in range(n):
        e, p = int(tok_entry[t]), int(positions[t])
        pg, slot = int(bt[e, p // page_size]), p % page_size
        assert rel_err(kp[pg, :, slot, :], k_ref[t]) < tol
        assert rel_err(vp[pg, :, :, slot], v_ref[t]) < tol
    # nothing else was written
    written = torch.zeros(n_pages, page_size, dtype=torch.bool)
    for t in range(n):
        e, p = int(tok_entry[t]), int(positions[t])
        written[int(bt[e, p // page_size]), p % page_size] = True
    assert float(kp.abs().sum(dim=(1, 3))[~written].sum()) == 0.0
    assert float(vp.abs().sum(dim=(1, 2))[~written].sum()) == 0.0


# ---------------------------------------------------------------------------
def test_sample_greedy_lowest_index_on_ties():
    o = ops()
    v = 1003
    logits = torch.zeros(3, v)
    logits[0, [17, 500, 900]] = 4.0
    logits[1, v - 1] = 1.0
    logits[2] = -1.0
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    o.sample(logits.to(DEV), torch.zeros(3, device=DEV), torch.full((3,), -1, dtype=torch.int32, device=DEV),
             torch.ones(3, device=DEV), torch.rand(3).to(DEV), torch.empty(3 * v, device=DEV), out)
    assert out.cpu().tolist() == [17, v - 1, 0]


def _draw(logits_row, temperature, top_k, top_p, n_draws, seed):
    o = ops()
    v = logits_row.numel()
    logits = logits_row.reshape(1, v).repeat(n_draws, 1).to(DEV)
    u = torch.rand(n_draws, generator=torch.Generator().manual_seed(seed)).to(DEV)
    out = torch.empty(n_draws, dtype=torch.int32, device=DEV)
    o.sample(logits, torch.full((n_draws,), temperature, device=DEV),
             torch.full((n_draws,), top_k, dtype=torch.int32, device=DEV), torch.full((n_draws,), top_p, device=DEV),
             u, torch.empty(n_draws * v, device=DEV), out)
    return out.cpu().long()


def test_sample_frequencies_match_softmax():
    g = torch.Generator().manual_seed(13)
    v = 37
    logits = torch.randn(v, generator=g) * 2
    n = 40000
    for temp in (0.7, 1.5):
        draws = _draw(logits, temp, -1, 1.0, n, seed=int(temp * 10))
        freq = torch.bincount(draws, minlength=v).double() / n
        p = torch.softmax(logits.double() / temp, 0)
        assert float((freq - p).abs().max()) < 4 * math.sqrt(0.25 / n) + 1e-3


def test_sample_top_k_and_top_p():
    g = torch.Generator().manual_seed(14)
    v = 500
    logits = torch.randn(v, generator=g) * 3
    p = torch.softmax(logits.double(), 0)
    order = torch.argsort(p, descending=True)
    draws = _draw(logits, 1.0, 3, 1.0, 5000, 1)          # the reference's own stochastic mode: the top three
    assert set(draws.tolist()) <= set(order[:3].tolist())
    freq = torch.bincount(draws, minlength=v).double()[order[:3]] / 5000
    assert float((freq - p[order[:3]] / p[order[:3]].sum()).abs().max()) < 0.03
    draws = _draw(logits, 1.0, -1, 0.5, 5000, 2)
    cum = torch.cumsum(p[order], 0)
    keep = int((cum < 0.5).sum()) + 1
    assert set(draws.tolist()) <= set(order[:keep].tolist())
    assert len(set(draws.tolist())) == keep or keep > 20
    # temperature towards zero is the argmax
    assert set(_draw(logits, 1e-4, -1, 1.0, 100, 3).tolist()) == {int(order[0])}
    # top_k = 1 is greedy whatever the temperature
    assert set(_draw(logits, 5.0, 1, 1.0, 100, 4).tolist()) == {int(order[0])}


@pytest.mark.parametrize("nh,kvh,d", [(28, 4, 128), (4, 2, 16), (16, 1, 48), (6, 2, 144)])   # 144: nine tiles of 16 dims
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("chunk", [64, 128, 1024])
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_attention_decode_kernel(nh, kvh, d, window, chunk, lp):
    """One token per entry, the keys cut into items on the device from the positions in memory."""
    o = ops()
    g = torch.Generator().manual_seed(nh + d + chunk)
    cached = [0, 15, 16, 17, 300, 63, 1000]
    lens = [c + 1 for c in cached]
    ks = [torch.randn(t, kvh, d, generator=g).to(lp).float() for t in lens]
    vs = [torch.randn(t, kvh, d, generator=g).to(lp).float() for t in lens]
    qs = [torch.randn(1, nh, d, generator=g).to(lp).float() for _ in lens]
    kp, vp, bt = make_pages(ks, vs, lens, 16, lp, 9)
    n = len(lens)
    q = torch.cat(qs).reshape(n, nh * d).to(lp).to(DEV)
    p_max = 16
    if -(-max(lens) // chunk) > p_max:
        pytest.skip("the host never chooses a chunk that needs more items than p_max")
    part_o = torch.full((n * p_max * kvh * 16 * d,), float("nan"), device=DEV)
    part_ml = torch.full((n * p_max * kvh * 32,), float("nan"), device=DEV)
    out = torch.full((n, nh * d), float("nan"), dtype=lp, device=DEV)
    scale = 1.0 / math.sqrt(d)
    o.attention_bf16_decode(q, kp.to(DEV), vp.to(DEV), bt.to(DEV), torch.tensor(cached, dtype=torch.int32, device=DEV),
                            torch.tensor([chunk, 0, 0, 0], dtype=torch.int32, device=DEV), p_max, out, part_o, part_ml,
                            nh, kvh, d, window, scale)
    ref = torch.cat([ref_attention(qs[e][0], ks[e], vs[e], cached[e], window, scale).reshape(1, -1) for e in range(n)])
    assert rel_err(out, ref) < ATT_TOL[lp]


@pytest.mark.parametrize("nh,kvh,d,rot", [(28, 4, 128, 128), (4, 2, 64, 32), (6, 2, 80, 0), (16, 1, 256, 256), (3, 1, 48, 32),
                                          (6, 2, 256, 256), (6, 2, 144, 128)])
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("chunk", [64, 1024])
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_attention_decode_fused_kernel(nh, kvh, d, rot, window, chunk, lp):
    """The decode attention that rotates and writes the pages itself against the separate rotation kernel followed
    by the plain decode attention, at two sets of positions."""
    o = ops()
    g = torch.Generator().manual_seed(nh + d + chunk + window)
    p_max, ps, max_pos = 16, 16, 1100
    half = rot // 2
    cos = sin = None
    if rot:
        ang = torch.rand(max_pos, half, generator=g, dtype=torch.float64) * 6.28
        cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    # (positions in every wave's first block of keys and in its second one: a wave asks for its first two blocks
    # before the token's own key and value are written, unless they hold them)
    for cached in ([0, 15, 16, 17, 300, 63, 1000], [31, 1, 999, 70, 119, 200]):
        n = len(cached)
        lens = [c + 1 for c in cached]
        ks = [torch.randn(t, kvh, d, generator=g).to(lp).float() for t in lens]
        vs = [torch.randn(t, kvh, d, generator=g).to(lp).float() for t in lens]
        kp, vp, bt = make_pages(ks, vs, lens, ps, lp, 9)
        kp, vp, bt = kp.to(DEV), vp.to(DEV), bt.to(DEV)
        # the last key and value of every entry come from the projection's row instead of the pages
        qkv = torch.randn(n, (nh + 2 * kvh) * d, generator=g).to(DEV)
        pos = torch.tensor(cached, dtype=torch.int32, device=DEV)
        tok_entry = torch.arange(n, dtype=torch.int32, device=DEV)
        kp_ref, vp_ref = kp.clone(), vp.clone()
        q_ref = torch.empty(n, nh * d, dtype=lp, device=DEV)
        o.rope_store(qkv, cos, sin, pos, tok_entry, bt, q_ref, kp_ref, vp_ref, nh, kvh, d)
        part_o = torch.full((n * p_max * kvh * 16 * d,), float("nan"), device=DEV)
        part_ml = torch.full((n * p_max * kvh * 32,), float("nan"), device=DEV)
        dec = torch.tensor([chunk, 0, 0, 0], dtype=torch.int32, device=DEV)
        scale = 1.0 / math.sqrt(d)
        out_ref = torch.full((n, nh * d), float("nan"), dtype=lp, device=DEV)
        o.attention_bf16_decode(q_ref, kp_ref, vp_ref, bt, pos, dec, p_max, out_ref, part_o.clone(), part_ml.clone(), nh, kvh,
                                d, window, scale)
        out = torch.full((n, nh * d), float("nan"), dtype=lp, device=DEV)
        o.attention_bf16_decode_fused(qkv, cos, sin, kp, vp, bt, pos, dec, p_max, out, part_o, part_ml, nh, kvh, d, window,
                                      scale)
        torch.cuda.synchronize()
        assert torch.equal(kp, kp_ref) and torch.equal(vp, vp_ref)       # the same bits in the pages
        assert bool(torch.isfinite(out.float()).all())
        assert rel_err(out, out_ref.float().cpu()) < 2e-3                 # the same products, merged in the same order


@pytest.mark.parametrize("d", list(range(16, 257, 16)))
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_attention_every_head_size(d, lp):
    """Every head size the kernels are compiled for, through every 16-bit attention kernel: portions (per-wave and
    tiled, keys split and unsplit), decoding, and decoding that rotates and writes the pages itself."""
    entries = [(0, 37), (300, 1), (45, 19), (0, 1), (16, 2), (0, 150)]
    got, ref = attention_case(lp, 6, 2, d, 16, 0, entries, seed=d)
    assert rel_err(got, ref) < ATT_TOL[lp]
    test_attention_decode_kernel(6, 2, d, 37, 128, lp)
    test_attention_decode_fused_kernel(6, 2, d, d if d % 32 == 0 else d - 16, 0, 64, lp)


@pytest.mark.parametrize("n,m,k", [(1, 48, 64), (8, 3584, 3584), (16, 100, 200), (5, 4608, 1000), (3, 40, 24)])
def test_linear_bf16_with_norm_in_front_and_residual_behind(n, m, k):
    """The few-row product that applies an RMSNorm to its input on the way and adds its result to the residual
    stream, against norm, product and addition in float64 from the same bfloat16 weights."""
    o = ops()
    g = torch.Generator().manual_seed(n * 7 + m + k)
    h = (torch.randn(n, k, generator=g) * 3).to(DEV)
    gain = (1 + 0.3 * torch.randn(k, generator=g)).to(DEV)
    w = (torch.randn(m, k, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    bias = torch.randn(m, generator=g).to(DEV)
    resid = torch.randn(n, m, generator=g).to(DEV)
    eps = 1e-5
    hd = h.double()
    normed = (gain.double() * hd) * torch.rsqrt((hd * hd).mean(-1, keepdim=True) + eps)
    ref = normed @ w.double().t() + bias.double()
    out = torch.empty(n, m, device=DEV)
    o.linear_bf16(h, w, bias, out, norm_gain=gain, norm_eps=eps)
    assert rel_err(out, ref) < 1e-2
    out2 = resid.clone()
    o.linear_bf16(h, w, None, out2, norm_gain=gain, norm_eps=eps, residual=out2)       # in place
    assert rel_err(out2, ref - bias.double() + resid.double()) < 1e-2
    x = normed.to(torch.bfloat16)
    out3 = resid.clone()
    o.linear_bf16(x, w, bias, out3, residual=out3)                                      # residual only
    assert rel_err(out3, x.double() @ w.double().t() + bias.double() + resid.double()) < 2e-3
    # the gated product with the norm in front
    inter = m
    wgu = (torch.randn(2 * inter, k, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    act = torch.empty(n, inter, device=DEV)
    o.gated_linear_bf16(h, wgu, act, norm_gain=gain, norm_eps=eps)
    gate, up = normed @ wgu[:inter].double().t(), normed @ wgu[inter:].double().t()
    assert rel_err(act, torch.nn.functional.silu(gate) * up) < 1e-2
    # more than 16 rows are refused
    with pytest.raises(Exception):
        o.linear_bf16(torch.zeros(17, k, device=DEV), w, None, torch.empty(17, m, device=DEV), norm_gain=gain, norm_eps=eps)


@pytest.mark.gpu
@pytest.mark.parametrize("nbytes, blocks", [(16, 1), (48 * 1024, 3), (1 << 20, 16), ((1 << 22) + 16 * 77, 256)])
def test_stream_read_reads_every_word_once(nbytes, blocks):
    # the kernel that measures the memory's ceiling: its checksum is the XOR of all words, tails included
    o = ops()
    rs = np.random.RandomState(nbytes % 1000)
    host = rs.randint(0, 1 << 31, size=nbytes // 4).astype(np.int32)
    buf = torch.from_numpy(host).cuda()
    sums = torch.zeros(blocks * 16, dtype=torch.int32, device="cuda")
    o.stream_read(buf, sums, blocks)
    got = np.bitwise_xor.reduce(sums.cpu().numpy().view(np.uint32))
    assert got == np.bitwise_xor.reduce(host.view(np.uint32))
    with pytest.raises(o.KernelError):
        o.stream_read(buf.view(torch.int16)[:4], sums, blocks)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,first", [(1, 0), (1000, 0), (70001, 12345), (3 * 257 * 129, 2 ** 33 + 5)])
def test_random_normal_kernel_makes_the_hosts_bits(dtype, n, first):
    """The device's counter-based generator against its numpy twin: equal to the bit, for matrices (mean 0) and
    gains (mean 1), at an offset beyond 32 bits too."""
    from vt_transformer_amd.weights.random_init import counter_normal, normal_scale
    for key, mean in ((0x0123456789ABCDEF, 0.0), (2 ** 64 - 3, 1.0)):
        out = torch.empty(n, dtype=dtype, device=DEV)
        ops().random_normal(out, key, normal_scale(0.02), mean, first=first)
        want = torch.from_numpy(counter_normal(key, first, n, 0.02, mean)).to(dtype)
        assert torch.equal(out.cpu(), want), (key, mean)


@pytest.mark.parametrize("n", [1, 5, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("h,k1,m2,gated", [(3584, 3584, 4608, False), (3584, 18944, 1184, True), (200, 96, 320, False),
                                           (1536, 8960, 2048, False), (8192, 512, 640, True), (72, 40, 56, True),
                                           (3584, 18944, 10240, False)])
@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_rmsnorm_handed_from_one_product_to_the_next(n, h, k1, m2, gated, lp):
    """A product that adds to the residual stream prepares the norm behind it (the stream times the gains in
    bfloat16, its blocks' shares of the rows' sums of squares); the product behind the norm takes those as its
    tokens and divides by the root.  Against the plain chain: add, RMSNorm, product.  Up to 16 rows a block per tile
    row produces; from 17 to 64 the kernel that keeps k inside a block, or the launch that adds the partial sums of a
    split k.  (Both 16-bit builds carry the kernels; the parts use them in bfloat16 only, because float16's range does
    not hold an un-normalised stream times gains: parts/linear.py, norm_inside_products.)"""
    o = ops()
    g = torch.Generator().manual_seed(n * 1000 + h)
    x = (torch.randn(n, k1, generator=g) * 0.5).to(lp)
    w1 = (torch.randn(h, k1, generator=g) * 0.05).to(lp)
    bias1 = torch.randn(h, generator=g) * 0.1
    resid = torch.randn(n, h, generator=g)
    gain = 1.0 + 0.1 * torch.randn(h, generator=g)
    w2 = (torch.randn((2 if gated else 1) * m2, h, generator=g) * 0.05).to(lp)
    eps = 1e-5
    shares, stride = o.linear_bf16_link_shares(n, h, k1), o.link_stride(n)
    assert shares > 0 and o.linear_bf16_adds_residual(n, h, k1)

    def workspace(rows, m, k):
        need = o.linear_bf16_workspace(rows, m, k) if rows > 16 else 0
        return torch.full((need,), float("nan"), device=DEV) if need else None
    hbuf = resid.clone().to(DEV)
    xn = torch.full((n, h), float("nan"), dtype=lp, device=DEV)
    ssq = torch.full((shares, stride), float("nan"), dtype=torch.float32, device=DEV)
    o.linear_bf16_link(x.to(DEV), o.pack_matrix_bf16(w1.to(DEV)), bias1.to(DEV), hbuf, residual=hbuf, xn_out=xn,
                       gain_next=gain.to(DEV), ssq_out=ssq, workspace=workspace(n, h, k1))
    h_ref = resid.double() + x.double() @ w1.double().t() + bias1.double()
    assert rel_err(hbuf, h_ref) < 1e-5
    assert rel_err(ssq[:, :n].sum(dim=0), (h_ref * h_ref).sum(dim=1)) < 1e-5
    assert bool((ssq[:, n:] == 0).all())
    # what the consumer reads: h * gain of the stream as the producer left it, rounded to 16 bits.  bfloat16: the very
    # bits of rounding the float32 product; float16: within half a unit in the last place of the product (the compiler
    # may round the product to 16 bits in one instruction, where the host rounds it to float32 first)
    prod = hbuf.cpu() * gain
    if lp == torch.bfloat16:
        assert torch.equal(xn.cpu(), prod.to(lp))
    else:
        assert bool(((xn.cpu().double() - prod.double()).abs() <= prod.double().abs() * 2.0 ** -11 * 1.001 + 2.0 ** -25).all())
    normed = xn.cpu().double() / torch.sqrt((h_ref * h_ref).mean(dim=1, keepdim=True) + eps)
    if gated:
        out = torch.empty(n, m2, dtype=torch.float32, device=DEV)
        o.gated_linear_bf16_link(xn, o.pack_matrix_bf16(w2.to(DEV), halves=2), out, ssq, eps)
        gate, up = normed @ w2[:m2].double().t(), normed @ w2[m2:].double().t()
        ref = gate / (1 + torch.exp(-gate)) * up
    else:
        bias2 = torch.randn(m2, generator=g) * 0.1
        out = torch.empty(n, m2, dtype=torch.float32, device=DEV)
        o.linear_bf16_link(xn, o.pack_matrix_bf16(w2.to(DEV)), bias2.to(DEV), out, ssq_in=ssq, eps_in=eps,
                           workspace=workspace(n, m2, h))
        ref = normed @ w2.double().t() + bias2.double()
    assert rel_err(out, ref) < 3e-5
    # and, up to 16 rows, the same as the product that applies the norm itself from the float32 stream
    if gated and n <= 16:
        same = torch.empty(n, m2, dtype=torch.float32, device=DEV)
        o.gated_linear_bf16(hbuf, o.pack_matrix_bf16(w2.to(DEV), halves=2), same, norm_gain=gain.to(DEV), norm_eps=eps)
        # (float16: the two kernels may round h * gain to 16 bits with different instructions, once or twice)
        assert rel_err(out, same) < (2e-6 if lp == torch.bfloat16 else 3e-5)


def test_rmsnorm_hand_over_is_refused_where_it_cannot_work():
    o = ops()
    assert o.linear_bf16_link_shares(65, 3584, 3584) == 0        # more than 64 rows
    assert o.linear_bf16_link_shares(8, 3584, 100) == 0          # k no multiple of 8
    assert o.linear_bf16_link_shares(8, 100, 64) == 0            # a width that the next product could not read by 16 bytes
    assert o.linear_bf16_link_shares(64, 152064, 3584) == 0      # many rows at 64 tokens: neither whole k in a block nor a split
    assert o.linear_bf16_link_shares(64, 3584, 18944) == 4       # k split over blocks: the adding launch, a share per 1,024 columns
    assert o.linear_bf16_link_shares(64, 3584, 3584) == 224 and o.linear_bf16_link_shares(64, 4608, 3584) == 144
    x = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    w = o.pack_matrix_bf16(torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV))
    out = torch.zeros(65, 32, device=DEV)
    ssq = torch.zeros(4, 64, device=DEV)
    with pytest.raises(Exception, match="up to 64 rows"):
        o.linear_bf16_link(x, w, None, out, ssq_in=ssq, eps_in=1e-6)
