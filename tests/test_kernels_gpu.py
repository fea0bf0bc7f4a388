"""Each kernel alone against its plain reference, at sizes other than the engine tests use."""

from __future__ import annotations

import math

import pytest
import torch

import plain_llama as pl
from tiny import ulps_of_row_max

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _ops():
    from nanospec_amd.kernels import ops

    return ops


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(dtype):
    ops = _ops()
    table = torch.randn(301, 72, dtype=dtype, device=DEV)
    ids = torch.tensor([0, 300, 5, 5, 17], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embed(table, ids), table[ids.long()])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim", [72, 1000, 4096])
def test_rmsnorm_plain_fused_and_gathered(dtype, dim):
    ops = _ops()
    torch.manual_seed(dim)
    n, eps = 7, 3e-6
    resid = torch.randn(n, dim, dtype=dtype, device=DEV) * 3
    x = torch.randn(n, dim, dtype=dtype, device=DEV)
    w = (1 + 0.1 * torch.randn(dim, device=DEV)).to(dtype)
    # plain
    ref = pl.rms_norm(resid.cpu(), w.cpu(), eps)
    torch.testing.assert_close(ops.rmsnorm(w, eps, resid=resid).cpu(), ref, **_tol(dtype))
    # fused sum, written back
    r2 = resid.clone()
    out = ops.rmsnorm(w, eps, resid=r2, x=x, write_resid=True)
    summed = pl.residual_add(resid.cpu(), x.cpu())
    assert torch.equal(r2.cpu(), summed)
    torch.testing.assert_close(out.cpu(), pl.rms_norm(summed, w.cpu(), eps), **_tol(dtype))
    # gathered rows, nothing written
    rows = torch.tensor([6, 0, 6, 3], dtype=torch.int32, device=DEV)
    r3 = resid.clone()
    out = ops.rmsnorm(w, eps, resid=r3, x=x, rows=rows)
    assert torch.equal(r3, resid)
    torch.testing.assert_close(out.cpu(), pl.rms_norm(summed, w.cpu(), eps)[rows.cpu().long()], **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 40, 24), (5, 130, 200), (8, 1003, 4096), (3, 7, 18), (70, 65, 17), (200, 300, 128)])
def test_linear_generic(dtype, m, n, k):
    ops = _ops()
    torch.manual_seed(m * n)
    x = torch.randn(m, k, dtype=dtype, device=DEV)
    w = torch.randn(n, k, dtype=dtype, device=DEV)
    ref = x.cpu().double() @ w.cpu().double().T
    # a 32-bit sum of K products is off by a few units in the last place of the sum of their magnitudes, not of the result
    bound = 2.0 ** -20 * (x.cpu().double().abs() @ w.cpu().double().abs().T)
    out = ops.linear_generic(x, w, out_f32=True)
    assert ((out.cpu().double() - ref).abs() <= bound).all()
    out2 = ops.linear_generic(x, w)
    if dtype == torch.float32:
        assert torch.equal(out2, out)
    else:
        torch.testing.assert_close(out2.cpu().float(), ref.to(dtype).float(), **_tol(dtype))
    ref = ref.float()
    # a row's result does not depend on the rows beside it (up to 8 rows of 32-bit x run a kernel of their own, whose sums
    # are ordered differently: compare within a kernel)
    few = 1 if m <= 8 or dtype != torch.float32 else 9
    assert torch.equal(ops.linear_generic(x[:few].contiguous(), w, out_f32=True), out[:few])
    if dtype == torch.float32 and m > 8:
        one = ops.linear_generic(x[:1].contiguous(), w, out_f32=True)
        torch.testing.assert_close(one, out[:1], rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("m", [1, 7, 16, 33, 64])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 4096), (257, 1064), (16, 8), (4096, 14336)])
def test_linear_tiled(m, n, k):
    """The streaming kernel on weights in the tiled layout: sizes that are no multiples of the tile, every wave count."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m, k, dtype=torch.bfloat16, device=DEV)
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    w2 = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt, wt2 = ops.TiledWeight(w), ops.TiledWeight(w2)
    ref = x.cpu().float() @ w.cpu().float().T
    for waves in (2, 4, 8):
        out = ops.linear_tiled(x, wt, out_f32=True, waves=waves)
        torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(k))
    assert ulps_of_row_max(ops.linear_tiled(x, wt).cpu(), ref).max() <= 1.0
    u = x.cpu().float() @ w2.cpu().float().T
    act = ops.linear_tiled(x, wt, w2=wt2)
    assert ulps_of_row_max(act.cpu(), ref * torch.sigmoid(ref) * u).max() <= 1.0
    if n >= 64:  # a slice of rows, as the stacked gate/up and q/k/v matrices are used
        part = ops.linear_tiled(x, wt.rows(16, 48), out_f32=True)
        torch.testing.assert_close(part.cpu(), ref[:, 16:48], rtol=1e-4, atol=1e-3 * math.sqrt(k))


@pytest.mark.parametrize("m", [1, 3, 8, 16])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 4096), (257, 1064), (14336, 512)])
def test_gated_product_in_half_tiles(m, n, k):
    """silu(x Wg^T) * (x Wu^T) with 8 rows of each matrix per workgroup: the same bits as with 16, at sizes off the tile."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m + 3, k + 8, dtype=torch.bfloat16, device=DEV)[:m, :k]
    wg, wu = (torch.randn(n, k, dtype=torch.bfloat16, device=DEV) * 0.3 for _ in range(2))
    tg, tu = ops.TiledWeight(wg), ops.TiledWeight(wu)
    g, u = x.cpu().float() @ wg.cpu().float().T, x.cpu().float() @ wu.cpu().float().T
    for waves in (2, 4, 8):
        whole = ops.linear_tiled(x, tg, w2=tu, waves=waves, halves=False)
        halves = ops.linear_tiled(x, tg, w2=tu, waves=waves, halves=True)
        assert torch.equal(whole, halves)
        assert ulps_of_row_max(halves.cpu(), g * torch.sigmoid(g) * u).max() <= 1.0


@pytest.mark.parametrize("m", [17, 33, 48, 64, 5])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 4096), (257, 1064), (4096, 14336)])
def test_linear_wide(m, n, k):
    """The kernel for 17 to 64 rows: x through LDS, K cut into ranges; every count of ranges, sizes off the tile."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m + 3, k + 8, dtype=torch.bfloat16, device=DEV)[:m, :k]  # a strided view of a wider buffer
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    w2 = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt, wt2 = ops.TiledWeight(w), ops.TiledWeight(w2)
    ref = x.cpu().float() @ w.cpu().float().T
    k_tiles = -(-k // 128)
    for ks in sorted({1, 2, min(5, k_tiles), k_tiles, 0} - {k_tiles + 1}):
        if ks > k_tiles:
            continue
        for nt in (1, 2):
            out = ops.linear_wide(x, wt, out_f32=True, ksplit=ks, nt=nt)
            torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(k))
    assert ulps_of_row_max(ops.linear_wide(x, wt).cpu(), ref).max() <= 1.0
    u = x.cpu().float() @ w2.cpu().float().T
    for nt in (1, 2):
        act = ops.linear_wide(x, wt, w2=wt2, nt=nt)
        assert ulps_of_row_max(act.cpu(), ref * torch.sigmoid(ref) * u).max() <= 1.0


@pytest.mark.parametrize("m", [17, 33, 48, 64, 5])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 4096), (257, 1064), (1440, 512)])
def test_linear_wide_dealt_to_the_compute_units(m, n, k):
    """The same kernel with three waves a workgroup (one matrix) and with gate and up by half tiles in workgroups of four
    or seven waves: every form adds a sum's terms in the same order, so the results are equal bit for bit."""
    ops = _ops()
    from nanospec_amd.kernels import KernelRefused

    torch.manual_seed(m + n + k + 1)
    x = torch.randn(m + 3, k + 8, dtype=torch.bfloat16, device=DEV)[:m, :k]
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    w2 = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt, wt2 = ops.TiledWeight(w), ops.TiledWeight(w2)
    ref = x.cpu().float() @ w.cpu().float().T
    k_tiles = -(-k // 128)
    for ks in sorted({1, 2, min(3, k_tiles)}):
        if ks > k_tiles:
            continue
        four = ops.linear_wide(x, wt, out_f32=True, ksplit=ks, nt=1, waves=4)
        three = ops.linear_wide(x, wt, out_f32=True, ksplit=ks, nt=1, waves=3)
        torch.testing.assert_close(three.cpu(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(k))
        assert torch.equal(three, four), f"{ks} ranges"
        if ks > 1:
            part = ops.linear_wide(x, wt, ksplit=ks, nt=1, waves=3, defer=True)
            assert torch.equal(ops.reduce_partial(part), ops.linear_wide(x, wt, ksplit=ks, nt=1, waves=4))
    u = x.cpu().float() @ w2.cpu().float().T
    whole = ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1, waves=4, halves=False)
    assert ulps_of_row_max(whole.cpu(), ref * torch.sigmoid(ref) * u).max() <= 1.0
    for waves in (4, 7):
        halves = ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1, waves=waves, halves=True)
        assert torch.equal(halves, whole), f"half tiles, {waves} waves"
    assert torch.equal(ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1), whole)  # whichever form the plan deals
    for bad in (dict(waves=7), dict(waves=3, w2=wt2), dict(waves=7, halves=True), dict(w2=wt2, waves=4, halves=True, ksplit=2),
                dict(waves=3, nt=2), dict(waves=5)):
        with pytest.raises(KernelRefused):
            ops.linear_wide(x, wt, **{"ksplit": 1, "nt": 1, **bad})


def test_wide_plans_deal_evenly():
    """What the plans choose at the three shapes' sizes on 256 compute units: q/k/v of the 8B shape in workgroups of three
    waves over two ranges (256 workgroups where four waves over three ranges are 288), gate and up by half tiles."""
    ops = _ops()
    assert ops.wide_plan(6144, 4096, 64, units=256) == (2, 1) and ops.wide_waves(6144, 4096, 64, 2, 1, units=256) == (3, False)
    assert ops.wide_plan(4096, 4096, 64, units=256) == (4, 1) and ops.wide_waves(4096, 4096, 64, 4, 1, units=256) == (4, False)
    assert ops.wide_plan(4096, 14336, 64, units=256) == (4, 1) and ops.wide_waves(4096, 14336, 64, 4, 1, units=256) == (4, False)
    assert ops.wide_waves(14336, 4096, 64, 1, 1, gated=True, units=256) == (7, True)   # 1,792 half tiles: 7 for each of 256 units
    assert ops.wide_waves(8192, 2048, 64, 1, 1, gated=True, units=256) == (4, True)    # 1,024 half tiles: 4 for each
    assert ops.wide_waves(28672, 8192, 64, 1, 1, gated=True, units=256) == (4, False)  # 448 workgroups of whole tiles fill the GPU
    assert ops.wide_waves(14336, 4096, 100, 1, 1, units=256) == (4, False)             # more than 64 rows of one matrix: four waves
    assert ops.wide_waves(14336, 4096, 100, 1, 1, gated=True, units=256) == (7, True)  # gate and up: half tiles only
    assert ops.wide_waves(8192, 2048, 100, 1, 1, gated=True, units=256) == (4, True)
    assert ops.wide_waves(14336, 4096, 64, 2, 1, gated=True, units=256) == (4, False)  # gate and up over ranges: whole tiles


def test_linear_tiled_refuses():
    ops = _ops()
    from nanospec_amd.kernels import KernelRefused

    w = torch.randn(16, 64, dtype=torch.bfloat16, device=DEV)
    wt = ops.TiledWeight(w)
    with pytest.raises(KernelRefused):
        ops.linear_tiled(torch.randn(65, 64, dtype=torch.bfloat16, device=DEV), wt)  # too many rows
    with pytest.raises(KernelRefused):
        ops.linear_tiled(torch.randn(4, 60, dtype=torch.bfloat16, device=DEV), wt)  # inner size differs
    with pytest.raises(KernelRefused):
        ops.linear_tiled(torch.randn(4, 64, dtype=torch.float32, device=DEV), wt)
    with pytest.raises(KernelRefused):
        ops.TiledWeight(w.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul(dtype):
    ops = _ops()
    gu = torch.randn(9, 2 * 88, dtype=dtype, device=DEV) * 3
    g, u = gu.cpu().float()[:, :88], gu.cpu().float()[:, 88:]
    torch.testing.assert_close(ops.silu_mul(gu).cpu().float(), (torch.nn.functional.silu(g) * u).to(dtype).float(), **_tol(dtype))


# ------------------------------------------------------------------------------------------------ cache helpers


def make_cache(pages, page, kvh, hd, dtype):
    k = torch.zeros(pages, kvh, page, hd, dtype=dtype, device=DEV)
    v = torch.zeros(pages, kvh, hd, page, dtype=dtype, device=DEV)
    return k, v


def scattered_tables(lens, page, pages, seed=0):
    """Block tables on scattered, non-contiguous pages."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(pages, generator=g).tolist()
    width = max(-(-n // page) for n in lens)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for b, n in enumerate(lens):
        for i in range(-(-n // page)):
            table[b, i] = perm.pop()
    return table


FORMS = [(False, 1.0), (True, 0.75)]  # (pairs of channels 2j and 2j + 1 instead of j and j + d/2, a factor on cosine and sine)


def plain_rotation(x, cos, sin, interleaved=False, factor=1.0):
    """The rotation of x [T, heads, d] in the given form.  The half-split form is the plain implementation's; the
    interleaved form turns channels 2j and 2j + 1 by the same angle j, written out here pair by pair."""
    if not interleaved:
        return pl.rotate(x, cos * factor, sin * factor)
    half = x.shape[-1] // 2
    c, s = (cos[:, None, :half] * factor), (sin[:, None, :half] * factor)
    a, b = x.float()[..., 0::2], x.float()[..., 1::2]
    out = torch.empty_like(x, dtype=torch.float32)
    out[..., 0::2] = a * c - b * s
    out[..., 1::2] = b * c + a * s
    return out.to(x.dtype)


@pytest.mark.parametrize("form", FORMS, ids=["halves", "interleaved"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rot", [24, 16, 0])
def test_rope_kv_write(dtype, rot, form):
    """q rotated in place, k rotated into its page slot, v into the transposed page; against the plain rotation."""
    ops = _ops()
    torch.manual_seed(1)
    heads, kvh, hd, page = 6, 3, 24, 4
    starts, lens = [0, 5, 9], [7, 1, 3]
    n = sum(lens)
    table = scattered_tables([s + l for s, l in zip(starts, lens)], page, 16).to(DEV)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
    qkv = torch.randn(n, (heads + 2 * kvh) * hd, dtype=dtype, device=DEV)
    before = qkv.clone().cpu()
    k, v = make_cache(16, page, kvh, hd, dtype)
    inv = pl.inverse_frequencies(rot, 10000.0, None) if rot else torch.zeros(1)
    ops.rope_kv_write(qkv, positions, token_req, table, inv.to(DEV), k, v, heads, kvh, hd, rot, interleaved=form[0], factor=form[1])
    q0 = before[:, : heads * hd].view(n, heads, hd)
    k0 = before[:, heads * hd : (heads + kvh) * hd].view(n, kvh, hd)
    v0 = before[:, (heads + kvh) * hd :].view(n, kvh, hd)
    if rot:
        cos, sin = pl.rotation_tables(positions.cpu(), inv)
        q_ref = torch.cat([plain_rotation(q0[..., :rot], cos, sin, *form), q0[..., rot:]], -1)
        k_ref = torch.cat([plain_rotation(k0[..., :rot], cos, sin, *form), k0[..., rot:]], -1)
    else:
        q_ref, k_ref = q0, k0
    tol = _tol(dtype)
    torch.testing.assert_close(qkv.cpu()[:, : heads * hd].view(n, heads, hd).float(), q_ref.float(), **tol)
    assert torch.equal(qkv.cpu()[:, heads * hd :], before[:, heads * hd :])  # k and v stay as they were in the buffer
    for t in range(n):
        b, p = int(token_req[t]), int(positions[t])
        pg, off = int(table[b, p // page]), p % page
        torch.testing.assert_close(k[pg, :, off].cpu().float(), k_ref[t].float(), **tol)
        assert torch.equal(v[pg, :, :, off].cpu(), v0[t])


@pytest.mark.parametrize("form", FORMS, ids=["halves", "interleaved"])
@pytest.mark.parametrize("heads,kvh,hd,rot,page", [(6, 3, 32, 32, 4), (4, 1, 48, 16, 8), (8, 2, 128, 128, 16), (2, 2, 16, 0, 4)])
def test_qkv_product_with_fused_rotation_and_cache_write(heads, kvh, hd, rot, page, form):
    """One kernel for x @ [Wq; Wk; Wv]^T, the rotation of q and k and the write of k and v into their pages, against the
    plain product followed by the plain rotation."""
    ops = _ops()
    torch.manual_seed(hd + rot)
    hidden = 72
    starts, lens = [3, 0, 9], [5, 1, 2]
    n = sum(lens)
    table = scattered_tables([s + l for s, l in zip(starts, lens)], page, 16, seed=2).to(DEV)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
    w = (torch.randn((heads + 2 * kvh) * hd, hidden) * 0.3).to(torch.bfloat16)
    x = torch.randn(n, hidden).to(torch.bfloat16)
    wt = ops.TiledWeight(w.to(DEV), ops.qkv_rope_row_order(heads, kvh, hd, rot, form[0]))
    q_out = torch.zeros(n, (heads + 2 * kvh) * hd, dtype=torch.bfloat16, device=DEV)
    k, v = make_cache(16, page, kvh, hd, torch.bfloat16)
    inv = pl.inverse_frequencies(rot, 10000.0, None) if rot else torch.zeros(1)
    ops.linear_qkv_rope(x.to(DEV), wt, q_out, positions, token_req, table, inv.to(DEV), k, v, heads, kvh, hd, rot, interleaved=form[0],
                        factor=form[1])
    full = x.float() @ w.float().T  # 32-bit sums: the kernel rotates before it rounds
    q0 = full[:, : heads * hd].view(n, heads, hd)
    k0 = full[:, heads * hd : (heads + kvh) * hd].view(n, kvh, hd)
    v0 = full[:, (heads + kvh) * hd :].view(n, kvh, hd)
    if rot:
        cos, sin = pl.rotation_tables(positions.cpu(), inv)
        q0 = torch.cat([plain_rotation(q0[..., :rot], cos, sin, *form), q0[..., rot:]], -1)
        k0 = torch.cat([plain_rotation(k0[..., :rot], cos, sin, *form), k0[..., rot:]], -1)
    assert ulps_of_row_max(q_out[:, : heads * hd].cpu(), q0.reshape(n, -1)).max() <= 1.0
    for t in range(n):
        b, p = int(token_req[t]), int(positions[t])
        pg, off = int(table[b, p // page]), p % page
        assert ulps_of_row_max(k[pg, :, off].cpu().reshape(1, -1), k0[t].reshape(1, -1)).max() <= 1.0
        assert ulps_of_row_max(v[pg, :, :, off].cpu().reshape(1, -1), v0[t].reshape(1, -1)).max() <= 1.0


@pytest.mark.parametrize("form", FORMS, ids=["halves", "interleaved"])
@pytest.mark.parametrize("rows", [17, 40, 64, 100, 128])
@pytest.mark.parametrize("heads,kvh,hd,rot,page,hidden,ksplit", [(6, 3, 32, 32, 4, 384, 3), (4, 1, 48, 16, 8, 520, 2), (8, 2, 128, 128, 16, 1024, 4),
                                                                 (2, 2, 16, 0, 4, 256, 2)])
def test_qkv_product_in_ranges_joined_by_the_rotation_kernel(rows, heads, kvh, hd, rot, page, hidden, ksplit, form):
    """17 to 128 rows: the stacked product with K cut into ranges from the matrix tiled in the few-row kernel's row order,
    and one kernel that adds the ranges, rotates q and k and writes k and v into their pages; against the plain product
    followed by the plain rotation.  Requests of several tokens and of one, pages scattered."""
    ops = _ops()
    torch.manual_seed(hd + rot + rows)
    lens = [rows - 9, 1, 5, 1, 2] if rows > 20 else [rows - 4, 1, 3]
    starts = [3, 0, 9, 30, 1][: len(lens)]
    n = sum(lens)
    assert n == rows
    table = scattered_tables([s + l for s, l in zip(starts, lens)], page, 64, seed=2).to(DEV)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
    w = (torch.randn((heads + 2 * kvh) * hd, hidden) * 0.3).to(torch.bfloat16)
    x = torch.randn(n, hidden).to(torch.bfloat16)
    wt = ops.TiledWeight(w.to(DEV), ops.qkv_rope_row_order(heads, kvh, hd, rot, form[0]))
    q_out = torch.zeros(n, (heads + 2 * kvh) * hd, dtype=torch.bfloat16, device=DEV)
    k, v = make_cache(64, page, kvh, hd, torch.bfloat16)
    inv = pl.inverse_frequencies(rot, 10000.0, None) if rot else torch.zeros(1)
    part = ops.linear_wide(x.to(DEV), wt, ksplit=ksplit, nt=1, defer=True)
    assert isinstance(part, ops.PartialSums) and part.ksplit == ksplit
    ops.rope_kv_from_partial(part, q_out, positions, token_req, table, inv.to(DEV), k, v, heads, kvh, hd, rot, interleaved=form[0],
                             factor=form[1])
    full = x.float() @ w.float().T  # 32-bit sums: the kernel rotates before it rounds
    q0 = full[:, : heads * hd].view(n, heads, hd)
    k0 = full[:, heads * hd : (heads + kvh) * hd].view(n, kvh, hd)
    v0 = full[:, (heads + kvh) * hd :].view(n, kvh, hd)
    if rot:
        cos, sin = pl.rotation_tables(positions.cpu(), inv)
        q0 = torch.cat([plain_rotation(q0[..., :rot], cos, sin, *form), q0[..., rot:]], -1)
        k0 = torch.cat([plain_rotation(k0[..., :rot], cos, sin, *form), k0[..., rot:]], -1)
    assert ulps_of_row_max(q_out[:, : heads * hd].cpu(), q0.reshape(n, -1)).max() <= 1.0
    assert torch.count_nonzero(q_out[:, heads * hd :]) == 0  # only q goes to the attention input
    for t in range(n):
        b, p = int(token_req[t]), int(positions[t])
        pg, off = int(table[b, p // page]), p % page
        assert ulps_of_row_max(k[pg, :, off].cpu().reshape(1, -1), k0[t].reshape(1, -1)).max() <= 1.0
        assert ulps_of_row_max(v[pg, :, :, off].cpu().reshape(1, -1), v0[t].reshape(1, -1)).max() <= 1.0
    # without the cache write only q is produced
    k2, v2 = make_cache(64, page, kvh, hd, torch.bfloat16)
    before = (k2.clone(), v2.clone())
    ops.rope_kv_from_partial(part, q_out, positions, token_req, table, inv.to(DEV), k2, v2, heads, kvh, hd, rot, write_kv=False)
    assert torch.equal(k2, before[0]) and torch.equal(v2, before[1])


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("hidden,inner", [(136, 264), (4096, 1024), (64, 8)])
def test_product_that_updates_the_residual_and_feeds_the_next_norm(m, hidden, inner):
    """resid += x @ W^T with what the following RMS norm needs as by-products, and the products that take them in place of a
    normalised input, against the plain sum, the plain norm and the plain product."""
    ops = _ops()
    torch.manual_seed(m + hidden)
    eps = 1e-5
    x = torch.randn(m, inner).to(torch.bfloat16)
    w = (torch.randn(hidden, inner) / math.sqrt(inner)).to(torch.bfloat16)
    resid0 = torch.randn(m, hidden).to(torch.bfloat16)
    w_norm = (1 + 0.2 * torch.randn(hidden)).to(torch.bfloat16)
    resid = resid0.to(DEV).clone()
    pre = ops.linear_resid_norm(x.to(DEV), ops.TiledWeight(w.to(DEV)), resid, w_norm.to(DEV), eps)
    # the sum: product rounded to bfloat16, then added in 32-bit and rounded (reference: model/llama.py:204-208)
    delta = (x.float() @ w.float().T).to(torch.bfloat16)
    want = (resid0.float() + delta.float()).to(torch.bfloat16)
    err = (resid.cpu().float() - want.float()).abs() / want.float().abs().clamp_min(0.25)
    assert err.max() <= 2.0 ** -6  # a flipped rounding of the product moves the sum by at most two of its last places
    got = resid.cpu()
    assert torch.equal(pre.x.cpu(), (got.float() * w_norm.float()).to(torch.bfloat16))
    assert pre.ssq.shape == (m, -(-hidden // 16))
    torch.testing.assert_close(pre.ssq.sum(1).cpu(), (got.float() ** 2).sum(-1), rtol=1e-5, atol=1e-6)
    # consumers: the plain norm of the kernel's own sum, then the plain products
    normed = pl.rms_norm(got, w_norm, eps)
    out_n = 152
    w3 = (torch.randn(out_n, hidden) / math.sqrt(hidden)).to(torch.bfloat16)
    w4 = (torch.randn(out_n, hidden) / math.sqrt(hidden)).to(torch.bfloat16)
    ref = normed.float() @ w3.float().T
    out = ops.linear_tiled(pre, ops.TiledWeight(w3.to(DEV)))
    assert ulps_of_row_max(out.cpu(), ref).max() <= 2.0
    out32 = ops.linear_tiled(pre, ops.TiledWeight(w3.to(DEV)), out_f32=True)
    assert ulps_of_row_max(out32.cpu(), ref).max() <= 1.0
    up = normed.float() @ w4.float().T
    act = ops.linear_tiled(pre, ops.TiledWeight(w3.to(DEV)), w2=ops.TiledWeight(w4.to(DEV)))
    assert ulps_of_row_max(act.cpu(), ref * torch.sigmoid(ref) * up).max() <= 2.0
    # the kernel that shares x through LDS takes the same input: whole tiles, half tiles in workgroups of 4 and 7 waves,
    # one matrix in workgroups of 3 and 4 waves
    t3, t4 = ops.TiledWeight(w3.to(DEV)), ops.TiledWeight(w4.to(DEV))
    for waves, halves in ((4, False), (4, True), (7, True)):
        act = ops.linear_wide(pre, t3, w2=t4, ksplit=1, nt=1, waves=waves, halves=halves)
        assert ulps_of_row_max(act.cpu(), ref * torch.sigmoid(ref) * up).max() <= 2.0, (waves, halves)
    for waves in (3, 4):
        assert ulps_of_row_max(ops.linear_wide(pre, t3, ksplit=1, nt=1, waves=waves, out_f32=True).cpu(), ref).max() <= 1.0
    if hidden >= 256:
        from nanospec_amd.kernels import KernelRefused

        with pytest.raises(KernelRefused):
            ops.linear_wide(pre, t3, ksplit=2, nt=1)  # a pre-normed input goes with one range


@pytest.mark.parametrize("m", [65, 81, 100, 113, 128])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 4096), (4096, 2056)])
def test_linear_wide_up_to_128_rows(m, n, k):
    """65 to 128 rows: one matrix, one row tile per wave; every count of ranges, sizes off the tile; other forms refused."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m + 3, k + 8, dtype=torch.bfloat16, device=DEV)[:m, :k]
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt = ops.TiledWeight(w)
    ref = x.cpu().float() @ w.cpu().float().T
    k_tiles = -(-k // 128)
    for ks in sorted({1, min(2, k_tiles), min(5, k_tiles), k_tiles, 0}):
        out = ops.linear_wide(x, wt, out_f32=True, ksplit=ks, nt=0 if ks == 0 else 1)
        torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(k))
    assert ulps_of_row_max(ops.linear_wide(x, wt).cpu(), ref).max() <= 1.0
    if k_tiles >= 2:
        part = ops.linear_wide(x, wt, ksplit=2, nt=1, defer=True)
        assert torch.equal(ops.reduce_partial(part), ops.linear_wide(x, wt, ksplit=2, nt=1))
    with pytest.raises(ops.KernelRefused):
        ops.linear_wide(x, wt, nt=2)
    with pytest.raises(ops.KernelRefused):
        ops.linear_wide(x, wt, w2=wt, ksplit=1, nt=1, waves=4, halves=False)  # whole tiles of two matrices: up to 64 rows
    with pytest.raises(ops.KernelRefused):
        ops.linear_wide(torch.randn(129, k, dtype=torch.bfloat16, device=DEV), wt)
    # gate and up by half tiles hold one set of sums, so they take these rows too
    w2 = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt2 = ops.TiledWeight(w2)
    want = ref * torch.sigmoid(ref) * (x.cpu().float() @ w2.cpu().float().T)
    seven = ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1, waves=7, halves=True)
    assert ulps_of_row_max(seven.cpu(), want).max() <= 1.0
    assert torch.equal(ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1, waves=4, halves=True), seven)
    assert torch.equal(ops.linear_wide(x, wt, w2=wt2, ksplit=1, nt=1), seven)  # (the form the plan deals: one of the two)
    assert torch.equal(seven[:64], ops.linear_wide(x[:64], wt, w2=wt2, ksplit=1, nt=1, waves=4, halves=False))


@pytest.mark.parametrize("m", [129, 300, 1031])
@pytest.mark.parametrize("n,k", [(48, 64), (130, 200), (1000, 2056), (4096, 1024)])
def test_linear_rows(m, n, k):
    """Any number of rows in blocks of 128 (what a model that keeps the tiled layout only runs its prompts through): every
    count of row tiles per wave and several counts of ranges, sizes off every tile, the gated form, 32-bit results."""
    ops = _ops()
    torch.manual_seed(m + n + k)
    x = torch.randn(m + 3, k + 8, dtype=torch.bfloat16, device=DEV)[:m, :k]
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    w2 = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    wt, wt2 = ops.TiledWeight(w), ops.TiledWeight(w2)
    ref = x.cpu().float() @ w.cpu().float().T
    k_tiles = -(-k // 128)
    for nt in (2, 4):
        for ks in sorted({1, min(3, k_tiles), 0}):
            out = ops.linear_rows(x, wt, out_f32=True, ksplit=ks, nt=nt if ks else 0)
            torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-3 * math.sqrt(k))
    assert ulps_of_row_max(ops.linear_rows(x, wt).cpu(), ref).max() <= 1.0
    u = x.cpu().float() @ w2.cpu().float().T
    for nt in (1, 2):
        for ks in (1, min(2, k_tiles)):
            act = ops.linear_rows(x, wt, w2=wt2, ksplit=ks, nt=nt)
            assert ulps_of_row_max(act.cpu(), ref * torch.sigmoid(ref) * u).max() <= 1.0
    with pytest.raises(ops.KernelRefused):
        ops.linear_rows(x, wt, nt=1)


@pytest.mark.parametrize("m", [17, 40, 64, 97, 128])
@pytest.mark.parametrize("hidden,inner,ksplit", [(136, 1024, 4), (4096, 1024, 2), (72, 512, 3)])
def test_ranges_of_a_product_added_by_the_norm_that_reads_them(m, hidden, inner, ksplit):
    """The 17-to-64-row product leaves the ranges of K unadded; the RMS norm adds them as it reads them, with the residual
    sum and with a row gather; ``reduce_partial`` gives the same tensor as the product run whole."""
    ops = _ops()
    torch.manual_seed(m + hidden)
    eps = 1e-5
    x = torch.randn(m, inner).to(torch.bfloat16).to(DEV)
    w = (torch.randn(hidden, inner) / math.sqrt(inner)).to(torch.bfloat16).to(DEV)
    wt = ops.TiledWeight(w)
    resid0 = torch.randn(m, hidden).to(torch.bfloat16)
    w_norm = (1 + 0.2 * torch.randn(hidden)).to(torch.bfloat16)
    part = ops.linear_wide(x, wt, ksplit=ksplit, nt=1, defer=True)
    assert isinstance(part, ops.PartialSums) and part.ws.numel() >= ksplit * m * hidden
    whole = ops.linear_wide(x, wt, ksplit=ksplit, nt=1)
    assert torch.equal(ops.reduce_partial(part), whole)
    # sum + norm
    resid = resid0.to(DEV).clone()
    out = ops.rmsnorm(w_norm.to(DEV), eps, resid=resid, x=part, write_resid=True)
    resid_ref = resid0.to(DEV).clone()
    ref = ops.rmsnorm(w_norm.to(DEV), eps, resid=resid_ref, x=whole, write_resid=True)
    assert torch.equal(resid, resid_ref)
    assert ulps_of_row_max(out.cpu(), ref.cpu().float()).max() <= 1.0
    want = pl.rms_norm((resid0.float() + whole.cpu().float()).to(torch.bfloat16), w_norm, eps)
    assert ulps_of_row_max(out.cpu(), want.float()).max() <= 1.0
    # gathered rows, no residual
    rows = torch.tensor([m - 1, 0, 5], dtype=torch.int32, device=DEV)
    got = ops.rmsnorm(w_norm.to(DEV), eps, x=part, rows=rows)
    want = pl.rms_norm(whole.cpu()[rows.cpu().long()], w_norm, eps)
    assert ulps_of_row_max(got.cpu(), want.float()).max() <= 1.0


def test_qkv_product_takes_a_prenormed_input():
    ops = _ops()
    torch.manual_seed(3)
    heads, kvh, hd, rot, page, hidden, eps = 6, 2, 32, 32, 8, 96, 1e-6
    starts, lens = [3, 0, 9], [5, 1, 2]
    n = sum(lens)
    table = scattered_tables([s + l for s, l in zip(starts, lens)], page, 16, seed=2).to(DEV)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
    r = torch.randn(n, hidden).to(torch.bfloat16)
    w_norm = (1 + 0.2 * torch.randn(hidden)).to(torch.bfloat16)
    w = (torch.randn((heads + 2 * kvh) * hd, hidden) * 0.3).to(torch.bfloat16)
    wt = ops.TiledWeight(w.to(DEV), ops.qkv_rope_row_order(heads, kvh, hd, rot))
    inv = pl.inverse_frequencies(rot, 10000.0, None).to(DEV)
    ssq = torch.zeros(n, 3)
    ssq[:, 1] = (r.float() ** 2).sum(-1)  # any split into parts has the same sum
    pre = ops.PreNormed((r.float() * w_norm.float()).to(torch.bfloat16).to(DEV), ssq.to(DEV), hidden, eps)
    outs = []
    for src in (pre, pl.rms_norm(r, w_norm, eps).to(DEV)):
        q_out = torch.zeros(n, heads * hd, dtype=torch.bfloat16, device=DEV)
        k, v = make_cache(16, page, kvh, hd, torch.bfloat16)
        ops.linear_qkv_rope(src, wt, q_out, positions, token_req, table, inv, k, v, heads, kvh, hd, rot)
        outs.append((q_out.cpu(), k.cpu(), v.cpu()))
    for a, b in zip(*outs):
        assert ulps_of_row_max(a.reshape(1, -1), b.reshape(1, -1).float()).max() <= 2.0
    assert outs[0][1].abs().sum() > 0


def fill_cache(k, v, table, lens, page, kvh, hd, dtype, seed=0, scale=1.0):
    """Random keys and values for positions [0, len) of every request, written through the block table.
    -> per request (K [len, kvh, hd], V [len, kvh, hd]) on the CPU."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for b, n in enumerate(lens):
        kk = (torch.randn(n, kvh, hd, generator=g) * scale).to(dtype)
        vv = torch.randn(n, kvh, hd, generator=g).to(dtype)
        for p in range(n):
            pg, off = int(table[b, p // page]), p % page
            if pg < 0:
                continue
            k[pg, :, off] = kk[p].to(DEV)
            v[pg, :, :, off] = vv[p].to(DEV)
        out.append((kk, vv))
    return out


def plain_paged_attention(q, kvs, starts, lens, heads, scale_fix=1.0, window=0):
    """Rows of q (flat over requests) attend to their request's keys 0 .. position with the plain attention."""
    outs, at = [], 0
    for (kk, vv), s, n in zip(kvs, starts, lens):
        qi = q[at : at + n]
        o = pl.causal_attention(qi.cpu(), kk[: s + n], vv[: s + n], first_query=s)
        if window:
            o = torch.stack([pl.causal_attention(qi[i : i + 1].cpu(), kk[max(0, s + i - window + 1) : s + i + 1],
                                                 vv[max(0, s + i - window + 1) : s + i + 1], first_query=min(s + i, window - 1))[0]
                             for i in range(n)])
        outs.append(o)
        at += n
    return torch.cat(outs)


CASES = {
    # the four cases of the reference's tests/test_backends.py:44-59
    "prefill": ([0], [40]),
    "decode": ([37], [1]),
    "append6": ([37], [6]),
    "mixed": ([21, 50, 0], [1, 6, 9]),
    "long": ([300, 0, 511], [1, 70, 1]),
    # more than 64 pages a request at every page size: the kernels hold 64 page ids at a time
    "beyond64pages": ([1300, 0], [1, 1100]),
    # a decode row and a late portion of a prompt nine thousand tokens in: many reloads of the page ids, long key ranges
    "far": ([9000, 8990], [1, 70]),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("heads,kvh,hd,page", [(8, 2, 128, 16), (6, 1, 48, 4), (4, 4, 16, 8)])
def test_attention_generic(dtype, case, heads, kvh, hd, page):
    ops = _ops()
    starts, lens = CASES[case]
    torch.manual_seed(3)
    total = [s + l for s, l in zip(starts, lens)]
    pages = sum(-(-t // page) for t in total) + 3
    table = scattered_tables(total, page, pages)
    k, v = make_cache(pages, page, kvh, hd, dtype)
    kvs = fill_cache(k, v, table, total, page, kvh, hd, dtype)
    n = sum(lens)
    q = torch.randn(n, heads * hd, dtype=dtype, device=DEV)
    positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
    token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
    out = torch.empty(n, heads * hd, dtype=dtype, device=DEV)
    ops.attention_generic(q, out, k, v, token_req, positions, table.to(DEV), heads, kvh, hd, 1 / math.sqrt(hd))
    ref = plain_paged_attention(q.view(n, heads, hd), kvs, starts, lens, heads).reshape(n, -1)
    if dtype == torch.float32:
        torch.testing.assert_close(out.cpu(), ref, rtol=1e-4, atol=1e-5)
    else:
        assert ulps_of_row_max(out.cpu(), ref).max() <= 4  # the reference's bound, tests/test_backends.py:71


@pytest.mark.parametrize("n,k", [(16, 128), (40, 72), (100, 264), (2048, 8192), (33, 8)])
def test_untile_gives_the_matrix_back(n, k):
    """The re-laid copy of a matrix written out in plain rows again (rows and k that are no multiples of the tile: the
    padding is not written, and nothing outside the matrix is)."""
    ops = _ops()
    torch.manual_seed(n + k)
    w = torch.randn(n, k, dtype=torch.bfloat16, device=DEV)
    guard = torch.full((n + 2, k), 7.0, dtype=torch.bfloat16, device=DEV)
    out = ops.untile(ops.TiledWeight(w), guard[1:-1])
    assert torch.equal(out, w)
    assert bool((guard[0] == 7).all()) and bool((guard[-1] == 7).all())
    with pytest.raises(ops.KernelRefused):
        ops.untile(ops.TiledWeight(w), torch.empty(n, k + 8, dtype=torch.bfloat16, device=DEV))
    if k > 128:  # a range of columns, into rows that are further apart than they are long
        k0, k1 = 128, k if k < 384 else 384
        wide = torch.full((n, k1 - k0 + 16), 7.0, dtype=torch.bfloat16, device=DEV)
        ops.untile(ops.TiledWeight(w), wide[:, : k1 - k0], k0, k1)
        assert torch.equal(wide[:, : k1 - k0], w[:, k0:k1]) and bool((wide[:, k1 - k0 :] == 7).all())
        with pytest.raises(ops.KernelRefused):
            ops.untile(ops.TiledWeight(w), wide[:, : k1 - k0 - 8], k0 + 8, k1)


def _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, window=0, force_splits=None, qt=2, coop=False, step_keys=0,
              chunk_splits=1, short_offsets=True, spare_tiles=0):
    n = sum(lens)
    indptr = [0]
    for l in lens:
        indptr.append(indptr[-1] + l)
    out = torch.zeros(n, heads * hd, dtype=torch.bfloat16, device=DEV)
    group = heads // kvh
    tile = lambda b, t0: [b, t0, indptr[b], lens[b], starts[b] + lens[b], 0, 0, 0]
    ct = [tile(b, t0) for b, l in enumerate(lens) if l != 1 for t0 in range(0, l, 16 * qt)]
    ct += [[len(lens) - 1, 0, 0, 0, 0, 0, 0, 0]] * (spare_tiles if ct else 0)  # tiles without tokens, as a captured step's spare ones
    dt = [tile(b, 0) for b, l in enumerate(lens) if l == 1]
    for t in dt:
        t[5] = step_keys  # the keys all decode rows of the step read: from some number on the kernel reads them past the cache
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    if ct:
        cols = len(ct) * 16 * qt * heads
        ws = None
        if chunk_splits > 1:  # filled with NaN: a range that is read without having been written shows
            ws = (torch.full((cols * chunk_splits * hd,), float("nan"), device=DEV), torch.full((cols * chunk_splits * 2,), float("nan"), device=DEV))
        ops.attention_mfma(q, out, k, v, i32(ct), table.to(DEV), heads, kvh, hd, 1 / math.sqrt(hd), window=window, hp=1,
                           splits=chunk_splits, workspace=ws, qt=qt, coop=coop and qt == 2,  # coop: one set of waves per workgroup
                           short_offsets=short_offsets)
    if dt:
        hp = 1
        while hp < min(group, 16):
            hp *= 2
        splits = force_splits or 3
        cols = len(dt) * (16 // hp) * heads
        # filled with NaN: a range (an empty one, say: with more than 16 the later ones are, below 8,192 keys) that is read
        # without having been written shows
        ws = (torch.full((cols * splits * hd,), float("nan"), device=DEV), torch.full((cols * splits * 2,), float("nan"), device=DEV))
        ops.attention_mfma(q, out, k, v, i32(dt), table.to(DEV), heads, kvh, hd, 1 / math.sqrt(hd), window=window, hp=hp,
                           splits=splits, workspace=ws if splits > 1 else None, coop=coop)
    return out


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("heads,kvh,hd,page", [(8, 2, 128, 16), (6, 1, 48, 4), (4, 4, 16, 8), (32, 8, 64, 16), (40, 2, 32, 16)])
def test_attention_mfma(case, heads, kvh, hd, page):
    ops = _ops()
    starts, lens = CASES[case]
    torch.manual_seed(4)
    total = [s + l for s, l in zip(starts, lens)]
    pages = sum(-(-t // page) for t in total) + 3
    table = scattered_tables(total, page, pages, seed=1)
    k, v = make_cache(pages, page, kvh, hd, torch.bfloat16)
    kvs = fill_cache(k, v, table, total, page, kvh, hd, torch.bfloat16, seed=2)
    n = sum(lens)
    q = torch.randn(n, heads * hd, dtype=torch.bfloat16, device=DEV)
    ref = plain_paged_attention(q.view(n, heads, hd), kvs, starts, lens, heads).reshape(n, -1)
    # the last number: ranges that the keys of a prompt portion's tiles are cut into (16: more than most tiles have blocks)
    for splits, qt, coop, step_keys, chunk_splits in ((1, 2, False, 0, 1), (3, 1, False, 0, 2), (7, 2, True, 0, 3), (33, 1, False, 2**30, 1),
                                                      (1, 1, True, 2**30, 5), (2, 2, True, 0, 16), (1, 2, True, 0, 1)):
        out = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, force_splits=splits, qt=qt, coop=coop, step_keys=step_keys,
                        chunk_splits=chunk_splits)
        u = ulps_of_row_max(out.cpu(), ref).max()
        assert u <= 4, f"{case} splits={splits} qt={qt} coop={coop} chunk_splits={chunk_splits}: {u:.2f} ulps"


# The prompt kernel for head sizes 64 and 128 brings keys and values straight into LDS, a page id per page of a block of
# 32 keys: every page size it takes (four, two, one page a block, a block inside a page), a group of three heads (a wave
# of the workgroup has no head), a group of eight (two workgroups a key/value head), and addresses of 64 bits.
@pytest.mark.parametrize("case", ["prefill", "mixed", "long", "beyond64pages", "far"])
@pytest.mark.parametrize("heads,kvh,hd,page,short_offsets", [(8, 2, 128, 8, True), (8, 2, 128, 32, True), (16, 4, 64, 64, True), (4, 1, 64, 8, False),
                                                             (6, 2, 128, 16, True), (8, 1, 128, 16, False), (4, 2, 64, 128, False)])
def test_attention_mfma_prompt_kernel_page_sizes_and_groups(case, heads, kvh, hd, page, short_offsets):
    ops = _ops()
    starts, lens = CASES[case]
    torch.manual_seed(14)
    total = [s + l for s, l in zip(starts, lens)]
    pages = sum(-(-t // page) for t in total) + 3
    table = scattered_tables(total, page, pages, seed=3)
    k, v = make_cache(pages, page, kvh, hd, torch.bfloat16)
    kvs = fill_cache(k, v, table, total, page, kvh, hd, torch.bfloat16, seed=4)
    n = sum(lens)
    q = torch.randn(n, heads * hd, dtype=torch.bfloat16, device=DEV)
    ref = plain_paged_attention(q.view(n, heads, hd), kvs, starts, lens, heads).reshape(n, -1)
    for coop, chunk_splits in ((False, 1), (True, 1), (True, 3), (False, 16)):
        out = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, qt=2, coop=coop, chunk_splits=chunk_splits, short_offsets=short_offsets,
                        spare_tiles=3 if chunk_splits in (1, 3) else 0)
        u = ulps_of_row_max(out.cpu(), ref).max()
        assert u <= 4, f"{case} coop={coop} chunk_splits={chunk_splits}: {u:.2f} ulps"


def test_attention_prompt_kernel_in_use():
    """Head sizes 64 and 128 with pages of 8 tokens or more run the 32x32 prompt kernel (it steps aside if it was ever
    compiled with scratch memory: then this fails, and says that the tests above did not run it), the other sizes
    the kernels they are made for."""
    ops = _ops()
    for hd, page in ((64, 8), (64, 16), (64, 64), (64, 128), (128, 8), (128, 16), (128, 32)):
        assert ops.attention_prompt_form(hd, page) == 32, (hd, page)
    assert ops.attention_prompt_form(32, 16) == 16 and ops.attention_prompt_form(96, 16) == 16
    assert ops.attention_prompt_form(48, 4) == 0 and ops.attention_prompt_form(144, 16) == 0


@pytest.mark.parametrize("hd,page", [(128, 16), (64, 8), (128, 32)])
@pytest.mark.parametrize("coop", [False, True])
def test_attention_prompt_dominant_key_at_block_and_ring_edges(hd, page, coop):
    """A prompt portion of 70 tokens over some hundred keys; one key is made to dominate every query that sees it, so
    their outputs must be its value.  Done for keys around the edges of the kernel's blocks of 32 keys, of its ring of
    three buffers (96 keys), of the pages, of the halves that two sets of waves take, and inside the portion itself, where
    only later tokens see the key."""
    ops = _ops()
    heads, kvh = 8, 2
    n, total, dtype = 70, 430, torch.bfloat16
    start = total - n
    pages = -(-total // page) + 2
    table = scattered_tables([total], page, pages, seed=6)
    torch.manual_seed(9)
    base = torch.randn(heads * hd, dtype=dtype, device=DEV)
    q = base.repeat(n, 1).contiguous()  # every token asks the same
    for special in (0, 1, 31, 32, 33, 63, 64, 95, 96, 97, 127, 128, 191, 192, 193, 215, 216, 287, 288, 359, 360, 361, 383, 384, 400, 428, 429):
        k, v = make_cache(pages, page, kvh, hd, dtype)
        kvs = fill_cache(k, v, table, [total], page, kvh, hd, dtype, seed=special, scale=0.05)
        pg, off = int(table[0, special // page]), special % page
        for h in range(kvh):
            k[pg, h, off] = (base.view(heads, hd)[h * (heads // kvh)] * 4).to(dtype)  # aligned with the group's first query head
        kvs[0][0][special] = k[pg, :, off].cpu()
        out = _run_mfma(ops, q, k, v, table, [start], [n], heads, kvh, hd, qt=2, coop=coop).view(n, heads, hd).float().cpu()
        ref = plain_paged_attention(q.view(n, heads, hd), kvs, [start], [n], heads).reshape(n, -1)
        assert ulps_of_row_max(out.reshape(n, -1), ref).max() <= 4, f"key {special}"
        for h in range(kvh):
            want = kvs[0][1][special, h].float()
            for t in range(n):
                if start + t >= special:
                    assert torch.allclose(out[t, h * (heads // kvh)], want, atol=0.05), f"key {special}, token {t}: output is not its value"


@pytest.mark.parametrize("kernel", ["generic", "mfma"])
def test_attention_far_key_and_page_edges(kernel):
    """One key among hundreds is made to dominate: its score stands out, so the output must be its value.
    Done for a key at every offset around page edges, so that a wrong page or slot shows."""
    ops = _ops()
    heads, kvh, hd, page = 4, 2, 32, 8
    total, dtype = 333, torch.bfloat16
    pages = -(-total // page) + 2
    table = scattered_tables([total], page, pages, seed=5)
    for special in (0, 7, 8, 9, 15, 16, 255, 256, 320, 331, 332):
        k, v = make_cache(pages, page, kvh, hd, dtype)
        kvs = fill_cache(k, v, table, [total], page, kvh, hd, dtype, seed=special, scale=0.05)
        q = torch.randn(1, heads * hd, dtype=dtype, device=DEV)
        pg, off = int(table[0, special // page]), special % page
        for h in range(kvh):
            k[pg, h, off] = (q.view(heads, hd)[h * (heads // kvh)] * 4).to(dtype)  # aligned with the group's first query head
        starts, lens = [total - 1], [1]
        if kernel == "mfma":
            out = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd)
        else:
            out = torch.empty_like(q)
            ops.attention_generic(q, out, k, v, torch.zeros(1, dtype=torch.int32, device=DEV),
                                  torch.tensor([total - 1], dtype=torch.int32, device=DEV), table.to(DEV), heads, kvh, hd, 1 / math.sqrt(hd))
        for h in range(kvh):
            got = out.view(heads, hd)[h * (heads // kvh)].float().cpu()
            want = kvs[0][1][special, h].float()
            assert torch.allclose(got, want, atol=0.05), f"key {special}: output is not its value"


@pytest.mark.parametrize("kernel", ["generic", "mfma"])
@pytest.mark.parametrize("window", [5, 16, 40])
@pytest.mark.parametrize("hd,page", [(32, 8), (128, 16), (64, 8)])  # (the prompt kernels: one for head sizes 64 and 128, one for the others)
def test_attention_window(kernel, window, hd, page):
    ops = _ops()
    heads, kvh = 4, 2
    starts, lens = [50, 0, 100], [1, 45, 20]
    dtype = torch.bfloat16
    total = [s + l for s, l in zip(starts, lens)]
    pages = sum(-(-t // page) for t in total) + 2
    table = scattered_tables(total, page, pages, seed=7)
    k, v = make_cache(pages, page, kvh, hd, dtype)
    kvs = fill_cache(k, v, table, total, page, kvh, hd, dtype, seed=8)
    # pages wholly before every query's window are released: the kernel must not touch them
    for b, (s, l) in enumerate(zip(starts, lens)):
        first_needed = max(0, s - window + 1) // page
        table[b, :first_needed] = -1
    n = sum(lens)
    q = torch.randn(n, heads * hd, dtype=dtype, device=DEV)
    ref = plain_paged_attention(q.view(n, heads, hd), kvs, starts, lens, heads, window=window).reshape(n, -1)
    if kernel == "mfma":
        out = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, window=window)
        cut = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, window=window, chunk_splits=3)
        assert ulps_of_row_max(cut.cpu(), ref).max() <= 4
        cut = _run_mfma(ops, q, k, v, table, starts, lens, heads, kvh, hd, window=window, chunk_splits=2, coop=True)
        assert ulps_of_row_max(cut.cpu(), ref).max() <= 4
    else:
        positions = torch.tensor([s + i for s, l in zip(starts, lens) for i in range(l)], dtype=torch.int32, device=DEV)
        token_req = torch.tensor([b for b, l in enumerate(lens) for _ in range(l)], dtype=torch.int32, device=DEV)
        out = torch.empty(n, heads * hd, dtype=dtype, device=DEV)
        ops.attention_generic(q, out, k, v, token_req, positions, table.to(DEV), heads, kvh, hd, 1 / math.sqrt(hd), window=window)
    assert ulps_of_row_max(out.cpu(), ref).max() <= 4


def test_sample_greedy_and_temperature():
    ops = _ops()
    torch.manual_seed(0)
    rows, vocab = 6, 1003
    z = torch.randn(rows, vocab, device=DEV) * 3
    z[2, 100] = z[2, 900] = z[2].max() + 1  # a tie: the lowest index wins
    T = torch.tensor([0.0, 0.8, 0.0, 1.0, 0.7, 1.3], device=DEV)
    u = torch.tensor([0.3, 0.9, 0.5, 0.0, 0.5, 0.9999], device=DEV)
    tok, lp, slp = ops.unpack_sample(ops.sample(z, T, u))
    zc = z.cpu()
    for r in range(rows):
        t = float(T[r])
        if t == 0:
            assert int(tok[r]) == int(zc[r].argmax()) or r == 2
            assert float(slp[r]) == 0.0
        else:
            ref = pl.draw_token(pl.processed_logprobs(zc[r], t, 0, 1.0), float(u[r]))
            assert abs(int(tok[r]) - ref) <= 1, (r, int(tok[r]), ref)  # the cumulative sums round differently
            assert abs(float(slp[r]) - float(pl.processed_logprobs(zc[r], t, 0, 1.0)[int(tok[r])])) < 1e-4
        assert abs(float(lp[r]) - float(torch.log_softmax(zc[r], -1)[int(tok[r])])) < 1e-4
    assert int(tok[2]) == 100


@pytest.mark.parametrize("vocab", [33, 257, 4100, 128256])
def test_sample_draws_at_other_vocabulary_sizes(vocab):
    """The inverse CDF is found in two cuts of the vocabulary and a walk: sizes below one cut, off every multiple, and
    the 8B shape's; uniform numbers at both ends; the draw must be the plain implementation's or its neighbour among the
    tokens that carry weight (the cumulative sums round differently)."""
    ops = _ops()
    torch.manual_seed(vocab)
    rows = 12
    z = torch.randn(rows, vocab, device=DEV) * 4
    z[3, : vocab // 2] = -math.inf  # weightless tokens are never drawn
    z[1, vocab - vocab // 3 :] = -math.inf  # ... nor when u * total rounds up to the total and the last token is taken
    T = torch.tensor([0.5, 0.8, 1.0, 1.0, 0.7, 1.3, 0.9, 1.1, 0.6, 1.0, 2.0, 0.0], device=DEV)
    u = torch.tensor([0.0, 0.9999999, 0.5, 0.001, 0.25, 0.75, 0.1, 0.9, 0.33, 0.66, 0.999, 0.5], device=DEV)
    tok, lp, slp = ops.unpack_sample(ops.sample(z, T, u))
    zc = z.cpu()
    for r in range(rows):
        t = float(T[r])
        if t == 0:
            assert int(tok[r]) == int(zc[r].argmax())
            continue
        ref_lp = pl.processed_logprobs(zc[r], t, 0, 1.0)
        ref = pl.draw_token(ref_lp, float(u[r]))
        got = int(tok[r])
        assert ref_lp[got] > -math.inf
        cdf = torch.cumsum(torch.exp(ref_lp.double()), 0)
        assert abs(float(cdf[got]) - float(cdf[ref])) < 1e-4, (r, got, ref)  # no more than rounding apart in the CDF
        assert abs(float(slp[r]) - float(ref_lp[got])) < 2e-4
        assert abs(float(lp[r]) - float(torch.log_softmax(zc[r], -1)[got])) < 2e-4


@pytest.mark.parametrize("vocab,spread", [(500, 2.0), (40000, 4.0), (40000, 0.05), (128256, 3.0)])
def test_sample_top_k_top_p(vocab, spread):
    """Small rows; rows whose kept tokens lie within a margin of the maximum (found among the tokens gathered in LDS);
    nearly flat rows, where more tokens lie within every margin than LDS holds or the cut lies below the margin."""
    ops = _ops()
    torch.manual_seed(1)
    z = torch.randn(4, vocab, device=DEV) * spread
    T = torch.tensor([0.7, 1.0, 1.0, 0.9], device=DEV)
    k = torch.tensor([5, 0, 3, 0], dtype=torch.int32, device=DEV)
    p = torch.tensor([1.0, 0.8, 0.5, 0.2], device=DEV)
    for uu in (0.01, 0.37, 0.62, 0.999):
        u = torch.full((4,), uu, device=DEV)
        tok, lp, slp = ops.unpack_sample(ops.sample(z, T, u, top_k=k, top_p=p))
        for r in range(4):
            ref_lp = pl.processed_logprobs(z[r].cpu(), float(T[r]), int(k[r]), float(p[r]))
            ref = pl.draw_token(ref_lp, uu)
            got = int(tok[r])
            if spread >= 1:
                assert ref_lp[got] > -math.inf, "a token outside the kept set was drawn"
                assert got == ref, (r, uu, got, ref)
                assert abs(float(slp[r]) - float(ref_lp[ref])) < 1e-4
            else:  # thousands of nearly equal tokens: the border of the kept set and the sums are a matter of rounding
                cdf = torch.cumsum(torch.exp(ref_lp.double()), 0)
                assert abs(float(cdf[got]) - float(cdf[ref])) < 2e-3, (r, uu, got, ref)
                assert abs(float(slp[r]) - float(ref_lp[ref])) < 1e-2


# ------------------------------------------------------------------------------------------------ the largest sizes


def _big(n, k, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(n, k, dtype=torch.float32, device=DEV, generator=g) * 0.05).to(torch.bfloat16)


@pytest.mark.parametrize("n,k", [(8192, 28672), (28672, 8192)])
def test_products_at_the_largest_feed_forward_sizes(n, k):
    """The hand-written products at an inner size and at an output width of 28,672 (the Llama-3.1-70B feed-forward): the
    streaming kernel at 1, 8 and 16 rows, the 17-to-128-row kernel at 64 and 128 rows with K in its planned ranges, the
    many-row kernel at 300 rows, the gated forms, and the product that ends in the residual stream and feeds the next
    norm; each against the 32-bit product of the same bfloat16 values."""
    ops = _ops()
    w, w2 = _big(n, k, 1), _big(n, k, 2)
    wt, wt2 = ops.TiledWeight(w), ops.TiledWeight(w2)
    wf, w2f = w.cpu().float(), w2.cpu().float()
    x_all = (torch.randn(300, k, dtype=torch.float32, device=DEV, generator=torch.Generator(device=DEV).manual_seed(3))).to(torch.bfloat16)
    ref_all = x_all.cpu().float() @ wf.T
    for m in (1, 8, 16):
        x, ref = x_all[:m], ref_all[:m]
        assert ulps_of_row_max(ops.linear_tiled(x, wt).cpu(), ref).max() <= 1.0, m
        u = x.cpu().float() @ w2f.T
        assert ulps_of_row_max(ops.linear_tiled(x, wt, w2=wt2).cpu(), ref * torch.sigmoid(ref) * u).max() <= 1.0, m
    for m in (64, 128):
        x, ref = x_all[:m], ref_all[:m]
        ksplit, nt = ops.wide_plan(n, k, m)
        out = ops.linear_wide(x, wt, ksplit=ksplit, nt=nt)
        assert ulps_of_row_max(out.cpu(), ref).max() <= 1.0, (m, ksplit, nt)
        part = ops.linear_wide(x, wt, ksplit=max(2, ksplit), nt=1, defer=True)
        assert ulps_of_row_max(ops.reduce_partial(part).cpu(), ref).max() <= 1.0, m
    u = x_all[:64].cpu().float() @ w2f.T
    act = ops.linear_wide(x_all[:64], wt, w2=wt2, ksplit=1, nt=1)
    assert ulps_of_row_max(act.cpu(), ref_all[:64] * torch.sigmoid(ref_all[:64]) * u).max() <= 1.0
    assert ulps_of_row_max(ops.linear_rows(x_all, wt).cpu(), ref_all).max() <= 1.0
    u = x_all.cpu().float() @ w2f.T
    assert ulps_of_row_max(ops.linear_rows(x_all, wt, w2=wt2, ksplit=1, nt=2).cpu(), ref_all * torch.sigmoid(ref_all) * u).max() <= 1.0
    # resid += x W^T with the next norm's inputs as by-products, 8 rows
    m = 8
    resid = (torch.randn(m, n, device=DEV) * 2).to(torch.bfloat16)
    w_next = (1 + 0.1 * torch.randn(n, device=DEV)).to(torch.bfloat16)
    before = resid.clone()
    pre = ops.linear_resid_norm(x_all[:m], wt, resid, w_next, 1e-5)
    want = (before.cpu().float() + ref_all[:m].to(torch.bfloat16).float()).to(torch.bfloat16)
    assert ulps_of_row_max(resid.cpu(), want.float()).max() <= 1.0
    torch.testing.assert_close(pre.ssq.sum(-1).cpu(), (resid.cpu().float() ** 2).sum(-1), rtol=1e-4, atol=0)
    assert torch.equal(pre.x.cpu(), (resid.cpu().float() * w_next.cpu().float()).to(torch.bfloat16))
    # a matrix copied back into plain rows, whole and in slices of its inner size
    plain = torch.empty_like(w)
    assert torch.equal(ops.untile(wt, plain), w)
    piece = torch.empty((n, 7168 if k > 8192 else 2048), dtype=torch.bfloat16, device=DEV)
    width = piece.shape[1]
    assert torch.equal(ops.untile(wt, piece, width, 2 * width), w[:, width : 2 * width])
