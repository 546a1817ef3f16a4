"""The MFMA form of latent attention against the row kernel and the PyTorch reference of the same op, on the same
bf16 inputs: random block tables, several sequences with unequal portions, windows that end inside, at and across
pages, decode columns (a row's heads side by side, also more than 16 heads) and prompt tiles."""
import math

import pytest
import torch

from distributed_sse_for_llm_response_amd import ops
from distributed_sse_for_llm_response_amd.ops import layers_reference as lref

pytestmark = pytest.mark.gpu


def _case(gpu, H, dn, dr, rk, window, seqs, qt_rows, seed):
    """seqs: [(context before the step, rows in the step)].  Returns the three outputs [T, H, rk]."""
    g = torch.Generator().manual_seed(seed)
    D = rk + dr
    total = sum(c + n for c, n in seqs)
    pages = sum(math.ceil((c + n) / 32) for c, n in seqs) + 3
    perm = torch.randperm(pages, generator=g).tolist()
    mb = max(math.ceil((c + n) / 32) for c, n in seqs) + 1
    bt = torch.zeros(len(seqs), mb, dtype=torch.int32)
    cache = torch.zeros(pages, 32, D, dtype=torch.bfloat16)
    vt = torch.zeros(pages, rk, 32, dtype=torch.bfloat16)
    rope = torch.zeros(max(c + n for c, n in seqs) + 1, dr // 2, 2)
    ang = torch.arange(rope.shape[0])[:, None] * (100.0 ** (-torch.arange(dr // 2) / (dr // 2)))[None, :]
    rope[..., 0], rope[..., 1] = ang.cos() * 1.1, ang.sin() * 1.1
    qs, ql, ctx, ws, wt, fs, ft = [], [], [], [], [], [], []
    T = sum(n for _, n in seqs)
    ckr = torch.randn(total, D, generator=g) * 1.5
    norm_w = (1.0 + 0.1 * torch.randn(rk, generator=g)).to(torch.bfloat16)
    pos, slots, at, row = [], [], 0, 0
    for i, (c, n) in enumerate(seqs):
        npg = math.ceil((c + n) / 32)
        mine, perm = perm[:npg], perm[npg:]
        bt[i, :npg] = torch.tensor(mine, dtype=torch.int32)
        for p in range(c + n):
            pos.append(p)
            slots.append(mine[p // 32] * 32 + p % 32)
        qs.append(row), ql.append(n), ctx.append(c + n)
        nt = math.ceil(n / qt_rows)
        ws += [i] * nt
        wt += list(range(nt))
        row += n
        at += c + n
    q = (torch.randn(T, H, dn + dr, generator=g) * 2.0).to(torch.bfloat16)
    q_abs = torch.randn(T, H, rk, generator=g) * 2.0
    dev = dict(device=gpu)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, **dev)  # noqa: E731
    cache_g, vt_g = cache.to(gpu), vt.to(gpu)
    ops.latent_kv_write(ckr.to(gpu), norm_w.to(gpu), i32(pos), i32(slots), rope.to(gpu), cache_g, 1e-5, vt_g)
    lref.latent_kv_write(ckr, norm_w, torch.tensor(pos, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32), rope,
                         cache, 1e-5, vt)
    assert torch.equal(cache_g.cpu(), cache) or torch.allclose(cache_g.cpu().float(), cache.float(), atol=2e-2, rtol=2e-2)
    assert torch.allclose(vt_g.cpu().float(), vt.float(), atol=2e-2, rtol=2e-2)
    scale = 0.5 / math.sqrt(dn + dr)
    args = (bt.to(gpu), i32(qs), i32(ql), i32(ctx))
    out_rows = torch.zeros(T, H, rk, dtype=torch.bfloat16, **dev)
    ops.latent_attention(q.to(gpu), q_abs.to(gpu), cache_g, *args, i32(ws), i32(wt), rope.to(gpu), out_rows, window, scale,
                         qt_rows)
    out_flash = torch.zeros_like(out_rows)
    hp = 16 // qt_rows if qt_rows in (1, 2, 4, 8, 16) else 1
    if qt_rows * hp == 16:
        ops.latent_attention(q.to(gpu), q_abs.to(gpu), cache_g, *args, i32(ws), i32(wt), rope.to(gpu), out_flash, window,
                             scale, qt_rows, vt_g, hp)
    if qt_rows == 1:  # decode: also with the keys split over partitions (more partitions than some items have pages)
        for nparts in (2, 5, 16):
            part = torch.full((ops.latent_flash_part_floats(len(ws), H, 16, nparts, rk),), float("nan"), **dev)
            out_split = torch.zeros_like(out_rows)
            ops.latent_attention(q.to(gpu), q_abs.to(gpu), cache_g, *args, i32(ws), i32(wt), rope.to(gpu), out_split,
                                 window, scale, 1, vt_g, 16, part, nparts)
            assert torch.allclose(out_split.float(), out_flash.float(), atol=2e-2, rtol=2e-2), nparts
    out_ref = torch.zeros(T, H, rk, dtype=torch.float32)
    lref.latent_attention(q, q_abs, cache_g.cpu(), bt, torch.tensor(qs), torch.tensor(ql), torch.tensor(ctx),
                          torch.tensor(ws), torch.tensor(wt), rope, out_ref, window, scale, qt_rows, vt_g.cpu())
    return out_rows.float().cpu(), out_flash.float().cpu(), out_ref


@pytest.mark.parametrize("H,dn,dr,rk", [(3, 16, 32, 64), (8, 32, 32, 128), (20, 8, 64, 256), (16, 24, 32, 512)])
@pytest.mark.parametrize("window", [1, 5, 32, 33, 70, 10 ** 6])
@pytest.mark.parametrize("rows_per_tile", [16, 4, 2])
def test_prompt_tiles(gpu, H, dn, dr, rk, window, rows_per_tile):
    seqs = [(0, 50), (37, 3), (64, 31), (5, 1), (90, 40)]
    rows, flash, ref = _case(gpu, H, dn, dr, rk, window, seqs, rows_per_tile, seed=H + window)
    assert torch.allclose(rows, ref, atol=3e-2, rtol=3e-2)
    assert torch.allclose(flash, ref, atol=5e-2, rtol=5e-2), float((flash - ref).abs().max())


@pytest.mark.parametrize("H,dn,dr,rk", [(3, 16, 32, 64), (8, 32, 32, 128), (20, 8, 64, 256), (33, 24, 32, 512)])
@pytest.mark.parametrize("window", [1, 2, 31, 32, 33, 64, 65, 10 ** 6])
def test_decode_columns(gpu, H, dn, dr, rk, window):
    seqs = [(0, 1), (31, 1), (32, 1), (33, 1), (63, 1), (64, 1), (130, 1), (7, 0), (95, 1)]
    rows, flash, ref = _case(gpu, H, dn, dr, rk, window, seqs, 1, seed=7 * H + window)
    assert torch.allclose(rows, ref, atol=3e-2, rtol=3e-2)
    assert torch.allclose(flash, ref, atol=5e-2, rtol=5e-2), float((flash - ref).abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,W,F,Fs,E,top", [(1, 64, 48, 0, 4, 2), (5, 96, 40, 56, 6, 3), (37, 100, 33, 17, 5, 1),
                                             (300, 128, 96, 64, 12, 4), (64, 72, 24, 24, 3, 3)])
def test_grouped_experts_against_row_kernel(gpu, dtype, M, W, F, Fs, E, top):
    """The grouped MFMA form (rows sorted by expert) against the token-major kernel and the PyTorch reference."""
    g = torch.Generator().manual_seed(M + W)
    mk = lambda *s: (torch.randn(*s, generator=g) / math.sqrt(s[-1])).to(dtype).to(gpu)  # noqa: E731
    x = (torch.randn(M, W, generator=g)).to(dtype).to(gpu)
    router, rb = mk(E, W), (0.1 * torch.randn(E, generator=g)).to(dtype).to(gpu)
    gate, up, down = mk(E, F, W), mk(E, F, W), mk(E, W, F)
    sg, su, sd = (mk(Fs, W), mk(Fs, W), mk(W, Fs)) if Fs else (None, None, None)
    tki = torch.zeros(M, top, dtype=torch.int32, device=gpu)
    tkw = torch.zeros(M, top, device=gpu)
    ops.moe_router(x, router, rb, tki, tkw)
    ri, rw = torch.zeros(M, top, dtype=torch.int32), torch.zeros(M, top)
    lref.moe_router(x.cpu(), router.cpu(), rb.cpu(), ri, rw)
    z = torch.zeros(M, E, device=gpu)
    ops.gemm_rm(x, router, z, bias=rb)
    ti2, tw2 = torch.zeros_like(tki), torch.zeros_like(tkw)
    ops.moe_topk(z, ti2, tw2)
    if dtype == torch.float32:
        assert torch.equal(tki.cpu().sort(-1).values, ri.sort(-1).values)
        assert torch.equal(ti2.cpu().sort(-1).values, ri.sort(-1).values)
        assert torch.allclose(tw2.cpu().sort(-1).values, rw.sort(-1).values, atol=1e-5)
    rows = torch.zeros(M, W, device=gpu)
    ops.moe_ffn(x, tki, tkw, gate, up, down, sg, su, sd, rows)
    S = top + (1 if Fs else 0)
    tiles = -(-M * S // 64) + E + 2
    o = torch.zeros(M * S, W, device=gpu)
    ops.moe_grouped(x, tki, tkw, gate, up, down, sg, su, sd, torch.zeros(tiles * 64, dtype=torch.int32, device=gpu),
                    torch.zeros(tiles, dtype=torch.int32, device=gpu), torch.zeros(1, dtype=torch.int32, device=gpu),
                    torch.zeros(M * S, -(-max(F, Fs) // 8) * 8, dtype=dtype, device=gpu), o)
    ref = torch.zeros(M * S, W)
    lref.moe_grouped(x.cpu(), tki.cpu(), tkw.cpu(), gate.cpu(), up.cpu(), down.cpu(), *(t.cpu() if t is not None else None
                                                                                         for t in (sg, su, sd)), ref)
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert torch.allclose(o.cpu(), ref, atol=tol, rtol=tol), float((o.cpu() - ref).abs().max())
    assert torch.allclose(o.view(M, S, W).sum(1).cpu(), rows.cpu(), atol=tol, rtol=tol)


@pytest.mark.parametrize("N,K", [(1024, 1024), (3072, 2048), (2048, 2560)])
def test_tiled_dispatch_matches_row_major(gpu, N, K):
    """Projections that fit the tiled-layout GEMMs (weights.fits_tiled) against the general row-major GEMM, for the row
    counts of decode buckets, mixed steps and prompt passes, with bf16 and fp32 output."""
    from distributed_sse_for_llm_response_amd.engine.weights import fits_tiled
    from distributed_sse_for_llm_response_amd.ops.reference import tile_weight

    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(gpu)
    assert fits_tiled(w)
    wt = tile_weight(w)
    for M in (1, 3, 16, 17, 64, 65, 130, 257, 600, 1113):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(gpu)
        for dt in (torch.float32, torch.bfloat16):
            a, b = torch.zeros(M, N, dtype=dt, device=gpu), torch.zeros(M, N, dtype=dt, device=gpu)
            ops.gemm_rm(x, w, a)
            ops.gemm_out(x, wt, b)
            tol = 2e-3 if dt == torch.float32 else 2e-2
            assert torch.allclose(a.float(), b.float(), atol=tol, rtol=tol), (M, dt, float((a.float() - b.float()).abs().max()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (5, 33, 100), (16, 576, 2048), (17, 96, 96), (70, 130, 257), (300, 512, 384),
                                    (1113, 160, 256)])
def test_general_gemm(gpu, dtype, M, N, K):
    """gemm_rm against the PyTorch reference: every launch shape (skinny split-K, 64 x 64, 128 x 128 tiles), edges in M,
    N and K, vector and scalar fragment loads, bias, gelu, fp32 and element-type output."""
    g = torch.Generator().manual_seed(M * N + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(gpu)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype).to(gpu)
    b = torch.randn(N, generator=g).to(dtype).to(gpu)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    for bias, act, odt in ((None, 0, torch.float32), (b, 0, dtype), (b, 1, torch.float32)):
        out, ref = torch.zeros(M, N, dtype=odt, device=gpu), torch.zeros(M, N, dtype=odt)
        ops.gemm_rm(x, w, out, bias, act)
        lref.gemm_rm(x.cpu(), w.cpu(), ref, None if bias is None else bias.cpu(), act)
        assert torch.allclose(out.cpu().float(), ref.float(), atol=tol, rtol=tol), (bias is not None, act, odt)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_general_gemm_batched_views(gpu, dtype):
    """Per-head slices of wider buffers as strided views (the query fold and the value up-projection's shapes)."""
    g = torch.Generator().manual_seed(3)
    M, H, dn, dr, rk = 37, 5, 24, 8, 40
    q = torch.randn(M, H, dn + dr, generator=g).to(dtype).to(gpu)
    w = (torch.randn(H, rk, dn, generator=g) / math.sqrt(dn)).to(dtype).to(gpu)
    out = torch.zeros(M, H, rk, device=gpu)
    ops.gemm_rm(q[:, :, :dn].permute(1, 0, 2), w, out.permute(1, 0, 2))
    ref = torch.einsum("mhd,hrd->mhr", q[:, :, :dn].float().cpu(), w.float().cpu())
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert torch.allclose(out.cpu(), ref, atol=tol, rtol=tol)
