"""HIP kernels of the pre-norm / matrix-state mechanisms against their plain PyTorch references (ops/layers_reference.py),
op by op, on shapes that hit the kernels' edges: head widths that are no multiple of the wave, key widths that need
one, several and sixteen waves per workgroup, grouped heads, strided column views, in-place calls, skipped rows."""
import math

import pytest
import torch

from distributed_sse_for_llm_response_amd import ops
from distributed_sse_for_llm_response_amd.ops import layers_reference as lref

pytestmark = pytest.mark.gpu

PAGE = 32


def dev():
    return torch.device("cuda")


def i32(x):
    return torch.tensor(x, dtype=torch.int32)


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    err = (a - b).abs().max().item()
    ref = b.abs().max().item() + 1e-6
    assert err <= tol * ref, f"max abs err {err} vs scale {ref}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_stream_step(dtype):
    g = torch.Generator().manual_seed(0)
    M, W, V = 7, 333, 50
    y, resid = torch.randn(M, W, generator=g), torch.randn(M, W, generator=g)
    embed = torch.randn(V, W, generator=g).to(dtype)
    ids = i32([3, 49, 0, 7, 7, 12, 100])  # the last id is out of range: row 0 of the table
    vec, w, b = torch.randn(W, generator=g), torch.randn(W, generator=g), torch.randn(W, generator=g)
    alpha = torch.tensor([0.7])
    for use in ((1, 1, 1, 1), (1, 0, 0, 1), (0, 0, 0, 1), (1, 0, 0, 0), (0, 1, 1, 1)):
        r_ref, x_ref = resid.clone(), torch.zeros(M, W, dtype=dtype)
        lref.stream_step(y if use[0] else None, 0.7, r_ref, ids if use[1] else None, embed if use[1] else None,
                         vec if use[2] else None, alpha if use[3] else None, w if use[3] else None,
                         b if use[3] else None, x_ref if use[3] else None)
        c = lambda t: t.to(dev())  # noqa: E731
        r_gpu, x_gpu = c(resid.clone()), torch.zeros(M, W, dtype=dtype, device=dev())
        ops.stream_step(c(y) if use[0] else None, 0.7, r_gpu, c(ids) if use[1] else None, c(embed) if use[1] else None,
                        c(vec) if use[2] else None, c(alpha) if use[3] else None, c(w) if use[3] else None,
                        c(b) if use[3] else None, x_gpu if use[3] else None)
        close(r_gpu, r_ref, 1e-6)
        if use[3]:
            close(x_gpu, x_ref, 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("kind", [0, 1])
def test_gated_act(kind):
    g = torch.Generator().manual_seed(1)
    M, F = 5, 77
    wide = torch.randn(M, 2 * F + 9, generator=g) * 3
    h_ref = torch.zeros(M, F)
    lref.gated_act(wide[:, 4:4 + 2 * F], h_ref, kind)
    wg = wide.to(dev())
    h = torch.zeros(M, F, device=dev())
    ops.gated_act(wg[:, 4:4 + 2 * F], h, kind)
    close(h, h_ref, 1e-5)


@pytest.mark.parametrize("nh,D,dims,kind", [(3, 40, 16, 1), (5, 64, 64, 0), (2, 96, 0, 2), (9, 33, 32, 2), (1, 512, 128, 1)])
def test_norm_rope_rows(nh, D, dims, kind):
    g = torch.Generator().manual_seed(2)
    T = 6
    wide = torch.randn(T, nh * D + 11, generator=g)
    x = wide[:, 5:5 + nh * D].unflatten(1, (nh, D))
    nw = torch.randn(nh * D, generator=g) if kind == 1 else None
    pos = i32([0, 1, 5, 63, 64, 200])
    ang = torch.arange(256, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(dims // 2, dtype=torch.float64) /
                                                                      max(1, dims // 2)))[None, :]
    rope = torch.stack([ang.cos(), ang.sin()], -1).float() if dims else None
    # 1. to a contiguous fp32 buffer
    o_ref = torch.zeros(T, nh, D)
    lref.norm_rope_rows(x, nw, pos, rope, o_ref, None, kind, 1e-5, 0.5)
    wg = wide.to(dev())
    xg = wg[:, 5:5 + nh * D].unflatten(1, (nh, D))
    c = lambda t: None if t is None else t.to(dev())  # noqa: E731
    o = torch.zeros(T, nh, D, device=dev())
    ops.norm_rope_rows(xg, c(nw), c(pos), c(rope), o, None, kind, 1e-5, 0.5)
    close(o, o_ref, 2e-6)
    # 2. into chosen rows of a paged bf16 buffer, one row skipped
    rows = i32([40, 3, -1, 63, 0, 17])
    cache_ref = torch.zeros(2, PAGE, nh, D, dtype=torch.bfloat16)
    lref.norm_rope_rows(x, nw, pos, rope, cache_ref, rows, kind, 1e-5, 1.0)
    cache = torch.zeros(2, PAGE, nh, D, dtype=torch.bfloat16, device=dev())
    ops.norm_rope_rows(xg, c(nw), c(pos), c(rope), cache, c(rows), kind, 1e-5, 1.0)
    close(cache, cache_ref, 1e-2)
    assert cache.view(-1, nh * D)[5].abs().sum().item() == 0
    # 3. in place
    ops.norm_rope_rows(xg, c(nw), c(pos), c(rope), xg, None, kind, 1e-5, 0.5)
    close(xg, o_ref, 2e-6)
    assert torch.equal(wg[:, :5].cpu(), wide[:, :5]) and torch.equal(wg[:, 5 + nh * D:].cpu(), wide[:, 5 + nh * D:])


def test_gate_math():
    g = torch.Generator().manual_seed(3)
    M, N = 9, 13
    wide = torch.randn(M, 2 * N + 3, generator=g) * 4
    p1, p2 = torch.randn(N, generator=g), torch.randn(N, generator=g)
    for kind, c0 in ((0, 0), (1, N), (2, 2)):
        ref = wide.clone()
        lref.gate_math(ref[:, c0:c0 + N], kind, p1, p2, 16.0)
        got = wide.to(dev())
        ops.gate_math(got[:, c0:c0 + N], kind, p1.to(dev()), p2.to(dev()), 16.0)
        close(got, ref, 2e-6)


def _pages(n_seq, lens, g):
    """Shuffled block tables for sequences of the given lengths."""
    need = [math.ceil(n / PAGE) for n in lens]
    perm = torch.randperm(sum(need) + 3, generator=g).tolist()
    bt = torch.zeros(n_seq, max(need) + 1, dtype=torch.int32)
    k = 0
    for s, n in enumerate(need):
        bt[s, :n] = torch.tensor(perm[k:k + n], dtype=torch.int32)
        k += n
    return bt, sum(need) + 3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 64, 64, 10 ** 9), (6, 1, 40, 24, 37), (3, 3, 128, 130, 10 ** 9),
                                            (8, 4, 16, 512, 100)])
def test_sink_attention(dtype, H, G, D, V, window):
    g = torch.Generator().manual_seed(4)
    ctx, ql = [300, 1, 70, 33], [40, 1, 70, 1]        # a late portion, a first token, a whole prompt, a decode row
    bt, pages = _pages(4, ctx, g)
    T = sum(ql)
    q = torch.randn(T, H, D, generator=g)
    kc = torch.randn(pages, PAGE, G, D, generator=g).to(dtype)
    vc = torch.randn(pages, PAGE, G, V, generator=g).to(dtype)
    sink, gate = torch.randn(H, generator=g), torch.randn(T, H + 2, generator=g)
    qs = i32([0, 40, 41, 111])
    qt = 4
    ws = [s for s, n in enumerate(ql) for _ in range(math.ceil(n / qt))]
    wt = [t for n in ql for t in range(math.ceil(n / qt))]
    for use_sink, use_gate in ((True, True), (False, False)):
        o_ref = torch.zeros(T, H, V, dtype=dtype)
        lref.sink_attention(q, kc, vc, bt, qs, i32(ql), i32(ctx), sink if use_sink else None,
                            gate[:, 1:1 + H] if use_gate else None, o_ref, window, 0.2)
        c = lambda t: t.to(dev())  # noqa: E731
        o = torch.zeros(T, H, V, dtype=dtype, device=dev())
        gg = c(gate)
        ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(ws)), c(i32(wt)),
                           c(sink) if use_sink else None, gg[:, 1:1 + H] if use_gate else None, o, window, 0.2, qt)
        close(o, o_ref, 1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("H,G,D,V,window", [(4, 2, 64, 64, 10 ** 9), (6, 1, 32, 16, 37), (5, 5, 128, 112, 10 ** 9),
                                            (8, 2, 96, 320, 100)])
def test_sink_attention_mfma_form(H, G, D, V, window):
    """Prompt portions on the MFMA form (values from the transposed pages) against the reference, which reads the same
    transposed pages: tiles that start and end inside pages, a first token, a portion deep into a long context."""
    g = torch.Generator().manual_seed(8)
    ctx, ql = [300, 1, 70, 45], [40, 1, 70, 2]
    bt, pages = _pages(4, ctx, g)
    T = sum(ql)
    q = torch.randn(T, H, D, generator=g)
    kc = torch.randn(pages, PAGE, G, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(pages, PAGE, G, V, generator=g).to(torch.bfloat16)
    off = torch.arange(PAGE)
    vt = torch.zeros(pages, G, V, PAGE, dtype=torch.bfloat16)
    vt[:, :, :, lref.vt_position(off)] = vc.permute(0, 2, 3, 1)
    sink, gate = torch.randn(H, generator=g), torch.randn(T, H, generator=g)
    qs = i32([0, 40, 41, 111])
    hs = [s for s, n in enumerate(ql) for _ in range(math.ceil(n / 16))]
    ht = [t for n in ql for t in range(math.ceil(n / 16))]
    for use in (True, False):
        o_ref = torch.zeros(T, H, V, dtype=torch.bfloat16)
        lref.sink_attention(q, kc, torch.zeros_like(vc), bt, qs, i32(ql), i32(ctx), sink if use else None,
                            gate if use else None, o_ref, window, 0.2, vt)
        c = lambda t: t.to(dev())  # noqa: E731
        o = torch.zeros(T, H, V, dtype=torch.bfloat16, device=dev())
        ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(hs)), c(i32(ht)),
                           c(sink) if use else None, c(gate) if use else None, o, window, 0.2, 16, c(vt))
        close(o, o_ref, 2e-2)
        if V <= 128:  # the same with every (tile, head)'s pages split over four waves
            o2 = torch.zeros_like(o)
            ops.sink_attention(c(q), c(kc), c(vc), c(bt), c(qs), c(i32(ql)), c(i32(ctx)), c(i32(hs)), c(i32(ht)),
                               c(sink) if use else None, c(gate) if use else None, o2, window, 0.2, 16, c(vt), True)
            close(o2, o_ref, 2e-2)


def test_transposed_value_pages_written_with_the_rows():
    g = torch.Generator().manual_seed(9)
    T, G, V = 40, 2, 48
    x = torch.randn(T, G, V, generator=g)
    rows = torch.randperm(3 * PAGE, generator=g)[:T].to(torch.int32)
    rows[5] = -1
    ref, ref_t = torch.zeros(3, PAGE, G, V, dtype=torch.bfloat16), torch.zeros(3, G, V, PAGE, dtype=torch.bfloat16)
    lref.norm_rope_rows(x, None, rows, None, ref, rows, 0, 0.0, 1.0, ref_t)
    out, out_t = ref.clone().zero_().to(dev()), ref_t.clone().zero_().to(dev())
    ops.norm_rope_rows(x.to(dev()), None, rows.to(dev()), None, out, rows.to(dev()), 0, 0.0, 1.0, out_t)
    assert torch.equal(out.cpu(), ref) and torch.equal(out_t.cpu(), ref_t)
    flat = ref.view(-1, G, V)
    for r in (0, 17, 95):   # the transposed page holds row r's numbers at vt_position(r % 32)
        assert torch.equal(ref_t[r // PAGE, :, :, int(lref.vt_position(torch.tensor(r % PAGE)))], flat[r])


@pytest.mark.parametrize("H,G,D,V", [(4, 2, 32, 32), (2, 2, 48, 100), (3, 1, 128, 64), (1, 1, 300, 70), (2, 1, 8, 5)])
@pytest.mark.parametrize("mode", ["delta", "channel", "fixed", "plain"])
def test_matrix_scan(H, G, D, V, mode):
    g = torch.Generator().manual_seed(5)
    ql, ctx, slot = [37, 1, 0, 5], [37, 9, 4, 25], [2, 0, 3, 1]   # fresh prompt, decode row, inactive, later portion
    T = sum(ql) + 1
    qs = i32([0, 37, 38, 38])
    wide = torch.randn(T, 2 * G * D + H * V + 7, generator=g)
    q = wide[:, 2:2 + G * D].unflatten(1, (G, D))
    k = wide[:, 2 + G * D:2 + 2 * G * D].unflatten(1, (G, D))
    k = k / k.norm(dim=-1, keepdim=True)
    v = wide[:, 2 + 2 * G * D:2 + 2 * G * D + H * V].unflatten(1, (H, V))
    kk = wide.clone()
    kk[:, 2 + G * D:2 + 2 * G * D] = k.flatten(1)
    wide = kk
    k = wide[:, 2 + G * D:2 + 2 * G * D].unflatten(1, (G, D))
    decay = {"delta": torch.rand(T, H, generator=g) * 0.5 + 0.5, "channel": torch.rand(T, H, D, generator=g) * 0.3 + 0.7,
             "fixed": torch.linspace(0.5, 0.99, H), "plain": None}[mode]
    beta = torch.rand(T, H, generator=g) if mode == "delta" else None
    state0 = torch.randn(4, H, D, V, generator=g)
    st_ref, o_ref = state0.clone(), torch.zeros(T, H, V)
    lref.matrix_scan(q, k, v, decay, beta, st_ref, qs, i32(ql), i32(ctx), i32(slot), o_ref, 0.3)
    c = lambda t: None if t is None else t.to(dev())  # noqa: E731
    wg = c(wide)
    qg = wg[:, 2:2 + G * D].unflatten(1, (G, D))
    kg = wg[:, 2 + G * D:2 + 2 * G * D].unflatten(1, (G, D))
    vg = wg[:, 2 + 2 * G * D:2 + 2 * G * D + H * V].unflatten(1, (H, V))
    from distributed_sse_for_llm_response_amd.ops.layers import scan_state_from_plain, scan_state_plain

    st, o = scan_state_from_plain(c(state0.clone())), torch.zeros(T, H, V, device=dev())
    ops.matrix_scan(qg, kg, vg, c(decay), c(beta), st, c(qs), c(i32(ql)), c(i32(ctx)), c(i32(slot)), o, 0.3)
    close(o, o_ref, 2e-5)
    close(scan_state_plain(st), st_ref, 2e-5)
    assert torch.equal(scan_state_plain(st)[3].cpu(), state0[3])   # the inactive sequence's slot is untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_head_norm_and_mix(dtype):
    g = torch.Generator().manual_seed(6)
    M, H, V, W = 7, 3, 50, 129
    o = torch.randn(M, H, V, generator=g)
    gate = torch.randn(M, H * V + 4, generator=g)
    w = torch.randn(V, generator=g)
    for ww in (w, None):
        ref = torch.zeros(M, H * V, dtype=dtype)
        lref.gated_head_norm(o, ww, gate[:, 4:], 1e-5, ref)
        out = torch.zeros(M, H * V, dtype=dtype, device=dev())
        ops.gated_head_norm(o.to(dev()), None if ww is None else ww.to(dev()), gate.to(dev())[:, 4:], 1e-5, out)
        close(out, ref, 1e-5 if dtype == torch.float32 else 1e-2)
    ya, yb = torch.randn(M, W, generator=g), torch.randn(M, W, generator=g) * 5
    wa, wb = torch.randn(W, generator=g), torch.randn(W, generator=g)
    ref = torch.zeros(M, W)
    lref.rms_mix(ya, wa, yb, wb, 1e-5, 0.5, ref)
    ga = ya.to(dev())
    ops.rms_mix(ga, wa.to(dev()), yb.to(dev()), wb.to(dev()), 1e-5, 0.5, ga)  # in place
    close(ga, ref, 2e-6)
    z = torch.randn(M, W, generator=g) * 40
    ref = z.clone()
    lref.logit_cap(ref, 0.25, 30.0)
    zg = z.to(dev())
    ops.logit_cap(zg, 0.25, 30.0)
    close(zg, ref, 2e-6)


def test_conv_state_strided_silu():
    g = torch.Generator().manual_seed(7)
    C, K = 70, 4
    ql, ctx, slot = [9, 1, 2], [9, 5, 30], [1, 0, 2]
    T = sum(ql)
    qs = i32([0, 9, 10])
    wide = torch.randn(T, C + 6, generator=g)
    taps = torch.randn(C, K, generator=g)
    tail0 = torch.randn(3, K - 1, C, generator=g)
    t_ref, o_ref = tail0.clone(), torch.zeros(T, C)
    lref.conv_state(wide[:, 3:3 + C], taps, None, t_ref, qs, i32(ql), i32(ctx), i32(slot), o_ref, None, None, 1)
    c = lambda t: t.to(dev())  # noqa: E731
    tl, o = c(tail0.clone()), torch.zeros(T, C, device=dev())
    ops.conv_state(c(wide)[:, 3:3 + C], c(taps), None, tl, c(qs), c(i32(ql)), c(i32(ctx)), c(i32(slot)), o, None, None, 1)
    close(o, o_ref, 2e-6)
    close(tl, t_ref, 1e-6)


@pytest.mark.parametrize("H,G,D,V", [(3, 1, 32, 40), (2, 2, 128, 64), (1, 1, 72, 16)])
@pytest.mark.parametrize("mode", ["channel", "fixed", "plain"])
def test_matrix_scan_two_level_walk(H, G, D, V, mode):
    """Long portions walked in chunks (parallel from zeros, carry, parallel again) against the plain reference walk:
    a fresh prompt that ends inside a chunk, a later portion continued from its slot, one exactly one chunk long, one
    shorter than a chunk."""
    from distributed_sse_for_llm_response_amd.ops.layers import scan_chunks, scan_state_from_plain, scan_state_plain

    g = torch.Generator().manual_seed(11)
    ql, ctx, slot = [200, 131, 64, 5], [200, 300, 64, 90], [2, 0, 3, 1]
    qs = [0, 200, 331, 395]
    T = sum(ql)
    q = torch.randn(T, G, D, generator=g) * 0.3
    k = torch.randn(T, G, D, generator=g) * 0.3
    v = torch.randn(T, H, V, generator=g)
    decay = {"channel": torch.rand(T, H, D, generator=g) * 0.1 + 0.9, "fixed": torch.linspace(0.9, 0.999, H),
             "plain": None}[mode]
    state0 = torch.randn(4, H, D, V, generator=g)
    st_ref, o_ref = state0.clone(), torch.zeros(T, H, V)
    lref.matrix_scan(q, k, v, decay, None, st_ref, i32(qs), i32(ql), i32(ctx), i32(slot), o_ref, 0.5)
    s_first, s_count, rows = scan_chunks(qs, ql, slot)
    assert s_count == [4, 3, 1, 1]
    c = lambda t: None if t is None else t.to(dev())  # noqa: E731
    st, o = scan_state_from_plain(c(state0.clone())), torch.zeros(T, H, V, device=dev())
    n = len(rows[0])
    scr = torch.full((n * H * D * V,), float("nan"), device=dev())
    ascr = torch.full((n * H * D,), float("nan"), device=dev()) if mode == "channel" else None
    ops.matrix_scan_chunked(c(q), c(k), c(v), c(decay), st, c(i32(qs)), c(i32(ql)), c(i32(ctx)), c(i32(slot)),
                            c(i32(s_first)), c(i32(s_count)), c(i32(rows)), scr, ascr, o, 0.5)
    close(o, o_ref, 3e-5)
    close(scan_state_plain(st), st_ref, 3e-5)


@pytest.mark.parametrize("H,G,D,V", [(4, 2, 32, 32), (2, 1, 128, 64), (1, 1, 300, 70)])
@pytest.mark.parametrize("mode", ["delta", "channel", "fixed"])
def test_matrix_scan_decode_rows(H, G, D, V, mode):
    """One row per sequence (a decode step: the kernel that keeps the state traffic coalesced), one slot inactive,
    one sequence at position 0."""
    from distributed_sse_for_llm_response_amd.ops.layers import scan_state_from_plain, scan_state_plain

    g = torch.Generator().manual_seed(12)
    ql, ctx, slot = [1, 1, 0, 1, 1], [9, 1, 4, 300, 2], [4, 0, 3, 1, 2]
    qs = i32([0, 1, 2, 3, 4])
    T = 5
    q, k = torch.randn(T, G, D, generator=g) * 0.3, torch.randn(T, G, D, generator=g) * 0.3
    v = torch.randn(T, H, V, generator=g)
    decay = {"delta": torch.rand(T, H, generator=g) * 0.5 + 0.5, "channel": torch.rand(T, H, D, generator=g) * 0.3 + 0.7,
             "fixed": torch.linspace(0.5, 0.99, H)}[mode]
    beta = torch.rand(T, H, generator=g) if mode == "delta" else None
    state0 = torch.randn(5, H, D, V, generator=g)
    st_ref, o_ref = state0.clone(), torch.zeros(T, H, V)
    lref.matrix_scan(q, k, v, decay, beta, st_ref, qs, i32(ql), i32(ctx), i32(slot), o_ref, 0.7)
    c = lambda t: None if t is None else t.to(dev())  # noqa: E731
    st, o = scan_state_from_plain(c(state0.clone())), torch.zeros(T, H, V, device=dev())
    ops.matrix_scan(c(q), c(k), c(v), c(decay), c(beta), st, c(qs), c(i32(ql)), c(i32(ctx)), c(i32(slot)), o, 0.7)
    close(o, o_ref, 2e-5)
    close(scan_state_plain(st), st_ref, 2e-5)
