"""Plain-PyTorch references of the layer-mechanism ops (``ops/layers.py``): exact semantics of the HIP kernels in
``csrc/kernels/{gemm_rowmajor,norms,latent_attention,recurrent,moe}.hip``, including the cache and state layouts.

As with ``ops/reference.py`` they are the numerics oracle of the kernel tests and the CPU execution path of the engine
(scheduler, cache and state-slot plumbing run here without a GPU).  Everything is computed in fp32 on whatever element
type the tensors carry.
"""
from __future__ import annotations

import math

import torch

PAGE = 32


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def gemm_rm(x, w, out, bias=None, act=0):
    y = torch.matmul(x.float(), w.float().transpose(-1, -2))
    if bias is not None:
        y = y + bias.float().unsqueeze(-2)
    if act == 1:
        y = gelu_tanh(y)
    out.copy_(y.to(out.dtype))


def scalar_norm(y, g, resid, xb, eps, nsum=1):
    src = resid if y is None else y.view(resid.shape[0], nsum, -1).sum(1)
    n = src * (g.float().reshape(()) / torch.sqrt(src.pow(2).mean(-1, keepdim=True) + eps))
    if y is None:
        xb.copy_(n.to(xb.dtype))
    else:
        resid.add_(n)
        xb.copy_(resid.to(xb.dtype))


def embed_rows(ids, embed, resid, xb):
    M = resid.shape[0]
    idx = ids[:M].long()
    idx = torch.where((idx >= 0) & (idx < embed.shape[0]), idx, torch.zeros_like(idx))
    rows = embed[idx]
    resid.copy_(rows.float())
    xb.copy_(rows)


def _rotate(v, cs):
    """v [..., dr] interleaved pairs, cs [..., dr / 2, 2] (cos, sin)."""
    a, b = v[..., 0::2], v[..., 1::2]
    out = torch.empty_like(v)
    out[..., 0::2] = a * cs[..., 0] - b * cs[..., 1]
    out[..., 1::2] = b * cs[..., 0] + a * cs[..., 1]
    return out


def vt_position(off):
    """Place of token `off` (0..31) inside a transposed latent page (the MFMA attention's key order)."""
    return ((off & 15) >> 2) * 8 + ((off >> 4) & 1) * 4 + (off & 3)


def latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt=None):
    T, rk = ckr.shape[0], norm_w.numel()
    flat = cache.view(-1, cache.shape[-1])
    c = ckr[:, :rk]
    c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    pos = positions[:T].long().clamp(0, rope.shape[0] - 1)
    kr = _rotate(ckr[:, rk:], rope[pos])
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    sl = slots[:T].long()
    ok = (sl >= 0) & (sl < flat.shape[0])
    flat[sl[ok]] = row[ok]
    if vt is not None:
        good = sl[ok]
        vt[good // PAGE, :, vt_position(good % PAGE)] = row[ok][:, :rk]


def latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out, window,
                     scale, qt, vt=None):
    """With vt the values come from the transposed pages (the same numbers in another place), so a wrong place shows."""
    rk = q_abs.shape[2]
    dr = cache.shape[2] - rk
    dn = q.shape[2] - dr
    flat = cache.view(-1, cache.shape[-1]).float()
    done = set()
    for s, t in zip(work_seq.tolist(), work_tile.tolist()):
        ql = int(q_len[s])
        for i in range(qt):
            off = t * qt + i
            if off >= ql or (s, off) in done:
                continue
            done.add((s, off))
            row = int(q_start[s]) + off
            pos = int(ctx_len[s]) - ql + off
            lo = max(0, pos - window + 1)
            j = torch.arange(lo, pos + 1)
            rows = block_tables[s].long()[j // PAGE] * PAGE + j % PAGE
            kv = flat[rows]  # [keys, rk + dr]
            qr = _rotate(q[row, :, dn:].float(), rope[min(max(pos, 0), rope.shape[0] - 1)])
            sc = (q_abs[row].float() @ kv[:, :rk].t() + qr @ kv[:, rk:].t()) * scale
            p = torch.softmax(sc, dim=-1)
            val = kv[:, :rk] if vt is None else vt[rows // PAGE, :, vt_position(rows % PAGE)].float()
            out[row] = (p @ val).to(out.dtype)


def conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias=None):
    K = taps.shape[1]
    tp = taps.float()
    ib = 0.0 if in_bias is None else in_bias.float()
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, slot = int(q_start[s]), int(state_slot[s])
        fresh = int(ctx_len[s]) - ql == 0
        prev = torch.zeros(K - 1, inp.shape[1]) if fresh else tail[slot].clone()
        seq = torch.cat([prev, inp[r0:r0 + ql] + ib])
        y = torch.zeros(ql, inp.shape[1]) if bias is None else bias.float().expand(ql, -1).clone()
        for k in range(K):
            y = y + seq[k:k + ql] * tp[:, k]
        out[r0:r0 + ql] = y
        out_b[r0:r0 + ql] = y.to(out_b.dtype)
        if K > 1:
            tail[slot] = seq[ql:]


def lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias=None, coeff=True):
    """coeff: first turn every row's gate pre-activations [recurrence | input] into the coefficients (a | b) of
    S = a S + b, in place; then walk each sequence's rows.  y is the gelu branch before its bias and gelu."""
    C = u.shape[1]
    bw = gates.shape[2] // 2
    if coeff:
        sp = torch.nn.functional.softplus(lam.float()).view(1, -1, bw)
        log_a = -c * torch.sigmoid(gates[:, :, :bw]) * sp
        b = torch.sqrt(-torch.expm1(2.0 * log_a)) * torch.sigmoid(gates[:, :, bw:]) * u.view(u.shape[0], -1, bw)
        gates[:, :, :bw] = torch.exp(log_a)
        gates[:, :, bw:] = b
    yb = 0.0 if y_bias is None else y_bias.float()
    for s in range(q_len.numel()):
        ql = int(q_len[s])
        if ql <= 0:
            continue
        r0, slot = int(q_start[s]), int(state_slot[s])
        S = torch.zeros(C) if int(ctx_len[s]) - ql == 0 else state[slot].clone()
        for t in range(ql):
            g = gates[r0 + t]
            S = g[:, :bw].reshape(C) * S + g[:, bw:].reshape(C)
            out[r0 + t] = (S * gelu_tanh(y[r0 + t].float() + yb)).to(out.dtype)
        state[slot] = S


def moe_topk(logits, topk_idx, topk_w):
    z = torch.nan_to_num(logits.float(), nan=0.0)
    val, idx = torch.topk(z, topk_idx.shape[1], dim=-1)
    topk_idx.copy_(idx.to(torch.int32))
    topk_w.copy_(torch.softmax(val, dim=-1))


def moe_router(x, w, b, topk_idx, topk_w):
    z = x.float() @ w.float().t()
    if b is not None:
        z = z + b.float()
    z = torch.nan_to_num(z, nan=0.0)
    val, idx = torch.topk(z, topk_idx.shape[1], dim=-1)
    topk_idx.copy_(idx.to(torch.int32))
    topk_w.copy_(torch.softmax(val, dim=-1))


def moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out):
    xf = x.float()

    def ffn(h, g, u, d):
        return (torch.nn.functional.silu(h @ g.float().t()) * (h @ u.float().t())) @ d.float().t()

    acc = torch.zeros_like(out)
    for e in range(gate.shape[0]):
        sel = topk_idx == e
        rows = sel.any(-1)
        if rows.any():
            acc[rows] += ffn(xf[rows], gate[e], up[e], down[e]) * (topk_w * sel)[rows].sum(-1, keepdim=True)
    if sgate is not None:
        acc += ffn(xf, sgate, sup, sdown)
    out.copy_(acc)


def moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, o):
    """o [M * S, W]: slot k < top of row r = weight * expert output, slot `top` = the shared expert."""
    xf = x.float()
    M, top = topk_idx.shape
    S = top + (1 if sgate is not None else 0)
    ov = o.view(M, S, -1)

    def ffn(h, g, u, d):
        return (torch.nn.functional.silu(h @ g.float().t()) * (h @ u.float().t())) @ d.float().t()

    for e in range(gate.shape[0]):
        rows, ks = torch.nonzero(topk_idx == e, as_tuple=True)
        if rows.numel():
            ov[rows, ks] = ffn(xf[rows], gate[e], up[e], down[e]) * topk_w[rows, ks].unsqueeze(-1)
    if sgate is not None:
        ov[:, top] = ffn(xf, sgate, sup, sdown)
