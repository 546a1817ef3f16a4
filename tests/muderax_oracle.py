"""Plain, slow oracle of the Muderax design: one function per mechanism, whole sequences only, no cache.

Written from the design's equations, in float64 by default, and shares no code with the package: the tests compare
the engine (its kernels, caches, state slots and scheduler) with this.  Inputs: the configuration as the dictionary
a checkpoint's ``config.json`` holds, and the weights as {tensor name: tensor}.

Notation: ``x`` is the residual stream [T, W]; a layer is ``x += n1(mixer(x)); x += n2(ffn(x))`` where ``n`` is the
one-number RMS norm ``v / sqrt(mean(v^2) + eps) * g``.
"""
from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def scalar_norm(v, g, eps):
    return unit_rms(v, eps) * g


def yarn_frequencies(rot: dict):
    """(frequencies [dims / 2], amplitude) of the rotation; plain powers of the base without a 'scaling' entry."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(v, positions, rot: dict):
    """Interleaved rotation of the first rot['dims'] coordinates of v [T, ..., D] (pairs 2i, 2i + 1)."""
    dims = int(rot["dims"])
    f, amp = yarn_frequencies(rot)
    ang = positions.to(torch.float64)[:, None] * f[None, :]
    cos, sin = ang.cos() * amp, ang.sin() * amp
    while cos.dim() < v.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def latent_attention(h, w: dict, p: str, m: dict, eps: float):
    """h [T, W] -> [T, W].  Keys and values are up-projected from the normed latent for every head (the plain form)."""
    T = h.shape[0]
    H, dn, dr, dv, rk = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T)
    q = (h @ w[p + "q"].T).view(T, H, dn + dr)
    q_n, q_r = q[..., :dn], rotate_pairs(q[..., dn:], pos, m["rot"])
    d = h @ w[p + "dkv"].T
    c = unit_rms(d[:, :rk], eps) * w[p + "dkv.norm"]
    k_r = rotate_pairs(d[:, rk:], pos, m["rot"])
    k_n = (c @ w[p + "uk"].T).view(T, H, dn)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q_n, k_n) + torch.einsum("ihd,jd->hij", q_r, k_r)) * float(m["scale"])
    i, j = pos[:, None], pos[None, :]
    seen = i - j >= 0
    if m.get("mask"):
        seen = seen & (i - j < int(m["mask"]["size"]))
    s = s.masked_fill(~seen[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(s, -1), v).reshape(T, H * dv)
    return o @ w[p + "o"].T


def causal_conv(u, taps, bias):
    """u [T, C], taps [C, K] ; taps[:, K - 1] weighs the newest input and the history before position 0 is empty."""
    T, K = u.shape[0], taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, u.shape[1], dtype=u.dtype), u])
    out = bias.expand(T, -1).clone()
    for k in range(K):
        out = out + pad[k:k + T] * taps[:, k]
    return out


def rglru(h, w: dict, p: str, m: dict):
    """Recurrent block: gelu branch times a real-gated linear recurrence over a short causal convolution."""
    T = h.shape[0]
    nb = int(m["blocks"])
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    ub = u.view(T, nb, -1)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(T, -1)
    g = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(T, -1)
    log_a = -8.0 * r * torch.nn.functional.softplus(w[p + "lam"])
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * g * u
    S = torch.zeros(u.shape[1], dtype=u.dtype)
    out = []
    for t in range(T):
        S = a[t] * S + drive[t]
        out.append(S)
    return (torch.stack(out) * y) @ w[p + "o"].T


def gated_ffn(h, w: dict, p: str):
    return (torch.nn.functional.silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe(h, w: dict, p: str, f: dict):
    """Top-k of the router's logits, their weights renormalised among themselves by a softmax; the shared expert is added for every row."""
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    z = h @ w[p + "router"].T + w[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    gate = torch.softmax(val, -1)
    out = torch.zeros_like(h)
    for e in range(E):
        sel = idx == e
        rows = sel.any(-1)
        if rows.any():
            out[rows] += gated_ffn(h[rows], w, f"{p}e{e}.") * (gate * sel)[rows].sum(-1, keepdim=True)
    if f.get("shared"):
        out = out + gated_ffn(h, w, p + "shared.")
    return out


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float64, layers_out: list | None = None):
    """Logits [T, vocab] of one whole sequence; layers_out (a list) receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for li, L in enumerate(cfg["layers"]):
        src = L.get("weights_of", li)
        p = f"l{src}."
        if L["type"] == "latent_attention":
            y = latent_attention(x, w, p + "mix.", L["mixer"], eps)
        elif L["type"] == "rglru":
            y = rglru(x, w, p + "mix.", L["mixer"])
        else:
            raise ValueError(L["type"])
        x = x + scalar_norm(y, w[p + "norm1"], eps)
        if L.get("mlp"):
            x = x + scalar_norm(moe(x, w, p + "mlp.", L["mlp"]), w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T
