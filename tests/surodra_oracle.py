"""Plain, slow oracle of the Surodra design: one function per mechanism, whole sequences only, no cache, no batching.

Written from the design's equations in float64 and shares no code with the package: the tests compare the engine (its
kernels, caches, state slots and scheduler) with this.  Inputs: the configuration as the dictionary a checkpoint's
``config.json`` holds, and the weights as {tensor name: tensor}.

Notation: ``x`` is the residual stream [T, W]; a layer is ``x += m * mixer(n1(x)); x += m * ff(n2(x))`` with the
element-wise norm ``n(v) = tanh(alpha * v) * w + b``.  Every recurrent mixer keeps a matrix state ``S`` [dim, vdim] per
head that is walked token by token here.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def tanh_norm(v, w: dict, name: str):
    return torch.tanh(w[name + ".alpha"] * v) * w[name] + w[name + ".b"]


def rotate_half(v, positions, rot: dict):
    """First rot['dims'] coordinates of v [T, heads, D]: coordinate i pairs with i + dims / 2."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = base ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    sc = rot.get("scaling")
    if sc:
        f = f / float(sc["factor"])
    ang = positions.to(F64)[:, None] * f[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = v[..., :half], v[..., half:dims]
    out = v.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


def short_conv(x, taps):
    """x [T, C], taps [C, K] (the last column weighs the current token), zeros before the start."""
    T, K = x.shape[0], taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for k in range(K):
        out = out + pad[k:k + T] * taps[:, k]
    return out


def delta_mixer(h, w: dict, p: str, m: dict, eps: float):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    g = torch.exp(-torch.exp(w[p + "A_log"]) * torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        kv = hd // (H // G)
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def sink_attention(h, w: dict, p: str, m: dict, eps: float):
    T = h.shape[0]
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = unit_rms(h @ w[p + "q"].T, eps) * w[p + "q.norm"]
    k = unit_rms(h @ w[p + "k"].T, eps) * w[p + "k.norm"]
    q = rotate_half(q.view(T, H, D), pos, m["rot"])
    k = rotate_half(k.view(T, G, D), pos, m["rot"])
    v = (h @ w[p + "v"].T).view(T, G, V)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    seen = pos[:, None] >= pos[None, :]
    for hd in range(H):
        kv = hd // (H // G)
        s = (q[:, hd] @ k[:, kv].T) * float(m["scale"])
        s = s.masked_fill(~seen, float("-inf"))
        sink = w[p + "sink"][hd]
        mx = torch.maximum(s.max(-1, keepdim=True).values, sink)
        e = torch.exp(s - mx)
        out[:, hd] = (e / (e.sum(-1, keepdim=True) + torch.exp(sink - mx))) @ v[:, kv]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ w[p + "o"].T


def gla_mixer(h, w: dict, p: str, m: dict, eps: float):
    T = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, V)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / float(m["tau"])).view(T, H, D)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = alpha[t, hd][:, None] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(h, w: dict, p: str, m: dict, eps: float):
    left = sink_attention(h, w, p + "left.", m["left"], eps)
    right = gla_mixer(h, w, p + "right.", m["right"], eps)
    return 0.5 * (unit_rms(left, eps) * w[p + "left.out"] + unit_rms(right, eps) * w[p + "right.out"])


def retention_mixer(h, w: dict, p: str, m: dict, eps: float):
    T = h.shape[0]
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = rotate_half((h @ w[p + "q"].T).view(T, H, D), pos, m["rot"])
    k = rotate_half((h @ w[p + "k"].T).view(T, H, D), pos, m["rot"]) * D ** -0.5
    v = (h @ w[p + "v"].T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = float(m["decay"][hd]) * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps)
    return (o.reshape(T, H * V) * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def dense_ff(h, w: dict, p: str):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


MIXERS = {"delta": delta_mixer, "parallel": parallel_mixer, "retention": retention_mixer}


def layer(x, w: dict, i: int, L: dict, cfg: dict):
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    p = f"l{i}."
    x = x + m * MIXERS[L["type"]](tanh_norm(x, w, p + "norm1"), w, p + "mix.", L["mixer"], eps)
    if L.get("mlp"):
        x = x + m * dense_ff(tanh_norm(x, w, p + "norm2"), w, p + "mlp.")
    return x


def layer_order(cfg: dict):
    """[(layer index, pass number or None, first of its pass)] in running order."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None, False) for i in range(a)]
    for t in range(times):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def forward(cfg: dict, weights: dict, tokens, trace: list | None = None):
    """Logits [T, vocab] of one whole sequence; `trace` receives the stream after every layer run."""
    w = {k: v.to(F64) for k, v in weights.items()}
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    for i, t, first in layer_order(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], cfg)
        if trace is not None:
            trace.append(x.clone())
    z = tanh_norm(x, w, "final.norm") @ w["head"].T * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    return float(cap) * torch.tanh(z / float(cap)) if cap else z
