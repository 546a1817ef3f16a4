"""Surodra: a decoder-only family of matrix-state mixers whose layer list comes from the checkpoint's ``config.json``.

Every layer is pre-norm, ``x += m * mixer(n1(x)); x += m * ff(n2(x))`` on an fp32 residual stream, with the
element-wise norm ``n(v) = tanh(alpha v) w + b`` (no mean, no variance) and one residual multiplier ``m`` for the
whole model.  A layer without a feed-forward has the first sublayer only.  Mixers:

* ``delta`` -- gated delta rule: per head a matrix state ``S`` [dim, vdim] with ``S = g S``, ``u = beta (v - S^T k)``,
  ``S += k u^T``, ``o = S^T q``; q / k / v pass a short causal convolution and SiLU, q and k are unit vectors per
  head, ``g = exp(-exp(A) softplus(a + dt))`` and ``beta = sigmoid(b)`` per head; output RMS norm per head times a
  SiLU gate.
* ``parallel`` -- two mixers that read the same input, each output RMS-normed over the width and averaged:
  ``left`` is softmax attention (grouped key/value heads, RMS norm of the whole query / key projection, rotate-half
  rotary on the leading coordinates with linear position scaling, a learned sink logit per head in the softmax
  denominator, a sigmoid output gate per head), ``right`` is gated linear attention (``S = diag(alpha) S + k v^T``
  with a low-rank per-key-channel decay ``alpha = sigmoid(z)^(1 / tau)``).
* ``retention`` -- ``S = decay_h S + k v^T``, ``o = S^T q`` with a fixed decay per head and rotary q / k.

A span of layers may run several times in a row with the same weights (``loop``); each pass has its own cache and
state, the embedding re-enters before every pass but the first and a learned vector per pass is added before each.
The head's logits are scaled and soft-capped with tanh.

This module holds the configuration (parsed from / written to the ``config.json`` dictionary), the checkpoint's tensor
naming, random initialisation for tests and benchmarks, and named configurations.  The forward pass lives in
``engine/layered_runner.py`` on the kernels of ``ops/layers.py``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

NO_WINDOW = 2 ** 31 - 1
UNIT_EPS = 1e-6     # inside the root of the delta mixer's per-head unit norm
ANY = -1            # a tensor dimension that the configuration leaves to the checkpoint


@dataclass(frozen=True)
class HalfRotarySpec:
    """Rotate-half rotary: coordinate i of a head pairs with i + dims / 2; angle = pos * base^(-2i/dims) / factor."""
    dims: int
    base: float
    factor: float = 1.0

    def table(self, max_pos: int, device=None) -> torch.Tensor:
        """fp32 [max_pos, dims / 2, 2] (cos, sin), made in float64."""
        f = self.base ** (-2.0 * torch.arange(self.dims // 2, dtype=torch.float64) / self.dims) / self.factor
        ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None, :]
        return torch.stack([ang.cos(), ang.sin()], dim=-1).float().to(device)

    @classmethod
    def from_dict(cls, r: dict) -> "HalfRotarySpec":
        sc = r.get("scaling") or {}
        return cls(dims=int(r["dims"]), base=float(r["base"]), factor=float(sc.get("factor", 1.0)))

    def to_dict(self) -> dict:
        d = {"base": self.base, "dims": self.dims}
        if self.factor != 1.0:
            d["scaling"] = {"factor": self.factor}
        return d


@dataclass(frozen=True)
class DeltaSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int


@dataclass(frozen=True)
class SinkAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: HalfRotarySpec
    window: int = NO_WINDOW


@dataclass(frozen=True)
class GlaSpec:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int = 16    # inner width of the decay's low-rank projection; a checkpoint's tensors decide it


@dataclass(frozen=True)
class ParallelSpec:
    left: SinkAttentionSpec
    right: GlaSpec


@dataclass(frozen=True)
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: HalfRotarySpec


@dataclass(frozen=True)
class DenseSpec:
    ff: int


@dataclass(frozen=True)
class LayerSpec:
    kind: str             # "delta" | "parallel" | "retention"
    mixer: object
    mlp: DenseSpec | None


@dataclass(frozen=True)
class LayerRun:
    layer: int            # index into layers (and the weights)
    index: int            # index of this run: its cache and state are keyed by it
    pass_no: int          # number of the loop pass that this run opens, else -1


@dataclass(frozen=True)
class SurodraConfig:
    vocab_size: int
    width: int
    eps: float
    layers: tuple
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0     # 0 = none
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0            # 0 = the checkpoint has no loop (and no per-pass vectors)
    name: str = "surodra"
    max_position: int = 32768
    bos_token_id: int = 1
    eos_token_id: int = 2
    raw: dict = field(default=None, compare=False, hash=False, repr=False)

    family = "surodra"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """The layer runs in order: layers before the loop, the looped span `loop_times` times, the rest."""
        n = len(self.layers)
        if self.loop_times <= 0:
            order = [(i, -1) for i in range(n)]
        else:
            order = [(i, -1) for i in range(self.loop_start)]
            for t in range(self.loop_times):
                order += [(i, t if i == self.loop_start else -1) for i in range(self.loop_start, self.loop_stop)]
            order += [(i, -1) for i in range(self.loop_stop, n)]
        return [LayerRun(layer=i, index=r, pass_no=t) for r, (i, t) in enumerate(order)]

    # ---- config.json <-> dataclasses
    @classmethod
    def from_dict(cls, d: dict, name: str = "surodra") -> "SurodraConfig":
        def attention(m):
            mask = m.get("mask") or {}
            return SinkAttentionSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                     dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                                     rot=HalfRotarySpec.from_dict(m["rot"]), window=int(mask.get("size", NO_WINDOW)))

        layers = []
        for i, L in enumerate(d["layers"]):
            m = L["mixer"]
            if L["type"] == "delta":
                mixer = DeltaSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                                  vdim=int(m["vdim"]), conv=int(m["conv"]))
            elif L["type"] == "parallel":
                r = m["right"]
                mixer = ParallelSpec(left=attention(m["left"]),
                                     right=GlaSpec(heads=int(r["heads"]), dim=int(r["dim"]), vdim=int(r["vdim"]),
                                                   tau=float(r["tau"]), decay_rank=int(r.get("rank", ANY))))
            elif L["type"] == "retention":
                mixer = RetentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                      decay=tuple(float(x) for x in m["decay"]), rot=HalfRotarySpec.from_dict(m["rot"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            mlp = None
            if f:
                if f.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
                mlp = DenseSpec(ff=int(f["ff"]))
            layers.append(LayerSpec(kind=L["type"], mixer=mixer, mlp=mlp))
        loop = d.get("loop") or {}
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]), layers=tuple(layers),
                  residual_mult=float(d.get("residual_mult", 1.0)), logit_scale=float(d.get("logit_scale", 1.0)),
                  logit_softcap=float(d.get("logit_softcap") or 0.0), loop_start=int(loop.get("start", 0)),
                  loop_stop=int(loop.get("stop", 0)), loop_times=int(loop.get("times", 0)), name=name, raw=d)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        out = {"architecture": "Surodra", "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
               "residual_mult": self.residual_mult, "logit_scale": self.logit_scale, "layers": []}
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.loop_times > 0:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        for L in self.layers:
            m = L.mixer
            if L.kind == "delta":
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
            elif L.kind == "parallel":
                a, r = m.left, m.right
                left = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                        "rot": a.rot.to_dict()}
                if a.window != NO_WINDOW:
                    left["mask"] = {"size": a.window}
                mixer = {"left": left, "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "tau": r.tau}}
            else:
                mixer = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay), "rot": m.rot.to_dict()}
            out["layers"].append({"type": L.kind, "mixer": mixer,
                                  "mlp": None if L.mlp is None else {"kind": "dense", "ff": L.mlp.ff}})
        return out

    def validate(self, tp: int = 1) -> None:
        if tp != 1:
            raise ValueError("Surodra runs on one GPU per replica (no tensor-parallel sharding of its layers)")
        n = len(self.layers)
        if self.loop_times > 0 and not 0 <= self.loop_start < self.loop_stop <= n:
            raise ValueError(f"loop span {self.loop_start}..{self.loop_stop} does not fit {n} layers")

        def rotary(i, rot, dim):
            if rot.dims % 2 or rot.dims > dim or rot.dims < 0:
                raise ValueError(f"layer {i}: rot.dims must be even and at most the head width")

        for i, L in enumerate(self.layers):
            m = L.mixer
            if L.kind == "delta":
                if m.heads % m.kv_heads or m.conv < 1:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, conv >= 1")
            elif L.kind == "parallel":
                if m.left.heads % m.left.kv_heads or m.left.window < 1:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads, window >= 1")
                rotary(i, m.left.rot, m.left.dim)
            else:
                if len(m.decay) != m.heads:
                    raise ValueError(f"layer {i}: one decay per head")
                rotary(i, m.rot, m.dim)
            for s in ((m.left, m.right) if L.kind == "parallel" else (m,)):
                if max(s.dim, s.vdim) > 512:
                    raise ValueError(f"layer {i}: head widths above 512 are not supported")

    def num_params(self) -> int:
        return sum(math.prod(max(x, 1) for x in s) for s in tensor_shapes(self).values())

    def cache_bytes_per_token(self, elem_bytes: int = 2) -> int:
        """Paged cache bytes per token: the attention halves of parallel mixers, once per run of their layer."""
        n = 0
        for r in self.runs():
            L = self.layers[r.layer]
            if L.kind == "parallel":
                n += L.mixer.left.kv_heads * (L.mixer.left.dim + L.mixer.left.vdim) * elem_bytes
        return n

    def state_bytes_per_sequence(self) -> int:
        """fp32 matrix states and convolution tails of one sequence over all runs."""
        n = 0
        for r in self.runs():
            L, m = self.layers[r.layer], self.layers[r.layer].mixer
            if L.kind == "delta":
                n += m.heads * m.dim * m.vdim + (m.conv - 1) * (2 * m.kv_heads * m.dim + m.heads * m.vdim)
            elif L.kind == "parallel":
                n += m.right.heads * m.right.dim * m.right.vdim
            else:
                n += m.heads * m.dim * m.vdim
        return 4 * n


def _norm_shapes(name: str, W: int) -> dict:
    return {name: (W,), name + ".b": (W,), name + ".alpha": ()}


def layer_tensor_shapes(cfg: SurodraConfig, i: int) -> dict:
    """{tensor name: shape} of layer i (checkpoint naming, linear weights [out, in]); ANY = the checkpoint decides."""
    L, W, p = cfg.layers[i], cfg.width, f"l{i}."
    m = L.mixer
    s = _norm_shapes(p + "norm1", W)
    if L.kind == "delta":
        qk, hv = m.kv_heads * m.dim, m.heads * m.vdim
        s.update({p + "mix.q": (qk, W), p + "mix.q.conv": (qk, m.conv), p + "mix.k": (qk, W),
                  p + "mix.k.conv": (qk, m.conv), p + "mix.v": (hv, W), p + "mix.v.conv": (hv, m.conv),
                  p + "mix.b": (m.heads, W), p + "mix.A_log": (m.heads,), p + "mix.norm": (m.vdim,),
                  p + "mix.a": (m.heads, W), p + "mix.dt_bias": (m.heads,), p + "mix.g": (hv, W), p + "mix.o": (W, hv)})
    elif L.kind == "parallel":
        a, r = m.left, m.right
        pl, pr = p + "mix.left.", p + "mix.right."
        s.update({pl + "q": (a.heads * a.dim, W), pl + "k": (a.kv_heads * a.dim, W), pl + "v": (a.kv_heads * a.vdim, W),
                  pl + "q.norm": (a.heads * a.dim,), pl + "k.norm": (a.kv_heads * a.dim,), pl + "sink": (a.heads,),
                  pl + "g": (a.heads, W), pl + "o": (W, a.heads * a.vdim), pl + "out": (W,),
                  pr + "q": (r.heads * r.dim, W), pr + "k": (r.heads * r.dim, W), pr + "v": (r.heads * r.vdim, W),
                  pr + "g": (r.heads * r.vdim, W), pr + "o": (W, r.heads * r.vdim), pr + "norm": (r.vdim,),
                  pr + "a1": (r.decay_rank, W), pr + "a2": (r.heads * r.dim, r.decay_rank),
                  pr + "a2.b": (r.heads * r.dim,), pr + "out": (W,)})
    else:
        s.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W),
                  p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                  p + "mix.o": (W, m.heads * m.vdim)})
    if L.mlp is not None:
        s.update(_norm_shapes(p + "norm2", W))
        s.update({p + "mlp.gate": (L.mlp.ff, W), p + "mlp.up": (L.mlp.ff, W), p + "mlp.down": (W, L.mlp.ff)})
    return s


def tensor_shapes(cfg: SurodraConfig) -> dict:
    s = {"embed": (cfg.vocab_size, cfg.width)}
    if cfg.loop_times > 0:
        s["loop.step"] = (cfg.loop_times, cfg.width)
    for i in range(len(cfg.layers)):
        s.update(layer_tensor_shapes(cfg, i))
    s.update(_norm_shapes("final.norm", cfg.width))
    s["head"] = (cfg.vocab_size, cfg.width)
    return s


@torch.no_grad()
def init_weights(cfg: SurodraConfig, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> dict:
    """Random weights in the checkpoint's naming: projections ~ N(0, 1 / fan-in), norm gains near 1, decay parameters
    spread so that fast and slow heads and channels occur."""
    dev = torch.device(device)
    gdev = dev if dev.type == "cuda" else torch.device("cpu")
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}

    def randn(shape):
        return torch.randn(tuple(shape), generator=g, device=gdev)

    def rand(shape):
        return torch.rand(tuple(shape), generator=g, device=gdev)

    for name, shape in tensor_shapes(cfg).items():
        shape = tuple(16 if x == ANY else x for x in shape)
        leaf = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(shape)
        elif leaf == "alpha":
            t = 0.5 + 0.3 * rand(shape)
        elif leaf in ("norm1", "norm2", "out") or name == "final.norm" or name.endswith((".q.norm", ".k.norm", "mix.norm",
                                                                                         "right.norm")):
            t = 1.0 + 0.2 * randn(shape)
        elif leaf == "b" and len(shape) == 1:     # a norm's shift or the decay projection's bias
            t = 0.1 * randn(shape) + (2.0 if name.endswith("a2.b") else 0.0)
        elif leaf == "step":
            t = 0.3 * randn(shape)
        elif leaf == "conv":
            t = randn(shape) / math.sqrt(shape[-1]) + 0.3
        elif leaf == "A_log":
            t = torch.log(0.05 + 2.0 * rand(shape))
        elif leaf == "dt_bias":
            t = randn(shape) - 1.0
        elif leaf == "sink":
            t = randn(shape)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(dtype).to(dev)
    return out


def _named(name: str, vocab: int, width: int, pattern: tuple, n_layers: int, heads: int, kv_heads: int, dim: int,
           vdim: int, ff: int, loop: tuple = (0, 0, 0), max_position: int = 32768) -> SurodraConfig:
    rot = HalfRotarySpec(dims=dim // 2, base=10000.0, factor=4.0)
    mix = {
        "delta": DeltaSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=4),
        "parallel": ParallelSpec(left=SinkAttentionSpec(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim,
                                                        scale=1.0 / math.sqrt(dim), rot=rot),
                                 right=GlaSpec(heads=heads // 2, dim=dim, vdim=vdim, tau=8.0)),
        "retention": RetentionSpec(heads=heads, dim=dim, vdim=vdim,
                                   decay=tuple(1.0 - 2.0 ** (-5 - (7 * h) // max(1, heads - 1)) for h in range(heads)),
                                   rot=HalfRotarySpec(dims=dim, base=100000.0)),
    }
    layers = tuple(LayerSpec(kind=k, mixer=mix[k], mlp=DenseSpec(ff=ff) if k == "parallel" else None)
                   for k in (pattern[i % len(pattern)] for i in range(n_layers)))
    cfg = SurodraConfig(vocab_size=vocab, width=width, eps=1e-6, layers=layers, residual_mult=0.5, logit_scale=0.5,
                        logit_softcap=20.0, loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2], name=name,
                        max_position=max_position)
    cfg.validate()
    return cfg


# Named configurations (random weights): a toy for smoke runs, and sizes that resemble real models' layers for the
# benchmark -- "mid" has 2048-wide layers, "wide" the 4096-wide layers of a 7B-class model.
TINY = _named("surodra-tiny", vocab=512, width=128, pattern=("delta", "parallel", "retention"), n_layers=3, heads=4,
              kv_heads=2, dim=32, vdim=32, ff=256, loop=(0, 2, 2), max_position=4096)
MID = _named("surodra-mid", vocab=32768, width=2048, pattern=("delta", "parallel", "retention"), n_layers=6, heads=16,
             kv_heads=8, dim=128, vdim=128, ff=8192)
WIDE = _named("surodra-wide", vocab=32768, width=4096, pattern=("delta", "parallel", "retention"), n_layers=6, heads=32,
              kv_heads=8, dim=128, vdim=128, ff=14336)

CONFIGS = {c.name: c for c in (TINY, MID, WIDE)}
