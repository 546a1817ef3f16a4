"""Muderax: a decoder-only family whose layer list comes from the checkpoint's ``config.json``.

Every layer is ``x += n1(mixer(x)); x += n2(ffn(x))`` on an fp32 residual stream, where the sublayers read the stream
itself and ``n`` is a one-number RMS norm on the sublayer's OUTPUT.  Mixers:

* ``latent_attention`` -- attention whose keys and values are up-projected from a cached low-rank latent (plus a single
  rotated key slice that every head uses), sliding-window mask, interleaved rotary pairs with YaRN frequency scaling;
* ``rglru`` -- a gelu branch times a real-gated linear recurrence over a short causal convolution, gates block-diagonal.

The feed-forward is a routed mixture of gated-SiLU experts (softmax over the chosen router logits) plus an always-on
shared expert.  A layer may borrow another layer's weights (``weights_of``) while keeping its own cache or state.

This module holds the configuration (parsed from / written to the ``config.json`` dictionary), the checkpoint's tensor
naming, random initialisation for tests and benchmarks, and named configurations.  The forward pass lives in
``engine/layered_runner.py`` on the kernels of ``ops/layers.py``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

LRU_DECAY_SCALE = 8.0       # log a = -8 r softplus(lam)
NO_WINDOW = 2 ** 31 - 1


@dataclass(frozen=True)
class RotarySpec:
    dims: int
    base: float
    factor: float = 1.0       # YaRN: 1 = no scaling entry
    original: float = 0.0
    fast: float = 0.0
    slow: float = 0.0

    @property
    def scaled(self) -> bool:
        return self.original > 0

    def frequencies(self) -> torch.Tensor:
        """float64 [dims / 2]: base^(-2i/dims), blended towards f / factor for the slow dimensions (YaRN)."""
        i = torch.arange(self.dims // 2, dtype=torch.float64)
        f = self.base ** (-2.0 * i / self.dims)
        if not self.scaled:
            return f

        def dim_of(turns: float) -> float:
            return self.dims * math.log(self.original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

        lo = max(math.floor(dim_of(self.fast)), 0)
        hi = min(math.ceil(dim_of(self.slow)), self.dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / self.factor * ramp + f * (1.0 - ramp)

    @property
    def amplitude(self) -> float:
        return 0.1 * math.log(self.factor) + 1.0 if self.scaled else 1.0

    def table(self, max_pos: int, width: int, device=None) -> torch.Tensor:
        """fp32 [max_pos, width / 2, 2] (cos, sin) x amplitude for a rotated part `width` wide; pairs past
        dims / 2 are the identity (those coordinates pass unchanged)."""
        ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * self.frequencies()[None, :]
        t = torch.zeros(max_pos, width // 2, 2, dtype=torch.float64)
        t[:, :, 0] = 1.0
        t[:, : self.dims // 2, 0] = ang.cos() * self.amplitude
        t[:, : self.dims // 2, 1] = ang.sin() * self.amplitude
        return t.float().to(device)


@dataclass(frozen=True)
class LatentAttentionSpec:
    heads: int
    dim: int         # unrotated query / key width per head
    rot_dim: int     # rotated width per head (the key's rotated part is shared by the heads)
    vdim: int
    kv_rank: int
    window: int
    scale: float
    rot: RotarySpec


@dataclass(frozen=True)
class RglruSpec:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class MoeSpec:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0    # 0 = no shared expert


@dataclass(frozen=True)
class LayerSpec:
    kind: str             # "latent_attention" | "rglru"
    mixer: object
    mlp: MoeSpec | None
    weights_of: int       # index of the layer whose tensors it uses (its own index when it has its own)


@dataclass(frozen=True)
class MuderaxConfig:
    vocab_size: int
    width: int
    eps: float
    layers: tuple
    name: str = "muderax"
    max_position: int = 32768
    bos_token_id: int = 1
    eos_token_id: int = 2
    raw: dict = field(default=None, compare=False, hash=False, repr=False)

    family = "muderax"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    # ---- config.json <-> dataclasses
    @classmethod
    def from_dict(cls, d: dict, name: str = "muderax") -> "MuderaxConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            m = L["mixer"]
            if L["type"] == "latent_attention":
                r = m["rot"]
                sc = r.get("scaling") or {}
                rot = RotarySpec(dims=int(r["dims"]), base=float(r["base"]), factor=float(sc.get("factor", 1.0)),
                                 original=float(sc.get("original", 0.0)), fast=float(sc.get("fast", 0.0)),
                                 slow=float(sc.get("slow", 0.0)))
                mask = m.get("mask") or {}
                mixer = LatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                            vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]),
                                            window=int(mask.get("size", NO_WINDOW)), scale=float(m["scale"]), rot=rot)
            elif L["type"] == "rglru":
                mixer = RglruSpec(width=int(m["width"]), blocks=int(m["blocks"]), conv=int(m["conv"]))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            mlp = None
            if f:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
                sh = f.get("shared") or {}
                mlp = MoeSpec(experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                              ff=int(f["expert"]["ff"]), shared_ff=int(sh.get("ff", 0)))
            layers.append(LayerSpec(kind=L["type"], mixer=mixer, mlp=mlp, weights_of=int(L.get("weights_of", i))))
        for i, L in enumerate(layers):  # a borrower of a borrower uses the tensors of the layer that owns them
            j, hops = L.weights_of, 0
            while layers[j].weights_of != j and hops < len(layers):
                j, hops = layers[j].weights_of, hops + 1
            if j != L.weights_of:
                layers[i] = LayerSpec(kind=L.kind, mixer=L.mixer, mlp=L.mlp, weights_of=j)
        cfg = cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]),
                  layers=tuple(layers), name=name, raw=d)
        cfg.validate()
        return cfg

    def to_dict(self) -> dict:
        out = {"architecture": "Muderax", "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
               "layers": []}
        for i, L in enumerate(self.layers):
            m = L.mixer
            if L.kind == "latent_attention":
                rot = {"base": m.rot.base, "dims": m.rot.dims}
                if m.rot.scaled:
                    rot["scaling"] = {"factor": m.rot.factor, "original": m.rot.original, "fast": m.rot.fast,
                                      "slow": m.rot.slow}
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                         "scale": m.scale, "rot": rot}
                if m.window != NO_WINDOW:
                    mixer["mask"] = {"size": m.window}
            else:
                mixer = {"width": m.width, "blocks": m.blocks, "conv": m.conv}
            e = {"type": L.kind, "mixer": mixer, "mlp": None}
            if L.mlp is not None:
                e["mlp"] = {"kind": "moe", "router": {"experts": L.mlp.experts, "top": L.mlp.top},
                            "expert": {"ff": L.mlp.ff}}
                if L.mlp.shared_ff:
                    e["mlp"]["shared"] = {"ff": L.mlp.shared_ff}
            if L.weights_of != i:
                e["weights_of"] = L.weights_of
            out["layers"].append(e)
        return out

    def validate(self, tp: int = 1) -> None:
        if tp != 1:
            raise ValueError("Muderax runs on one GPU per replica (no tensor-parallel sharding of its layers)")
        for i, L in enumerate(self.layers):
            src = self.layers[L.weights_of]
            # a borrower runs with its OWN constants (window, scale, rotation) on the lender's tensors: the kinds and
            # every tensor shape must agree
            if L.weights_of != i and (src.weights_of != L.weights_of or src.kind != L.kind or
                                      _shape_key(src) != _shape_key(L)):
                raise ValueError(f"layer {i} borrows the weights of layer {L.weights_of}, whose tensors differ in shape")
            m = L.mixer
            if L.kind == "latent_attention":
                if m.rot_dim % 2 or m.rot.dims % 2 or m.rot.dims > m.rot_dim or m.kv_rank > 1024 or m.window < 1:
                    raise ValueError(f"layer {i}: rotated widths must be even, rot.dims <= rot_dim, kv_rank <= 1024")
            elif m.width % m.blocks or m.conv < 1:
                raise ValueError(f"layer {i}: recurrent width must divide into its blocks, conv >= 1")
            if L.mlp is not None and not 1 <= L.mlp.top <= L.mlp.experts:
                raise ValueError(f"layer {i}: top must be within 1..experts")

    def num_params(self) -> int:
        n = 2 * self.vocab_size * self.width + 1
        for i, L in enumerate(self.layers):
            if L.weights_of == i:
                n += sum(math.prod(s) for s in layer_tensor_shapes(self, i).values())
        return n

    def cache_bytes_per_token(self, elem_bytes: int = 2) -> int:
        return sum((L.mixer.kv_rank + L.mixer.rot_dim) * elem_bytes for L in self.layers
                   if L.kind == "latent_attention")


def _shape_key(L: LayerSpec) -> tuple:
    m = L.mixer
    mix = (m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank) if L.kind == "latent_attention" else (m.width, m.blocks, m.conv)
    f = L.mlp
    return mix, (None if f is None else (f.experts, f.ff, f.shared_ff))


def layer_tensor_shapes(cfg: MuderaxConfig, i: int) -> dict:
    """{tensor name: shape} of layer i's own tensors (checkpoint naming, linear weights [out, in])."""
    L, W, p = cfg.layers[i], cfg.width, f"l{i}."
    m = L.mixer
    s = {p + "norm1": ()}
    if L.kind == "latent_attention":
        s.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                  p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                  p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.o": (W, m.heads * m.vdim)})
    else:
        bw = m.width // m.blocks
        s.update({p + "mix.y": (m.width, W), p + "mix.y.b": (m.width,), p + "mix.x": (m.width, W),
                  p + "mix.x.b": (m.width,), p + "mix.conv": (m.width, m.conv), p + "mix.conv.b": (m.width,),
                  p + "mix.ra": (m.blocks, bw, bw), p + "mix.ra.b": (m.blocks, bw), p + "mix.ri": (m.blocks, bw, bw),
                  p + "mix.ri.b": (m.blocks, bw), p + "mix.lam": (m.width,), p + "mix.o": (W, m.width)})
    if L.mlp is not None:
        f = L.mlp
        s[p + "norm2"] = ()
        names = [f"e{e}" for e in range(f.experts)] + (["shared"] if f.shared_ff else [])
        for n in names:
            ff = f.shared_ff if n == "shared" else f.ff
            s.update({f"{p}mlp.{n}.gate": (ff, W), f"{p}mlp.{n}.up": (ff, W), f"{p}mlp.{n}.down": (W, ff)})
        s.update({p + "mlp.router": (f.experts, W), p + "mlp.router.b": (f.experts,)})
    return s


def tensor_shapes(cfg: MuderaxConfig) -> dict:
    s = {"embed": (cfg.vocab_size, cfg.width)}
    for i, L in enumerate(cfg.layers):
        if L.weights_of == i:
            s.update(layer_tensor_shapes(cfg, i))
    s.update({"final.norm": (), "head": (cfg.vocab_size, cfg.width)})
    return s


@torch.no_grad()
def init_weights(cfg: MuderaxConfig, seed: int = 0, device="cpu", dtype=torch.bfloat16) -> dict:
    """Random weights in the checkpoint's naming: projections ~ N(0, 1 / fan-in), norm gains near 1, recurrence
    parameters spread so that decays cover fast and slow channels."""
    dev = torch.device(device)
    gdev = dev if dev.type == "cuda" else torch.device("cpu")   # large models are drawn on the GPU itself
    g = torch.Generator(device=gdev).manual_seed(seed)
    out = {}

    def randn(shape):
        return torch.randn(shape, generator=g, device=gdev)

    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if name == "embed":
            t = randn(shape)
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.2 * randn(shape)
        elif name.endswith("dkv.norm"):
            t = 1.0 + 0.1 * randn(shape)
        elif leaf == "lam":
            t = torch.rand(shape, generator=g, device=gdev) * 4.0 - 3.0
        elif leaf == "b":
            t = 0.3 * randn(shape)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(dtype).to(dev)
    return out


def _uniform(n_layers: int, pattern: tuple, att: LatentAttentionSpec, rec: RglruSpec, mlp: MoeSpec) -> tuple:
    return tuple(LayerSpec(kind=k, mixer=att if k == "latent_attention" else rec, mlp=mlp, weights_of=i)
                 for i, k in ((i, pattern[i % len(pattern)]) for i in range(n_layers)))


def _named(name: str, vocab: int, width: int, n_layers: int, heads: int, dim: int, rot_dim: int, vdim: int, rank: int,
           window: int, rec_width: int, blocks: int, experts: int, top: int, ff: int, shared_ff: int,
           max_position: int = 32768) -> MuderaxConfig:
    att = LatentAttentionSpec(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=rank, window=window,
                              scale=1.0 / math.sqrt(dim + rot_dim),
                              rot=RotarySpec(dims=rot_dim, base=10000.0, factor=8.0, original=4096.0, fast=32.0, slow=1.0))
    rec = RglruSpec(width=rec_width, blocks=blocks, conv=4)
    mlp = MoeSpec(experts=experts, top=top, ff=ff, shared_ff=shared_ff)
    cfg = MuderaxConfig(vocab_size=vocab, width=width, eps=1e-6, name=name, max_position=max_position,
                        layers=_uniform(n_layers, ("rglru", "rglru", "latent_attention"), att, rec, mlp))
    cfg.validate()
    return cfg


# Named configurations (random weights): a toy for smoke runs and sizes that resemble real models' layers for the
# benchmark -- "mid" has the per-layer shapes of a ~2B hybrid, "wide" the 4096-wide layers of a 7B-class model.
TINY = _named("muderax-tiny", vocab=512, width=128, n_layers=3, heads=4, dim=32, rot_dim=16, vdim=32, rank=64,
              window=48, rec_width=160, blocks=4, experts=6, top=2, ff=80, shared_ff=112, max_position=4096)
MID = _named("muderax-mid", vocab=32768, width=2048, n_layers=6, heads=16, dim=128, rot_dim=64, vdim=128, rank=512,
             window=2048, rec_width=2560, blocks=10, experts=16, top=2, ff=1408, shared_ff=2816)
WIDE = _named("muderax-wide", vocab=32768, width=4096, n_layers=6, heads=32, dim=128, rot_dim=64, vdim=128, rank=512,
              window=4096, rec_width=4096, blocks=16, experts=16, top=2, ff=3584, shared_ff=7168)

CONFIGS = {c.name: c for c in (TINY, MID, WIDE)}
