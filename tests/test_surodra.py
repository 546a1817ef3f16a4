"""Surodra on the engine against the plain oracle (tests/surodra_oracle.py).

Every test builds its own small configuration and random weights, drives the engine through its own entry points
(LLMEngine.force_step for given tokens, add_request + step for generation) and compares the logits with the oracle's
whole-sequence forward in float64.  The same tests run on the CPU (PyTorch reference ops: scheduler, cache and state
plumbing) and, marked ``gpu``, on the HIP kernels in fp32 (tight tolerance) and bf16.
"""
from __future__ import annotations

import copy
import json

import pytest
import torch

import surodra_oracle as oracle
from distributed_sse_for_llm_response_amd.engine.engine import LLMEngine, SamplingParams
from distributed_sse_for_llm_response_amd.engine.weights import convert_surodra
from distributed_sse_for_llm_response_amd.models import registry
from distributed_sse_for_llm_response_amd.models.surodra import HalfRotarySpec, SurodraConfig, init_weights, tensor_shapes

GPU = pytest.param("cuda", marks=pytest.mark.gpu)
DEVICES = ["cpu", GPU]


def delta(heads=4, kv_heads=2, dim=12, vdim=10, conv=3):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def rot(dims, base=300.0, factor=None):
    r = {"base": base, "dims": dims}
    if factor:
        r["scaling"] = {"factor": factor}
    return r


def par(heads=4, kv_heads=2, dim=12, vdim=10, dims=8, factor=4.0, scale=0.3, rheads=3, rdim=9, rvdim=7, tau=8.0):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot(dims, factor=factor)},
        "right": {"heads": rheads, "dim": rdim, "vdim": rvdim, "tau": tau}}}


def ret(heads=3, dim=10, vdim=6, decay=None, dims=None):
    decay = decay or [1.0 - 2.0 ** (-2 - h) for h in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                                           "rot": rot(dim if dims is None else dims, base=1000.0)}}


def ff(layer, n=20):
    layer = copy.deepcopy(layer)
    layer["mlp"] = {"kind": "dense", "ff": n}
    return layer


def config(layers, width=28, vocab=61, eps=2e-6, loop=None, mult=0.6, logit_scale=0.5, cap=8.0):
    out = []
    for L in layers:
        L = copy.deepcopy(L)
        L.setdefault("mlp", None)
        out.append(L)
    d = {"architecture": "Surodra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out,
         "residual_mult": mult, "logit_scale": logit_scale}
    if cap:
        d["logit_softcap"] = cap
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


HYBRID = config([delta(), ff(par()), ret(), ff(delta(heads=2, kv_heads=2, conv=4))], loop=(1, 3, 2))


class Model:
    """Configuration + random weights + an engine on `device` in `dtype`."""

    def __init__(self, cfg_dict, device, dtype=torch.float32, seed=0, max_tokens=256, max_seqs=4, tweak=None):
        self.cfg_dict = cfg_dict
        self.cfg = SurodraConfig.from_dict(cfg_dict)
        self.weights = init_weights(self.cfg, seed=seed)
        if tweak:
            tweak(self.weights)
        self.device, self.dtype = torch.device(device), dtype
        w = convert_surodra(self.cfg, self.weights, device=self.device, dtype=dtype)
        fam = registry.family_of(self.cfg)
        assert fam.name == "surodra"
        self.runner = registry.make_runner(fam, w, num_blocks=-(-max_tokens // 32), max_batch=max_seqs,
                                           max_model_len=max_tokens, max_prefill_tokens=max_tokens, device=self.device,
                                           use_graphs=False)
        self.engine = LLMEngine(self.runner, eos_id=-1)
        self.engine.watermark = 0

    def expect(self, tokens, cfg_dict=None, weights=None):
        return oracle.forward(cfg_dict or self.cfg_dict, weights or self.weights, tokens).float()

    def tol(self):
        return 2e-4 if self.dtype == torch.float32 else 6e-2

    def check(self, got, want, what=""):
        """Row-wise: rms of the difference (mean taken off) over the rms of the expected logits; every row is judged."""
        got, want = got.detach().float().cpu(), want.float()
        assert got.shape == want.shape, (got.shape, want.shape)
        assert torch.isfinite(got).all(), what
        d = got - want
        d = d - d.mean(-1, keepdim=True)
        err = d.pow(2).mean(-1).sqrt() / (want - want.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().clamp_min(1e-6)
        assert float(err.max()) < self.tol(), f"{what}: worst row {int(err.argmax())} error {float(err.max()):.3g}"

    def run_cut(self, cid, tokens, cuts, end=True):
        """Feed `tokens` in portions of the given sizes (the last size repeats), all logits wanted."""
        out, at, k = [], 0, 0
        while at < len(tokens):
            n = min(cuts[min(k, len(cuts) - 1)], len(tokens) - at)
            last = at + n == len(tokens)
            out.append(self.engine.force_step([(cid, tokens[at:at + n], list(range(n)))], [cid] if last and end else []))
            at, k = at + n, k + 1
        return torch.cat(out)


def toks(n, vocab=61, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def modes(device):
    return [torch.float32] if device == "cpu" else [torch.float32, torch.bfloat16]


def gap(a, b, rows=slice(None)):
    """Median over rows of |a - b| rms relative to b's rms: how far a variant of the design is from the design."""
    a, b = a[rows], b[rows]
    return float(((a - b).pow(2).mean(-1).sqrt() / b.pow(2).mean(-1).sqrt().clamp_min(1e-6)).median())


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cfgd", [
    ("delta rule, grouped keys", config([delta()])),
    ("delta rule, a key head per head, one tap", config([delta(heads=3, kv_heads=3, conv=1)])),
    ("sink attention beside gated linear attention", config([par()])),
    ("rotation of the whole head, no position scaling", config([par(dims=12, factor=None, kv_heads=4)])),
    ("no rotation at all", config([par(dims=0, factor=None, kv_heads=1)])),
    ("retention", config([ret()])),
    ("retention, part of the head rotated", config([ret(dims=4)])),
    ("dense feed-forward", config([ff(ret(heads=1))])),
    ("no logit cap, no logit scale, unit residual", config([ff(delta())], mult=1.0, logit_scale=1.0, cap=None)),
    ("a loop of one layer, three passes", config([ret(), ff(delta()), ret()], loop=(1, 2, 3))),
    ("a loop of everything, one pass", config([delta(), par()], loop=(0, 2, 1))),
])
def test_mechanism_alone(device, name, cfgd):
    for dtype in modes(device):
        m = Model(cfgd, device, dtype)
        t = toks(37)
        m.check(m.run_cut("a", t, [len(t)]), m.expect(t), name)


def test_each_mixer_against_its_oracle_function():
    """The engine's layer trace (stream after every layer run) against the oracle's, mixer by mixer."""
    from distributed_sse_for_llm_response_amd.engine.model_runner import PrefillSeq

    m = Model(HYBRID, "cpu")
    t = toks(29, seed=3)
    want = []
    oracle.forward(HYBRID, m.weights, t, want)
    got = []
    m.runner.prefill([PrefillSeq(slot=0, tokens=t, start_pos=0, block_table=[0], last_chunk=False)], 0, trace=got)
    assert len(got) == len(want) == 6     # layer 0, layers 1-2 twice, layer 3
    for i, (g, w) in enumerate(zip(got, want)):
        assert torch.allclose(g.double(), w, atol=2e-4, rtol=2e-4), f"layer run {i}"


def test_rotation_table_matches_oracle():
    for factor in (None, 4.0):
        r = rot(8, factor=factor)
        tab = HalfRotarySpec.from_dict(r).table(50).double()
        v = torch.randn(50, 3, 12, dtype=torch.float64)
        want = oracle.rotate_half(v, torch.arange(50), r)
        a, b = v[..., :4], v[..., 4:8]
        got = v.clone()
        got[..., :4] = a * tab[:, None, :, 0] - b * tab[:, None, :, 1]
        got[..., 4:8] = b * tab[:, None, :, 0] + a * tab[:, None, :, 1]
        assert torch.allclose(got, want, atol=1e-5)
        assert torch.equal(got[..., 8:], v[..., 8:])


# ---------------------------------------------------------------------------------------------- cuts and batches
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_against_token_by_token(device):
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        t = toks(45, seed=1)
        want = m.expect(t)
        m.check(m.run_cut("whole", t, [len(t)]), want, "whole prompt")
        m.check(m.run_cut("single", t, [1]), want, "token by token")
        m.check(m.run_cut("tail", t, [30, 1]), want, "prompt, then decoded tokens")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 7], [5, 1, 1, 2, 11], [31, 2, 1], [33, 1], [64, 2]])
def test_portions(device, cuts):
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        t = toks(70, seed=2)
        m.check(m.run_cut("p", t, cuts), m.expect(t), f"portions {cuts}")


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_against_each_alone(device):
    """Four requests of unequal length advance together, portions beside single tokens; one is left out of some steps
    and one starts with a single token."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        seqs = {"a": toks(50, seed=3), "b": toks(9, seed=4), "c": toks(33, seed=5), "d": toks(21, seed=6)}
        plan = {"a": [17, 2, 1, 1, 1, 9, 1], "b": [1, 1, 1, 1], "c": [2, 30, 1], "d": [1, 3, 1, 1, 5, 1]}
        at = {k: 0 for k in seqs}
        got = {k: [] for k in seqs}
        step = 0
        while any(at[k] < len(seqs[k]) for k in seqs):
            entries, names = [], []
            for k, t in seqs.items():
                if at[k] >= len(t) or (k == "c" and step % 3 == 1):
                    continue
                p = plan[k]
                n = min(p[min(step, len(p) - 1)], len(t) - at[k])
                entries.append((k, t[at[k]:at[k] + n], list(range(n))))
                names.append((k, n))
                at[k] += n
            out = m.engine.force_step(entries, [k for k, _ in names if at[k] == len(seqs[k])])
            o = 0
            for k, n in names:
                got[k].append(out[o:o + n])
                o += n
            step += 1
        for k, t in seqs.items():
            m.check(torch.cat(got[k]), m.expect(t), f"request {k} in the batch")
        assert m.engine.alloc.num_free == m.engine.alloc.num_blocks and all(s is None for s in m.engine.slots)


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(device):
    """A pool of three pages and two slots serves a stream of requests: every page and every state slot changes hands,
    also while the other slot's sequence is still running, and a stale matrix state, convolution tail or cache row
    would show."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype, max_tokens=96, max_seqs=2)
        long = toks(60, seed=7)
        m.engine.force_step([("long", long[:20], [])])
        at = 20
        for i, n in enumerate([30, 5, 32, 1, 17, 29]):
            t = toks(n, seed=10 + i)
            out = m.engine.force_step([(f"s{i}", t, list(range(n))), ("long", long[at:at + 2], [])], [f"s{i}"])
            at += 2
            m.check(out, m.expect(t), f"request {i} in a used slot")
        out = m.engine.force_step([("long", long[at:], list(range(len(long) - at)))], ["long"])
        m.check(out, m.expect(long)[at:], "the request that ran beside them")
        assert m.engine.alloc.num_free == 3


@pytest.mark.parametrize("device", DEVICES)
def test_pool_exhaustion_raises(device):
    m = Model(config([par()]), device, max_tokens=64, max_seqs=2)
    m.engine.force_step([("a", toks(40), [])])
    with pytest.raises(MemoryError):
        m.engine.force_step([("b", toks(40), [])])


# ---------------------------------------------------------------------------------------------- what random weights hide
def _sharp(w):
    """Sharpen attention so that single keys carry the weight, and let the attention half of a parallel pair lead."""
    for k in w:
        if k.endswith("left.q.norm"):
            w[k] = (w[k].float() * 5.0).to(w[k].dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_among_hundreds(device):
    """One early token stays visible from far away through the attention's pages (no window): its loss -- a cache row
    overwritten, a page mapped wrongly -- would change later logits.  Portions end on and off page borders."""
    cfgd = config([par(kv_heads=1), ff(par(heads=2, kv_heads=2))], cap=None)
    t = toks(300, seed=9)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, max_tokens=320, tweak=_sharp)
        want = m.expect(t)
        moved = t[:]
        moved[3] = (moved[3] + 1) % 61
        assert float((m.expect(moved) - want)[250:].abs().max()) > 1e-2, "far tokens do not matter in this construction"
        m.check(m.run_cut("f", t, [290, 1]), want, "far keys, prompt then decoding")
        m.check(m.run_cut("g", t, [64, 32, 1, 95, 2]), want, "far keys, portions on page borders")


@pytest.mark.parametrize("device", DEVICES)
def test_sink_counts_once_and_unscaled(device):
    """Large sinks: a denominator without the sink, with the sink scaled like a score, or with it counted per key
    would be far from the design; the engine is not."""
    def big_sinks(w):
        for k in w:
            if k.endswith("left.sink"):
                w[k] = (w[k].float() + 2.5).to(w[k].dtype)

    cfgd = config([par(scale=0.05), par(heads=2, kv_heads=1, scale=0.05)])
    t = toks(60, seed=15)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, tweak=big_sinks)
        want = m.expect(t)
        none = {k: (v.float() - 60.0).to(v.dtype) if k.endswith("left.sink") else v for k, v in m.weights.items()}
        scaled = {k: (v.float() * 0.05).to(v.dtype) if k.endswith("left.sink") else v for k, v in m.weights.items()}
        for other, what in ((none, "no sink"), (scaled, "a scaled sink")):
            if dtype == torch.float32:  # the fp32 run is the judge of the sink
                assert gap(m.expect(t, weights=other), want) > 100 * m.tol(), f"the test would not see {what}"
        m.check(m.run_cut("s", t, [len(t)]), want, "sinks, whole prompt")
        m.check(m.run_cut("d", t, [20, 3, 1]), want, "sinks, portions and decoding")


@pytest.mark.parametrize("device", DEVICES)
def test_state_carries_far(device):
    """Slow decays: what an early token wrote into the matrix states still shapes the logits two hundred tokens on,
    across portions, decoding and a slot that changes hands in between."""
    def slow(w):
        for k in w:
            if k.endswith("A_log"):
                w[k] = (w[k].float() - 6.0).to(w[k].dtype)       # delta rule: g close to 1
            if k.endswith("a2.b"):
                w[k] = (w[k].float() + 4.0).to(w[k].dtype)       # gated linear attention: alpha close to 1

    cfgd = config([delta(), par(), ret(decay=[0.999, 0.9995, 1.0])], cap=None)
    t = toks(230, seed=16)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, max_tokens=256, max_seqs=2, tweak=slow)
        want = m.expect(t)
        moved = t[:]
        moved[2] = (moved[2] + 7) % 61
        assert float((m.expect(moved) - want)[200:].abs().max()) > 1e-2, "early tokens do not matter in this construction"
        m.check(m.run_cut("a", t, [200, 1]), want, "prompt, then decoding")
        got = [m.engine.force_step([("b", t[:90], list(range(90)))])]
        m.run_cut("other", toks(40, seed=17), [13, 1])                     # another sequence comes and goes
        got.append(m.run_cut("b", t[90:], [2, 61, 1]))
        m.check(torch.cat(got), want, "portions with another sequence in between")


@pytest.mark.parametrize("device", DEVICES)
def test_delta_write_is_seen_by_its_own_read(device):
    """beta near 1 and no decay: the delta rule replaces what the key recalled with the new value, and the read-out of
    the same token sees it.  An update that reads before it writes, or that forgets the correction term, is far off."""
    def strong(w):
        for k in w:
            if k.endswith("mix.b"):
                w[k] = (w[k].float() * 0.0).to(w[k].dtype)
            if k.endswith("A_log"):
                w[k] = (w[k].float() - 8.0).to(w[k].dtype)

    cfgd = config([delta(heads=2, kv_heads=1, dim=6, vdim=5)], cap=None)
    t = toks(50, seed=18)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, tweak=strong)
        m.check(m.run_cut("w", t, [len(t)]), m.expect(t), "whole")
        m.check(m.run_cut("d", t, [7, 2, 1]), m.expect(t), "portions and decoding")


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device):
    """Positions 0, 1, 2: the convolution's empty history, the recurrences from a zero state, one-key attention (where
    the sink weighs most); as a one-token request, as single tokens from the start, and in a slot that held another
    sequence."""
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype, max_seqs=1)
        m.run_cut("warm", toks(40, seed=11), [40])
        for n in (1, 2, 3):
            t = toks(n, seed=12 + n)
            m.check(m.run_cut(f"n{n}", t, [1]), m.expect(t), f"{n} first tokens, one by one")
            m.check(m.run_cut(f"w{n}", t, [n]), m.expect(t), f"{n} first tokens, at once")


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(device):
    """Decoding runs over several pages; every state is carried through every step."""
    t = toks(150, seed=13)
    for dtype in modes(device):
        m = Model(HYBRID, device, dtype)
        m.check(m.run_cut("l", t, [5, 1]), m.expect(t), "long decoding")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cfgd", [
    ("all ones", config([delta(heads=1, kv_heads=1, dim=1, vdim=1, conv=1),
                         ff(par(heads=1, kv_heads=1, dim=2, vdim=1, dims=2, rheads=1, rdim=1, rvdim=1), 1),
                         ret(heads=1, dim=2, vdim=1)], width=2, vocab=7, loop=(0, 3, 1))),
    ("odd sizes", config([delta(heads=6, kv_heads=2, dim=7, vdim=9, conv=5), ff(par(heads=6, kv_heads=3, dim=14, vdim=5,
                                                                                     dims=6, rheads=5, rdim=11, rvdim=13), 17),
                          ff(ret(heads=5, dim=6, vdim=11, dims=2), 9)], width=19, vocab=23, loop=(1, 3, 2))),
    ("sizes that vector loads like", config([ff(delta(heads=4, kv_heads=4, dim=32, vdim=64, conv=4), 128),
                                             ff(par(heads=8, kv_heads=2, dim=64, vdim=32, dims=32, rheads=2, rdim=64,
                                                    rvdim=128), 128), ret(heads=4, dim=32, vdim=32)], width=64, vocab=96)),
    ("key widths over several waves", config([delta(heads=2, kv_heads=1, dim=80, vdim=70),
                                              par(heads=2, kv_heads=1, dim=136, vdim=72, dims=64, rheads=1, rdim=264,
                                                  rvdim=40), ret(heads=1, dim=130, vdim=66)], width=48, vocab=50)),
    ("projections on the tiled-layout GEMMs", config([delta(heads=8, kv_heads=4, dim=64, vdim=128),
                                                      ff(par(heads=8, kv_heads=4, dim=128, vdim=64, dims=64, rheads=4,
                                                             rdim=64, rvdim=64), 2048),
                                                      ret(heads=4, dim=128, vdim=128)], width=1024, vocab=1024)),
])
def test_other_sizes(device, name, cfgd):
    vocab = cfgd["vocab"]
    t = toks(41, vocab=vocab, seed=14)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype)
        m.check(m.run_cut("x", t, [len(t)]), m.expect(t), name + ", whole")
        m.check(m.run_cut("y", t, [7, 2, 1]), m.expect(t), name + ", portions and decoding")


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompts_over_many_pages(device):
    """Three hundred tokens: prompts cut on and off page borders, then decoding, loops with their own pages."""
    cfgd = config([ff(par(heads=4, kv_heads=2, dim=32, vdim=16, dims=16, rheads=2, rdim=16, rvdim=24), 64),
                   delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=4), ret(heads=2, dim=32, vdim=16)],
                  width=96, vocab=200, loop=(0, 2, 2))
    t = toks(300, vocab=200, seed=50)
    for dtype in modes(device):
        m = Model(cfgd, device, dtype, max_tokens=320)
        want = m.expect(t)
        m.check(m.run_cut("a", t, [280, 1]), want, "prompt, then decoding")
        m.check(m.run_cut("b", t, [64, 3, 97, 1]), want, "portions")


# ---------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(device):
    """add_request + step: admission, chunked prompt passes (a 16-token budget), mixed steps, decode with sampling at
    temperature 0, slot release.  Each generated token is the oracle's argmax given the tokens before it (a step
    whose two best logits are closer than the tolerance is not judged)."""
    m = Model(HYBRID, device, torch.float32, max_tokens=512, max_seqs=3)
    eng = LLMEngine(m.runner, eos_id=-1, prefill_budget=16, idle_prefill_budget=16)
    prompts = {"g0": toks(19, seed=20), "g1": toks(40, seed=21), "g2": toks(3, seed=22), "g3": toks(33, seed=23)}
    for cid, p in prompts.items():
        eng.add_request(cid, p, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    out = {cid: [] for cid in prompts}
    for ev in eng.run_until_idle():
        if not ev.done:
            out[ev.conversation_id].append(ev.token_id)
    for cid, p in prompts.items():
        assert len(out[cid]) == 12, (cid, out[cid])
        logits = m.expect(p + out[cid])
        for i, tok in enumerate(out[cid]):
            row = logits[len(p) + i - 1]
            top = torch.topk(row, 2).values
            if float(top[0] - top[1]) > 1e-3 * float(row.abs().max()):
                assert tok == int(row.argmax()), f"{cid}: token {i} is {tok}, the oracle says {int(row.argmax())}"
    assert eng.alloc.num_free == eng.alloc.num_blocks


@pytest.mark.gpu
def test_decode_graphs_match_eager():
    """The captured decode step replayed over several steps (with eager work between the replays) gives the eager
    step's logits."""
    m = Model(HYBRID, "cuda", torch.bfloat16)
    t = toks(60, seed=30)
    eager = m.run_cut("e", t, [20, 1])
    m.runner.use_graphs = True
    m.runner.capture()
    assert m.runner.graphs
    graphed = m.run_cut("g", t, [20, 1])
    assert torch.allclose(eager, graphed, atol=1e-5, rtol=1e-5)
    m.check(graphed, m.expect(t), "graph replays")


def test_config_round_trip_and_registry(tmp_path):
    cfg = SurodraConfig.from_dict(HYBRID)
    again = SurodraConfig.from_dict(cfg.to_dict())
    assert again.layers == cfg.layers and again == cfg
    assert [(r.layer, r.pass_no) for r in cfg.runs()] == [(0, -1), (1, 0), (2, -1), (1, 1), (2, -1), (3, -1)]
    from safetensors.torch import save_file

    (tmp_path / "config.json").write_text(json.dumps(HYBRID))
    weights = init_weights(cfg, seed=3)
    weights["l1.mix.right.a1"] = weights["l1.mix.right.a1"][:5].clone()          # the checkpoint decides this width
    weights["l1.mix.right.a2"] = weights["l1.mix.right.a2"][:, :5].clone()
    save_file({k: v.contiguous() for k, v in weights.items()}, str(tmp_path / "model.safetensors"))
    fam, cfg2, path = registry.resolve(str(tmp_path))
    assert fam.name == "surodra" and cfg2.layers == cfg.layers and cfg2.width == cfg.width and path == str(tmp_path)
    w = registry.load_weights(fam, cfg2, path, device="cpu", dtype=torch.float32)
    assert w.layers[1].mix.a2.shape == (27, 5) and w.step.shape == (2, 28) and w.head.dtype == torch.float32
    assert set(tensor_shapes(cfg)) == set(weights)
    assert registry.resolve("surodra-tiny")[0].name == "surodra"
    bad = dict(weights)
    bad["l0.mix.q"] = bad["l0.mix.q"][:-1]
    with pytest.raises(ValueError):
        convert_surodra(cfg, bad)


def test_serving_builds_the_family_by_name():
    """The serving launcher's engine builder resolves the family through the registry and generates with it."""
    from distributed_sse_for_llm_response_amd.serving.app import build_engine
    from distributed_sse_for_llm_response_amd.serving.config import ServeConfig

    eng, _ = build_engine(ServeConfig(model="surodra-tiny", engine="cpu"))
    eng.add_request("c1", [5, 6, 7, 8, 9, 10], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
    eng.add_request("c2", [11, 12], SamplingParams(temperature=0.8, max_tokens=3, ignore_eos=True))
    ev = eng.run_until_idle()
    assert sum(1 for e in ev if e.conversation_id == "c1" and not e.done) == 4
    assert sum(1 for e in ev if e.conversation_id == "c2" and not e.done) == 3
