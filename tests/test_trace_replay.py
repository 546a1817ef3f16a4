"""The trace replayer (bin/trace_run, engine/trace.py) and LLMEngine.force_step on both families, on the CPU."""
import json
import os
import subprocess
import sys

import numpy as np
import torch

from distributed_sse_for_llm_response_amd.engine.engine import LLMEngine
from distributed_sse_for_llm_response_amd.models import registry
from distributed_sse_for_llm_response_amd.models.mistral import TINY, init_standard_weights, reference_forward

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_force_step_on_the_dense_family_matches_its_reference():
    """Given tokens through the Mistral runner: a prompt portion, a mixed step (a single token beside another request's
    portion) and a decode-only step give the logits of the fp32 reference forward."""
    fam, cfg, _ = registry.resolve("mistral-tiny")
    assert cfg is TINY
    w = registry.load_weights(fam, cfg, None, device="cpu", seed=5)
    r = registry.make_runner(fam, w, num_blocks=16, max_batch=2, max_model_len=128, device="cpu", use_graphs=False)
    eng = LLMEngine(r, eos_id=-1)
    eng.watermark = 0
    g = torch.Generator().manual_seed(1)
    a = torch.randint(3, cfg.vocab_size, (21,), generator=g).tolist()
    b = torch.randint(3, cfg.vocab_size, (9,), generator=g).tolist()
    got_a = [eng.force_step([("a", a[:19], [0, 18])])]
    out = eng.force_step([("a", a[19:20], [0]), ("b", b, [8])])
    got_a.append(out[:1])
    got_b = out[1:]
    got_a.append(eng.force_step([("a", a[20:21], [0])], ["a", "b"]))
    std = init_standard_weights(cfg, seed=5)
    ref_a, _ = reference_forward(cfg, std, torch.tensor(a))
    ref_b, _ = reference_forward(cfg, std, torch.tensor(b))
    assert torch.allclose(torch.cat(got_a), ref_a[[0, 18, 19, 20]], atol=0.15, rtol=0.05)
    assert torch.allclose(got_b, ref_b[[8]], atol=0.15, rtol=0.05)
    assert eng.alloc.num_free == eng.alloc.num_blocks


def _run(args, lines):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), *args], input="\n".join(lines) + "\n",
                          capture_output=True, text=True, timeout=300)


def test_trace_run_command_line(tmp_path):
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": [5, 17, 3, 9], "want": [0, 3]}], "end": []},
        {"step": 1, "entries": [{"id": "x", "tokens": [11], "want": []}, {"id": "y", "tokens": [4, 4], "want": [1]}], "end": ["y"]},
        {"step": 2, "entries": [{"id": "x", "tokens": [2], "want": [0]}], "end": ["x"]},
    ]
    out = tmp_path / "out"
    res = _run(["--model", "muderax-tiny", "--dtype", "float32", "--out", str(out), "--max-tokens", "128", "--device", "cpu"],
               [json.dumps(s) for s in steps])
    assert res.returncode == 0, res.stderr[-2000:]
    assert [ln for ln in res.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    vocab = registry.resolve("muderax-tiny")[1].vocab_size
    shapes = {n: np.fromfile(out / f"{n}.f32", dtype="<f4").size // vocab for n in (0, 1, 2)}
    assert shapes == {0: 2, 1: 1, 2: 1}
    # the same tokens in one piece give the same logits
    whole = _run(["--model", "muderax-tiny", "--dtype", "float32", "--out", str(tmp_path / "w"), "--max-tokens", "128",
                  "--device", "cpu"],
                 [json.dumps({"step": 0, "entries": [{"id": "z", "tokens": [5, 17, 3, 9, 11, 2], "want": [0, 3, 5]}], "end": ["z"]})])
    assert whole.returncode == 0, whole.stderr[-2000:]
    w = np.fromfile(tmp_path / "w" / "0.f32", dtype="<f4").reshape(3, vocab)
    cut = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4"), np.fromfile(out / "2.f32", dtype="<f4")]).reshape(3, vocab)
    assert np.allclose(w, cut, atol=1e-4)


def test_trace_run_refuses_float32_without_32_bit_kernels(tmp_path):
    res = _run(["--model", "mistral-tiny", "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64",
                "--device", "cpu"], [])
    assert res.returncode == 3
