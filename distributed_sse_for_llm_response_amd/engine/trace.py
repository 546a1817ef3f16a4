"""Trace replay: feed given token ids through the serving engine step by step and write the logits it computes.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Reads one JSON object per line from standard input,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

runs all entries of the step as ONE engine step (LLMEngine.force_step: portions of prompts as prompt chunks, single
next tokens in the decode rows, through the engine's slots, block allocator and kernels), writes the fp32 logits at the
wanted offsets to ``DIR/<step>.f32`` (little-endian, [wanted, vocab]) when any are wanted, and prints ``done <step>``.
Nothing is sampled.  ``--max-tokens`` sizes the cache pool (pages of 32 tokens); four sequences can be live at a time
(``--max-seqs``).  The model family is chosen from ``config.json`` by the registry; float32 is refused with exit code
3 by families that have no 32-bit kernels.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import torch


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="checkpoint directory (config.json + *.safetensors) or a config name")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--device", default=None, help="cuda (default when a GPU is present) or cpu")
    ap.add_argument("--seed", type=int, default=0, help="random weights when --model is a config name")
    a = ap.parse_args(argv)

    from ..models import registry
    from .engine import LLMEngine
    from .kv_cache import PAGE

    fam, cfg, path = registry.resolve(a.model)
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    if dtype not in fam.dtypes:
        print(f"trace_run: the {fam.name} family has no {a.dtype} kernels", file=sys.stderr)
        return 3
    dev = torch.device(a.device or ("cuda" if torch.cuda.is_available() else "cpu"))
    if dev.type == "cuda":
        from .. import ops

        ops.load_library(required=True)
        torch.backends.cuda.matmul.allow_tf32 = False
    w = registry.load_weights(fam, cfg, path, device=dev, dtype=dtype, seed=a.seed)
    blocks = -(-a.max_tokens // PAGE)
    runner = registry.make_runner(fam, w, num_blocks=blocks, max_batch=a.max_seqs, max_model_len=blocks * PAGE,
                                  max_prefill_tokens=blocks * PAGE, device=dev,
                                  use_graphs=dev.type == "cuda" and os.environ.get("DSSE_TRACE_GRAPHS", "1") != "0")
    if hasattr(runner, "capture") and runner.use_graphs and fam.name != "mistral":
        runner.capture()
    engine = LLMEngine(runner, eos_id=-1)
    engine.watermark = 0
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = engine.force_step([(e["id"], e["tokens"], e.get("want", [])) for e in st.get("entries", [])],
                                   st.get("end", []))
        if logits is not None:
            data = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif dev.type == "cuda":
            torch.cuda.synchronize(dev)
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
