"""Trace replay: feed given token ids through a model step by step and write logits.

    dli trace-run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry brings a request's next tokens (a request is admitted at its first entry and may
skip steps); all entries of a step run as one batch through ``LLMEngine.replay_step`` — the
engine's scheduler builds the step, its block manager and state slots hold the pages and
states, its runner executes the model's step function. ``want`` are the places among an
entry's tokens whose logits are written to ``<out>/<step>.f32`` (little-endian fp32,
[wanted, vocab], entry order); ``end`` lists the requests that give their pages and state back
after the step. After every step ``done <step>`` is printed. Nothing is sampled.

The cache pool holds ``--max-tokens`` tokens (each live request rounded up to whole pages) and
there are ``--max-live`` state slots, so a long trace reuses pages and slots.

``--dtype float32`` runs weights, GEMM operands and caches in fp32 (exit code 3 if the model's
family has no fp32 kernels on this device).
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def main(argv=None) -> int:
    ap = argparse.ArgumentParser("dli trace-run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json + model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-live", type=int, default=4, help="state slots (live requests)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)

    import torch
    from ..models.hf import config_from_hf, load_hf_dir
    from .llm_engine import LLMEngine

    dev = a.device or ("cuda:0" if torch.cuda.is_available() else "cpu")
    dtype = torch.float32 if a.dtype == "float32" else torch.bfloat16
    with open(os.path.join(a.model, "config.json")) as f:
        cfg = config_from_hf(json.load(f))
    if dtype == torch.float32 and dev != "cpu" and not cfg.is_hybrid:
        print("float32 is not available for this model family on a GPU", file=sys.stderr)
        return 3
    cfg, params = load_hf_dir(a.model, device=dev, dtype=dtype)
    bs = a.block_size
    blocks = -(-a.max_tokens // bs) + a.max_live      # a partial page per live request
    eng = LLMEngine(cfg, device=dev, dtype=dtype, params=params, max_batch=a.max_live,
                    max_model_len=1 << 30, block_size=bs, num_blocks=blocks, use_graphs=False,
                    lookahead=False)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"]) for e in st["entries"]]
        want = [list(e.get("want") or []) for e in st["entries"]]
        logits = eng.replay_step(entries, want, st.get("end") or ())
        if logits.shape[0]:
            arr = logits.detach().float().cpu().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(arr).tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif dev != "cpu":
            torch.cuda.synchronize()
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
