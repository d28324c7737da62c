"""Trace replay: feed given token ids through a model step by step, dump logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step run as one batch through the engine's own step function
(engine.runner.ModelRunner.step: the model, cache and kernels that generation
uses); nothing is sampled.  For a step in which something is wanted the logits
at the wanted places are written to DIR/<step>.f32 as little-endian float32
[wanted, vocab], in the order of the entries and of `want`.  After each step a
line `done <step>` is printed and flushed.  Requests named in `end` give their
pages back after the step.  The cache pool holds --max-tokens tokens (in pages
of --page-size, default 16), so pages are used again.

The reference has no such tool; nearest are `--input-ids` (src/main.cpp:100-105)
and the interleaved engine test (tests/test_paged_generate_engine.cpp:428-552).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict


def parse_args(argv=None):
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__, formatter_class=argparse.RawTextHelpFormatter)
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens the live requests hold at any time (each rounded up to 64)")
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--max-requests", type=int, default=16, help="request slots")
    return p.parse_args(argv)


def replay(model, out_dir: str, max_tokens: int, page_size: int, max_requests: int, stdin, stdout) -> None:
    """Feed the steps on `stdin` through `model` (a bound models.decoder.DecoderLM): one
    ModelRunner.step per line, the wanted logits to `out_dir`, `done <step>` to `stdout`."""
    import numpy as np
    import torch

    from ..cache import CacheManager
    from ..engine import ModelRunner, StepEntry

    os.makedirs(out_dir, exist_ok=True)
    num_pages = (max_tokens + page_size - 1) // page_size
    cache = CacheManager(
        model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
        dtype=model.ctx.dtype, device=model.ctx.device,
    )
    runner = ModelRunner(model, cache)
    slots: Dict[str, int] = {}

    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = str(e["id"])
            if rid not in slots:
                slots[rid] = runner.admit()
            entries.append(StepEntry(slots[rid], list(e["tokens"]), list(e.get("want", []))))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid in slots:
                runner.release(slots.pop(rid))
        stdout.write(f"done {step}\n")
        stdout.flush()


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.max_tokens <= 0:
        raise SystemExit("--max-tokens must be greater than 0")
    if args.page_size <= 0:
        raise SystemExit("--page-size must be positive")

    from ..models import load_model

    model = load_model(args.model, args.dtype)
    replay(model, args.out, args.max_tokens, args.page_size, args.max_requests, sys.stdin, sys.stdout)
    return 0


if __name__ == "__main__":
    sys.exit(main())
