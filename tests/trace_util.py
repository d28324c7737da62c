"""Builds traces for bin/trace_run and checks its dumps against the plain model."""
from __future__ import annotations

import io
import json
import os
import random
import subprocess
import sys
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from tests.plain import qwen3_plain as plain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def round64(n: int) -> int:
    return (n + 63) // 64 * 64


class TraceBuilder:
    """Collects steps; remembers which (request, position) every dumped row is."""

    def __init__(self):
        self.steps: List[dict] = []
        self.rows: Dict[int, List[Tuple[str, int]]] = {}
        self.fed: Dict[str, int] = {}
        self.live: Dict[str, int] = {}
        self.max_tokens = 0

    def step(self, entries: Sequence[Tuple[str, List[int], List[int]]], end: Sequence[str] = ()):
        n = len(self.steps)
        recs, rows = [], []
        for rid, tokens, want in entries:
            at = self.fed.get(rid, 0)
            recs.append({"id": rid, "tokens": list(tokens), "want": list(want)})
            rows += [(rid, at + w) for w in want]
            self.fed[rid] = at + len(tokens)
            self.live[rid] = self.fed[rid]
        self.max_tokens = max(self.max_tokens, sum(round64(v) for v in self.live.values()))
        for rid in end:
            self.live.pop(rid, None)
            self.fed.pop(rid, None)
        self.steps.append({"step": n, "entries": recs, "end": list(end)})
        if rows:
            self.rows[n] = rows

    def text(self) -> str:
        return "".join(json.dumps(s) + "\n" for s in self.steps)


def whole(tb: TraceBuilder, rid: str, tokens: List[int]):
    tb.step([(rid, tokens, list(range(len(tokens))))], end=[rid])


def tail_one_by_one(tb: TraceBuilder, rid: str, tokens: List[int], tail: int = 32):
    head = len(tokens) - tail
    tb.step([(rid, tokens[:head], list(range(head)))])
    for i in range(head, len(tokens)):
        tb.step([(rid, [tokens[i]], [0])], end=[rid] if i == len(tokens) - 1 else [])


def changing_portions(tb: TraceBuilder, rid: str, tokens: List[int], seed: int):
    rng = random.Random(seed)
    at = 0
    sizes = [2, 17, 3, 2, 31, 5]
    while at < len(tokens):
        n = sizes.pop(0) if sizes else rng.choice([2, 2, 3, 7, 16, 29])
        n = min(n, len(tokens) - at)
        if len(tokens) - at - n == 1:  # never leave a single token for a "portion"
            n += 1
        tb.step([(rid, tokens[at : at + n], list(range(n)))], end=[rid] if at + n == len(tokens) else [])
        at += n


def mixed(tb: TraceBuilder, requests: Dict[str, List[int]], seed: int, max_live: int = 4):
    """Up to `max_live` requests at a time; each step some get a portion of
    their prompt, those past two thirds get single tokens, some sit a step out."""
    rng = random.Random(seed)
    todo = list(requests.items())
    live: Dict[str, int] = {}
    while todo or live:
        while todo and len(live) < max_live:
            rid, _ = todo.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            tokens = requests[rid]
            at = live[rid]
            if rng.random() < 0.2 and len(live) > 1:
                continue  # left out of this step, goes on later
            left = len(tokens) - at
            if at >= 2 * len(tokens) // 3:
                n = 1
            else:
                n = min(left, rng.choice([2, 3, 5, 8, 13, 21]))
            want = sorted(set(rng.sample(range(n), min(n, 3))) | {n - 1})
            entries.append((rid, tokens[at : at + n], want))
            live[rid] = at + n
            if live[rid] == len(tokens):
                end.append(rid)
                del live[rid]
        if entries:
            tb.step(entries, end)


def run_tool(model_dir: str, dtype: str, out_dir: str, trace: TraceBuilder, max_tokens: int = None,
             page_size: int = None, in_process_ops=None) -> None:
    """Run bin/trace_run over the trace (as a child process, as a user would;
    `in_process_ops` runs its main() here on the CPU with substitute kernels)."""
    max_tokens = max_tokens or trace.max_tokens
    if in_process_ops is not None:
        # the tool's own loop over the steps, with a model loaded here for the CPU stand-in kernels
        from litellmengine_amd.entrypoints.trace_run import replay
        from litellmengine_amd.models import load_model

        out = io.StringIO()
        model = load_model(model_dir, dtype, device="cpu", ops=in_process_ops)
        replay(model, out_dir, max_tokens, page_size or 16, 16, io.StringIO(trace.text()), out)
        done = out.getvalue().split("\n")
    else:
        argv = ["--model", model_dir, "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)]
        if page_size:
            argv += ["--page-size", str(page_size)]
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run")] + argv, input=trace.text(),
                              text=True, capture_output=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-3000:]
        done = proc.stdout.split("\n")
    assert [l for l in done if l] == [f"done {i}" for i in range(len(trace.steps))]


def check_dumps(out_dir: str, trace: TraceBuilder, expected: Dict[str, torch.Tensor], tol: float) -> float:
    """Every dumped row against the plain model's logits of that request and position."""
    worst = 0.0
    files = {f for f in os.listdir(out_dir) if f.endswith(".f32")}
    assert files == {f"{n}.f32" for n in trace.rows}, "a dump file for exactly the steps that want something"
    for n, rows in trace.rows.items():
        vocab = next(iter(expected.values())).shape[1]
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{n}.f32"), dtype="<f4").reshape(len(rows), vocab))
        for i, (rid, pos) in enumerate(rows):
            rid0 = rid.split("#")[0]
            want = expected[rid0][pos]
            err = (got[i].double() - want).abs().max().item() / max(1.0, want.abs().max().item())
            assert err < tol, f"step {n}, request {rid}, position {pos}: error {err:.3g} (first wrong row of the step: {i})"
            worst = max(worst, err)
    return worst


def plain_logits(model_dir: str, requests: Dict[str, List[int]]) -> Dict[str, torch.Tensor]:
    cfg, w = plain.read_model_dir(model_dir)
    return {rid: plain.model_logits_fast(tokens, w, cfg) for rid, tokens in requests.items()}
