"""bin/trace_run replays the same requests whole, with the last 32 tokens one by
one, in portions of changing size, and mixed with other requests in a pool so
small that pages are used again; every dumped row is compared with the plain
implementation.  The GPU tests run the tool as a child process in float32 and
bfloat16; the CPU test runs its main() with substitute kernels."""
import pytest
import torch

from tests.tiny import CONFIGS, PAGE_SIZES, make_model_dir, random_tokens
from tests.torch_ops import TorchOps
from tests.trace_util import (TraceBuilder, changing_portions, check_dumps, mixed, plain_logits, run_tool,
                              tail_one_by_one, whole)

LENGTHS = {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 90}
TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def make_requests(vocab, seed=0):
    return {rid: random_tokens(n, vocab, seed + i) for i, (rid, n) in enumerate(LENGTHS.items())}


def all_ways_trace(requests):
    tb = TraceBuilder()
    for rid in ("a", "c"):
        whole(tb, rid + "#whole", requests[rid])
    for rid in ("a", "e"):
        tail_one_by_one(tb, rid + "#tail", requests[rid])
    for i, rid in enumerate(("c", "f")):
        changing_portions(tb, rid + "#cut", requests[rid], seed=i)
    mixed(tb, {rid + "#mix": t for rid, t in requests.items()}, seed=5)
    return tb


def test_trace_cpu(tmp_path):
    d = make_model_dir(tmp_path, "C")
    requests = make_requests(CONFIGS["C"]["vocab_size"])
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, "float32", out, tb, in_process_ops=TorchOps())
    check_dumps(out, tb, plain_logits(d, requests), 2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_trace_gpu(tmp_path, which, dtype):
    d = make_model_dir(tmp_path, which, dtype=torch.bfloat16)
    requests = make_requests(CONFIGS[which]["vocab_size"], seed=10)
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, dtype, out, tb, page_size=PAGE_SIZES[which] if which != "A" else None)
    worst = check_dumps(out, tb, plain_logits(d, requests), TOL[dtype])
    print(f"trace {which} {dtype}: worst relative error {worst:.3g}, pool {tb.max_tokens} tokens")
