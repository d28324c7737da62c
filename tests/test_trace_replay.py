"""bin/trace_run replays the same requests whole, with the last 32 tokens one by
one, in portions of changing size, and mixed with other requests in a pool so
small that pages are used again; every dumped row is compared with the plain
implementation.  The GPU tests run the tool as a child process in float32 and
bfloat16; the CPU test runs its main() with substitute kernels."""
import pytest
import torch

from tests.tiny import CONFIGS, PAGE_SIZES, make_model_dir, random_tokens, sharpen_attention
from tests.torch_ops import TorchOps
from tests.trace_util import (TraceBuilder, changing_portions, check_dumps, mixed, plain_logits, run_tool,
                              tail_one_by_one, whole)

LENGTHS = {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 90}
# about five times the worst error seen over dozens of seeds (float32 7e-7, bfloat16 7e-3 at these sizes)
TOL = {"float32": 4e-6, "bfloat16": 2e-2}


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
@pytest.mark.parametrize("which", ["A", "A/default page", "B", "C", "D"])
def test_trace_gpu(tmp_path, which, dtype):
    which, default_page = which[0], len(which) > 1
    d = make_model_dir(tmp_path, which, dtype=torch.bfloat16)
    requests = make_requests(CONFIGS[which]["vocab_size"], seed=10)
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, dtype, out, tb, page_size=None if default_page else PAGE_SIZES[which])
    worst = check_dumps(out, tb, plain_logits(d, requests), TOL[dtype])
    print(f"trace {which} {dtype}: worst relative error {worst:.3g}, pool {tb.max_tokens} tokens")


def peaked_trace(vocab):
    """Long requests (a far key among hundreds) in every way of cutting, few pages."""
    requests = {"p": random_tokens(300, vocab, 41), "q": random_tokens(170, vocab, 42),
                "r": random_tokens(230, vocab, 43), "s": random_tokens(90, vocab, 44)}
    tb = TraceBuilder()
    whole(tb, "p#whole", requests["p"])
    tail_one_by_one(tb, "p#tail", requests["p"])
    changing_portions(tb, "r#cut", requests["r"], seed=3)
    mixed(tb, {rid + "#mix": t for rid, t in requests.items()}, seed=6)
    return requests, tb


# Larger scores carry the rounding of q and k further into the softmax weights: with the
# factors below, a float32 run of plain torch on the CPU (tests/torch_ops.py, no code shared
# with the kernels) is up to 5e-5 from the float64 model, a bfloat16 run up to 5e-2.  One key
# lost at a window's edge moves the logits of these models by 0.35 (median over positions).
PEAK = {"float32": (3.0, 1e-4), "bfloat16": (2.0, 1e-1)}


def attention_is_peaked(model_dir, tokens, share):
    """The plain model's first layer gives one key more than half of the weight for
    at least `share` of the queries past the first few: the sharpening did what it is for."""
    from tests.plain import qwen3_plain as plain

    cfg, w = plain.read_model_dir(model_dir)
    probs = plain.first_layer_attention_probs(tokens, w, cfg)  # [heads, T, T]
    top = probs[:, 32:, :].max(dim=-1).values
    return (top > 0.5).double().mean().item() > share


def test_peaked_attention_trace_cpu(tmp_path):
    d = make_model_dir(tmp_path, "C")
    factor, tol = PEAK["float32"]
    sharpen_attention(d, factor)
    requests, tb = peaked_trace(CONFIGS["C"]["vocab_size"])
    assert attention_is_peaked(d, requests["p"], 0.8)
    out = str(tmp_path / "out")
    run_tool(d, "float32", out, tb, in_process_ops=TorchOps())
    check_dumps(out, tb, plain_logits(d, requests), tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["B", "C", "D"])
def test_peaked_attention_trace_gpu(tmp_path, which, dtype):
    d = make_model_dir(tmp_path, which, dtype=torch.bfloat16)
    factor, tol = PEAK[dtype]
    sharpen_attention(d, factor)
    requests, tb = peaked_trace(CONFIGS[which]["vocab_size"])
    assert attention_is_peaked(d, requests["p"], 0.35)
    out = str(tmp_path / "out")
    run_tool(d, dtype, out, tb, page_size=PAGE_SIZES[which])
    worst = check_dumps(out, tb, plain_logits(d, requests), tol)
    print(f"peaked trace {which} {dtype}: worst relative error {worst:.3g}, pool {tb.max_tokens} tokens")


# -- two layers at the Qwen3-8B layer sizes: the kernels that the benchmark runs ------------------
QWEN3_8B_LAYERS = dict(
    architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6,
    rms_norm_eps=1e-6, tie_word_embeddings=False)
# float32: the oracle is a float32 run of the plain model here (float64 would not fit the time)
TOL_8B = {"float32": 2e-5, "bfloat16": 4e-2}
PEAK_8B = {"float32": (2.0, 4e-5), "bfloat16": (2.0, 1e-1)}


@pytest.fixture(scope="module")
def model_dirs_8b(tmp_path_factory):
    """The model folder and its sharpened twin, written once for all tests of this module,
    with the plain model's logits of the requests that the traces below replay."""
    import os
    import shutil

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.weights import write_model_dir
    from tests.plain import qwen3_plain as plain

    root = tmp_path_factory.mktemp("m8b")
    cfg = Qwen3Config.from_dict(QWEN3_8B_LAYERS)
    made = {}

    def get(sharp: bool):
        if sharp not in made:
            d = str(root / ("sharp" if sharp else "base"))
            write_model_dir(cfg, d, 3, torch.bfloat16)
            if sharp:
                sharpen_attention(d, PEAK_8B["float32"][0])
            requests = make_requests(cfg.vocab_size, seed=20)
            pcfg, w = plain.read_model_dir(d, dtype=torch.float32)
            want = {rid: plain.model_logits_fast(t, w, pcfg).double() for rid, t in requests.items()}
            peaked = attention_is_peaked(d, requests["c"], 0.35) if sharp else None
            made[sharp] = (d, requests, want, peaked)
        return made[sharp]

    yield get
    shutil.rmtree(str(root), ignore_errors=True)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sharp", [False, True], ids=["random", "sharpened"])
def test_trace_qwen3_8b_layer_sizes_mixed(tmp_path, model_dirs_8b, sharp, dtype):
    """Heads of 128, page size 16, the widths of the 8B model: prompt portions beside single
    tokens of up to four live requests, in a pool of the live peak so that pages are used
    again (tests/test_paged_generate_engine.cpp:428-552 interleaves requests in this way)."""
    d, requests, want, peaked = model_dirs_8b(sharp)
    assert peaked is not False, "the sharpening was meant to make single keys carry the softmax"
    tb = TraceBuilder()
    mixed(tb, {rid + "#mix": t for rid, t in requests.items()}, seed=5)
    tail_one_by_one(tb, "a#tail", requests["a"])
    out = str(tmp_path / "out")
    run_tool(d, dtype, out, tb, page_size=16)
    tol = PEAK_8B[dtype][1] if sharp else TOL_8B[dtype]
    worst = check_dumps(out, tb, want, tol)
    print(f"8B-size mixed trace {dtype} sharp={sharp}: worst relative error {worst:.3g}, pool {tb.max_tokens} tokens")


class SomeRows:
    """The plain model's logits at some positions of a request, indexed by position
    (what check_dumps asks of the expected logits of a request)."""

    def __init__(self, positions, logits):
        self.at = {int(p): i for i, p in enumerate(positions)}
        self.logits = logits
        self.shape = (max(self.at) + 1, logits.shape[1])

    def __getitem__(self, pos):
        return self.logits[self.at[int(pos)]]


_long_oracle = {}


def long_trace_oracle(d, long_ids, short_ids, wanted):
    """The plain model in float64 at the wanted positions (the head runs on those rows only);
    made once for both dtypes.  The rotation angles are the reference's float32 products: at
    position 4055 the exact angle differs from them by up to 2.4e-4 radians, which moves these
    logits by 4e-5 of their size, twice the tolerance of the float32 run."""
    from tests.plain import qwen3_plain as plain

    if d not in _long_oracle:
        pcfg, w = plain.read_model_dir(d, dtype=torch.float64)
        _long_oracle[d] = {rid: SomeRows(wanted[rid], plain.model_logits_fast(ids, w, pcfg, rows=wanted[rid], float32_angles=True))
                           for rid, ids in (("long", long_ids), ("short", short_ids))}
    return _long_oracle[d]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_qwen3_8b_layer_sizes_across_4096(tmp_path, model_dirs_8b, dtype):
    """A request of 4200 tokens at the 8B layer sizes: most of it in two portions, then token by
    token from position 4056 to the end, across the context of 4096 at which the benchmark runs
    (sixteen key splits at batch 1) and across the table's 256th page; a short request decodes
    beside it for a while (another batch bucket), and is ended so that its pages are used again."""
    d, requests, _, _ = model_dirs_8b(False)
    vocab = QWEN3_8B_LAYERS["vocab_size"]
    long_ids, short_ids = random_tokens(4200, vocab, 31), random_tokens(120, vocab, 32)
    head = 4056
    tb = TraceBuilder()
    tb.step([("long", long_ids[:2048], [0, 2047])])
    tb.step([("long", long_ids[2048:head], [0, head - 2049]), ("short", short_ids[:70], [69])])
    for i in range(head, len(long_ids)):
        entries = [("long", [long_ids[i]], [0])]
        j = 70 + (i - head)
        if j < len(short_ids):
            entries.append(("short", [short_ids[j]], [0]))
        last_short = j == len(short_ids) - 1
        tb.step(entries, end=(["short"] if last_short else []) + (["long"] if i == len(long_ids) - 1 else []))
    wanted = {"long": sorted({pos for rows in tb.rows.values() for rid, pos in rows if rid == "long"}),
              "short": sorted({pos for rows in tb.rows.values() for rid, pos in rows if rid == "short"})}
    want = long_trace_oracle(d, long_ids, short_ids, wanted)
    out = str(tmp_path / "out")
    run_tool(d, dtype, out, tb, page_size=16)
    worst = check_dumps(out, tb, want, TOL_8B[dtype])
    print(f"8B-size trace across 4096 {dtype}: worst relative error {worst:.3g}, pool {tb.max_tokens} tokens")
