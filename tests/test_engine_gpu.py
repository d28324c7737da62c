"""The engine on the GPU against the plain implementation: whole prompts, the
last tokens one by one, portions of changing size; float32 and bfloat16."""
import pytest
import torch

from litellmengine_amd.cache import CacheManager
from litellmengine_amd.engine import ModelRunner, StepEntry
from litellmengine_amd.models import load_model
from tests.plain import qwen3_plain as plain
from tests.tiny import PAGE_SIZES, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu

# about five times the worst error seen over dozens of seeds (float32 7e-7, bfloat16 7e-3 at these sizes)
TOL = {"float32": 4e-6, "bfloat16": 2e-2}


def make_runner(model_dir, dtype, page_size, num_pages, max_requests=4):
    model = load_model(model_dir, dtype)
    cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=model.ctx.dtype, device=model.ctx.device)
    return ModelRunner(model, cache)


def run_cut(runner, tokens, cuts):
    slot = runner.admit()
    rows, at = [], 0
    for c in cuts:
        part = tokens[at : at + c]
        rows.append(runner.step([StepEntry(slot, part, list(range(len(part))))]).cpu())
        at += c
    runner.release(slot)
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C", "D"])
def test_cuts_match_plain(tmp_path, which, dtype):
    d = make_model_dir(tmp_path, which, dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    tokens = random_tokens(77, cfg["vocab_size"], 7)
    want = plain.model_logits_fast(tokens, w, cfg)
    runner = make_runner(d, dtype, PAGE_SIZES[which], 80 // PAGE_SIZES[which] + 1)
    for cuts in ([77], [45] + [1] * 32, [2, 7, 16, 3, 2, 15, 30, 2]):
        got = run_cut(runner, tokens, cuts)
        err = (got.double() - want).abs().max().item()
        assert err < TOL[dtype], (cuts, err)
    assert all(g.pool.num_held == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(tmp_path, dtype):
    """Decode steps through a captured graph, replayed many times with eager work
    (prompt portions of other requests, table updates) between the replays, against
    the same steps run without graphs."""
    d = make_model_dir(tmp_path, "B", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    seqs = [random_tokens(n, cfg["vocab_size"], 50 + i) for i, n in enumerate((61, 50, 80))]
    outs = {}
    for use_graphs in (True, False):
        model = load_model(d, dtype)
        cache = CacheManager(model, page_size=16, num_pages=40, max_requests=4, dtype=model.ctx.dtype,
                             device=model.ctx.device)
        runner = ModelRunner(model, cache, use_graphs=use_graphs)
        assert runner.use_graphs == use_graphs
        slots = [runner.admit() for _ in seqs]
        got = []
        runner.step([StepEntry(slots[0], seqs[0][:20]), StepEntry(slots[1], seqs[1][:9])])
        at = [20, 9, 0]
        for it in range(31):
            entries = [StepEntry(slots[i], [seqs[i][at[i]]], [0]) for i in (0, 1)]
            got.append(runner.step(entries).cpu())  # a decode step of two requests
            at[0] += 1
            at[1] += 1
            if it % 3 == 0 and at[2] < 70:  # eager work between the replays
                runner.step([StepEntry(slots[2], seqs[2][at[2] : at[2] + 7])])
                at[2] += 7
            if it == 20:  # three decoding rows: another graph
                got.append(runner.step([StepEntry(slots[i], [seqs[i][at[i]]], [0]) for i in (0, 1, 2)]).cpu())
                at = [a + 1 for a in at]
        if use_graphs:
            assert len(runner._graphs) >= 2
        outs[use_graphs] = torch.cat(got)
    assert (outs[True] - outs[False]).abs().max() < TOL[dtype] / 4
    want = plain.model_logits_fast(seqs[0], w, cfg)
    assert (outs[True][0].double() - want[20]).abs().max() < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("split_from", [None, 4], ids=["", "keys split early"])
def test_long_decoding_and_first_tokens(tmp_path, dtype, split_from):
    """A short prompt, then hundreds of tokens one by one (several pages, several
    context buckets of the decode graphs); the very first positions of a sequence
    (position 0 sees itself only) are checked on their own.  Once more with the keys of a
    decode step split between workgroups from 128 keys on (contexts this short are not split
    otherwise), so that the split count changes several times along the way."""
    d = make_model_dir(tmp_path, "B", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    tokens = random_tokens(600, cfg["vocab_size"], 77)
    want = plain.model_logits_fast(tokens, w, cfg)
    runner = make_runner(d, dtype, 16, 40)
    if split_from:
        runner.model.ctx.ops.DECODE_MIN_STEPS_TO_SPLIT = split_from
        runner.model.ctx.ops.DECODE_MIN_STEPS_PER_SPLIT = 2
    try:
        _long_decoding(runner, tokens, want, dtype)
    finally:
        for name in ("DECODE_MIN_STEPS_TO_SPLIT", "DECODE_MIN_STEPS_PER_SPLIT"):
            runner.model.ctx.ops.__dict__.pop(name, None)


def _long_decoding(runner, tokens, want, dtype):
    slot = runner.admit()
    first = runner.step([StepEntry(slot, tokens[:1], [0])]).cpu()
    assert (first.double() - want[:1]).abs().max() < TOL[dtype]
    second = runner.step([StepEntry(slot, tokens[1:3], [0, 1])]).cpu()
    assert (second.double() - want[1:3]).abs().max() < TOL[dtype]
    worst = 0.0
    for i in range(3, 600):
        got = runner.step([StepEntry(slot, [tokens[i]], [0])], borrow=True)
        if i % 7 == 0 or i > 590:
            worst = max(worst, (got.cpu().double() - want[i : i + 1]).abs().max().item())
    assert worst < TOL[dtype], worst
    runner.release(slot)


def test_qwen3_8b_layer_sizes(tmp_path):
    """Two layers at the Qwen3-8B layer sizes (hidden 4096, 32/8 heads of 128, feed-forward
    12288, vocabulary 151936): float32 against the plain implementation in three cuttings,
    bfloat16 against the same."""
    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.weights import write_model_dir

    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936, rope_theta=1e6,
        rms_norm_eps=1e-6, tie_word_embeddings=False))
    d = str(tmp_path / "m8b")
    write_model_dir(cfg, d, 3, torch.bfloat16)
    pcfg, w = plain.read_model_dir(d, dtype=torch.float32)
    tokens = random_tokens(120, cfg.vocab_size, 5)
    want = plain.model_logits_fast(tokens, w, pcfg).double()
    scale = max(1.0, want.abs().max().item())
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 4e-2)):  # the oracle itself is float32 here
        runner = make_runner(d, dtype, 16, 8)
        # (120, 88 and 68 rows: o_proj and down_proj in slices of K with eight, six and six tiles of rows)
        for cuts in ([120], [88] + [1] * 32, [2, 17, 3, 30, 68]):
            got = run_cut(runner, tokens, cuts)
            err = (got.double() - want).abs().max().item() / scale
            assert err < tol, (dtype, cuts, err)
        del runner
        torch.cuda.empty_cache()


def test_graph_replays_with_library_products(tmp_path):
    """Decode steps of 24 requests at the Qwen3-8B layer widths: more rows than the
    weight-streaming kernel takes, so the captured graph holds library matrix products.
    Every replay is compared with the same step run without a graph, and the rows of some
    requests with the plain implementation's logits for their whole history."""
    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.weights import write_model_dir

    cfg = Qwen3Config.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], num_hidden_layers=2, hidden_size=4096, num_attention_heads=32,
        num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=32000, rope_theta=1e6,
        rms_norm_eps=1e-6, tie_word_embeddings=True))
    d = str(tmp_path / "m24")
    write_model_dir(cfg, d, 5, torch.bfloat16)
    model = load_model(d, "bfloat16")
    B = 24
    prompts = [random_tokens(30 + 3 * i, cfg.vocab_size, 200 + i) for i in range(B)]
    feed = [random_tokens(8, cfg.vocab_size, 300 + i) for i in range(B)]
    outs = {}
    for use_graphs in (True, False):
        cache = CacheManager(model, page_size=16, num_pages=B * 8, max_requests=B, dtype=model.ctx.dtype,
                             device=model.ctx.device)
        runner = ModelRunner(model, cache, use_graphs=use_graphs)
        slots = [runner.admit() for _ in range(B)]
        runner.step([StepEntry(s, p) for s, p in zip(slots, prompts)])
        got = []
        for t in range(8):
            got.append(runner.step([StepEntry(s, [feed[i][t]], [0]) for i, s in enumerate(slots)]).float().cpu())
            if t == 3:  # eager work between replays
                extra = runner.admit() if cache.num_free_slots else None
        outs[use_graphs] = torch.stack(got)  # [step, request, vocabulary]
    diff = (outs[True] - outs[False]).abs().max().item()
    assert diff < 2e-2, diff
    pcfg, w = plain.read_model_dir(d, dtype=torch.float32)
    for i in (0, 11, 23):
        want = plain.model_logits_fast(prompts[i] + feed[i], w, pcfg)[len(prompts[i]):].double()
        err = (outs[True][:, i].double() - want).abs().max().item() / max(1.0, want.abs().max().item())
        assert err < 4e-2, (i, err)


ODD = [
    # head size 80 (no matrix-core attention), width not a multiple of 4, odd vocabulary, page size 3
    dict(num_hidden_layers=2, hidden_size=102, num_attention_heads=5, num_key_value_heads=5, head_dim=80,
         intermediate_size=150, vocab_size=1001, rope_theta=3e4, rms_norm_eps=2e-6, tie_word_embeddings=True, page=3),
    # one kv head for seven q heads, head size 64, page size 32, widths that are multiples of 2 only
    dict(num_hidden_layers=1, hidden_size=70, num_attention_heads=7, num_key_value_heads=1, head_dim=64,
         intermediate_size=94, vocab_size=333, rope_theta=1e6, rms_norm_eps=1e-5, tie_word_embeddings=False, page=32),
    # head size 256, a window of 9 on every layer, page size 1; a width that the products around a folded
    # norm take and a feed-forward width that they do not (a multiple of 4 only)
    dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=2, num_key_value_heads=2, head_dim=256,
         intermediate_size=76, vocab_size=50, rope_theta=1e4, rms_norm_eps=1e-6, tie_word_embeddings=False,
         sliding_window=9, layer_types=["sliding_attention", "sliding_attention"], page=1),
    # head size 96 (matrix cores, three 32-element steps), group of 3, page size 48
    dict(num_hidden_layers=2, hidden_size=96, num_attention_heads=6, num_key_value_heads=2, head_dim=96,
         intermediate_size=136, vocab_size=257, rope_theta=5e5, rms_norm_eps=1e-6, tie_word_embeddings=True, page=48),
    # a group of 16: one decoded token fills the 16-row tile of the decode kernels exactly; heads of 128
    dict(num_hidden_layers=2, hidden_size=72, num_attention_heads=32, num_key_value_heads=2, head_dim=128,
         intermediate_size=104, vocab_size=211, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, page=16),
    # a group of 32 on one kv head: a decoded token has more rows than a tile, so it goes the prompt kernels' way
    dict(num_hidden_layers=2, hidden_size=88, num_attention_heads=32, num_key_value_heads=1, head_dim=64,
         intermediate_size=120, vocab_size=197, rope_theta=2e5, rms_norm_eps=1e-5, tie_word_embeddings=True, page=16),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("index", range(len(ODD)))
def test_odd_sizes(tmp_path, index, dtype):
    """Sizes that push the kernels off their fast paths (or onto rarely used ones)."""
    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.weights import write_model_dir

    spec = dict(ODD[index])
    page = spec.pop("page")
    cfg = Qwen3Config.from_dict(dict(spec, architectures=["Qwen3ForCausalLM"]))
    d = str(tmp_path / f"odd{index}")
    write_model_dir(cfg, d, 21 + index, torch.bfloat16)
    pcfg, w = plain.read_model_dir(d)
    tokens = random_tokens(50, cfg.vocab_size, 9)
    want = plain.model_logits_fast(tokens, w, pcfg)
    runner = make_runner(d, dtype, page, 64 // page + 2)
    for cuts in ([50], [18] + [1] * 32, [2, 9, 20, 2, 17]):
        got = run_cut(runner, tokens, cuts)
        err = (got.double() - want).abs().max().item() / max(1.0, want.abs().max().item())
        assert err < TOL[dtype], (cuts, err)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_kernel_error_in_the_middle_of_a_step_leaves_the_cache_consistent(tmp_path, dtype):
    """The attention of the second layer refuses to launch (a KernelError, forced from the host)
    after the first layer has written its keys and values: pages, tables and lengths are what
    they were before the step, and the same entries stepped again match the plain model."""
    from litellmengine_amd.csrc.ops import KernelError

    d = make_model_dir(tmp_path, "B", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    runner = make_runner(d, dtype, 8, 12)
    cache, ops = runner.cache, runner.model.ctx.ops
    a, b = random_tokens(40, cfg["vocab_size"], 3), random_tokens(19, cfg["vocab_size"], 4)
    sa, sb = runner.admit(), runner.admit()
    runner.step([StepEntry(sa, a[:21]), StepEntry(sb, b[:3])])
    snapshot = lambda: ([g.pool.num_free for g in cache.groups], [[g.tables[s] for s in (sa, sb)] for g in cache.groups],
                        [cache.length(sa), cache.length(sb)])
    before = snapshot()
    calls, real = [0], ops.paged_attention

    def failing(*args, **kw):
        calls[0] += 1
        if calls[0] == 2:
            raise KernelError("lle_paged_attention_mfma failed to launch: forced by the test")
        return real(*args, **kw)

    ops.paged_attention = failing
    entries = [StepEntry(sa, a[21:40], list(range(19))), StepEntry(sb, b[3:19], list(range(16)))]
    try:
        with pytest.raises(KernelError):
            runner.step(entries)
    finally:
        del ops.paged_attention  # the instance attribute: the class's method is back
    assert calls[0] == 2 and snapshot() == before
    got = runner.step(entries).cpu()
    want = torch.cat([plain.model_logits_fast(a, w, cfg)[21:], plain.model_logits_fast(b, w, cfg)[3:]])
    assert (got.double() - want).abs().max().item() < TOL[dtype]
    runner.release(sa)
    runner.release(sb)
    assert all(g.pool.num_held == 0 for g in cache.groups)
