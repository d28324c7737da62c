"""The cache, the batch layout and the step function, exercised on the CPU with
plain torch forms of the kernels (tests/torch_ops.py) in place of the HIP ones,
against the plain whole-sequence implementation."""
import pytest
import torch

from litellmengine_amd.cache import CacheManager
from litellmengine_amd.engine import ModelRunner, StepEntry
from litellmengine_amd.models import load_model
from tests.plain import qwen3_plain as plain
from tests.tiny import CONFIGS, PAGE_SIZES, make_model_dir, random_tokens
from tests.torch_ops import TorchOps


def make_runner(model_dir, page_size, num_pages, max_requests=4, dtype=torch.float32):
    model = load_model(model_dir, dtype, device="cpu", ops=TorchOps())
    cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=dtype, device="cpu")
    return ModelRunner(model, cache)


def run_cut(runner, tokens, cuts):
    """Feed `tokens` in portions of the sizes in `cuts`; logits of every position."""
    slot = runner.admit()
    rows = []
    at = 0
    for c in cuts:
        part = tokens[at : at + c]
        rows.append(runner.step([StepEntry(slot, part, list(range(len(part))))]))
        at += c
    assert at == len(tokens)
    runner.release(slot)
    return torch.cat(rows)


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_cuts_match_plain(tmp_path, which):
    d = make_model_dir(tmp_path, which)
    cfg, w = plain.read_model_dir(d)
    tokens = random_tokens(45, cfg["vocab_size"], 7)
    want = plain.model_logits_fast(tokens, w, cfg)
    runner = make_runner(d, PAGE_SIZES[which], 16)
    for cuts in ([45], [13] + [1] * 32, [2, 7, 16, 3, 2, 15], [1] * 45):
        got = run_cut(runner, tokens, cuts)
        err = (got.double() - want).abs().max().item()
        assert err < 2e-5, (cuts, err)
    assert all(g.pool.num_held == 0 for g in runner.cache.groups)


def test_page_size_and_batch_order_do_not_matter(tmp_path):
    """The same three requests, stepped together in portions, with pages of 1, 4 and 16
    tokens and with the entries of every step in both orders: the same logits."""
    d = make_model_dir(tmp_path, "B")
    cfg, w = plain.read_model_dir(d)
    reqs = [random_tokens(n, cfg["vocab_size"], 60 + i) for i, n in enumerate((19, 7, 12))]
    want = [plain.model_logits_fast(t, w, cfg) for t in reqs]

    def run(page_size, reverse):
        runner = make_runner(d, page_size, 64 // page_size + 4)
        slots = [runner.admit() for _ in reqs]
        got = [[] for _ in reqs]
        at = [0] * len(reqs)
        for portion in (5, 1, 6, 1, 8):
            entries, who = [], []
            for i, t in enumerate(reqs):
                part = t[at[i] : at[i] + portion]
                if part:
                    entries.append(StepEntry(slots[i], part, list(range(len(part)))))
                    who.append(i)
                    at[i] += len(part)
            if reverse:
                entries, who = entries[::-1], who[::-1]
            rows = runner.step(entries)
            start = 0
            for e, i in zip(entries, who):
                got[i].append(rows[start : start + len(e.tokens)])
                start += len(e.tokens)
        for s in slots:
            runner.release(s)
        return [torch.cat(g) for g in got]

    base = run(4, False)
    for g, x in zip(base, want):
        assert (g.double() - x).abs().max().item() < 2e-5
    for page_size, reverse in ((1, False), (16, False), (4, True), (16, True)):
        for g, b in zip(run(page_size, reverse), base):
            assert (g - b).abs().max().item() < 1e-5, (page_size, reverse)


def test_a_cache_record_that_is_no_key_value_pair_on_the_cpu(monkeypatch):
    """The latent-vector mixer of tests/test_parts_gpu.py (a per-token cache record with one
    field, with and without a window) through the same cache manager and step function, with
    the substitute kernels."""
    import torch

    import tests.test_parts_gpu as parts_tests
    from litellmengine_amd.parts.base import BuildContext
    from tests.torch_ops import TorchOps

    monkeypatch.setattr(parts_tests, "make_context",
                        lambda dtype: BuildContext(dtype=dtype, device=torch.device("cpu"), ops=TorchOps()))
    parts_tests.test_a_cache_record_that_is_no_key_value_pair(torch.float32)


def test_every_group_has_a_page_size_and_a_pool_of_its_own(tmp_path):
    """Tiny C has layers with a window of 20 beside layers that see everything: two groups.
    The windowed group gets pages of 4 tokens and a pool sized by its window, the other pages
    of 16 and the whole capacity; the logits do not change, and a request four times as long
    as the windowed pool fits."""
    from litellmengine_amd.cache import GroupSizes
    from litellmengine_amd.engine import LLMEngine

    d = make_model_dir(tmp_path, "C")
    cfg, w = plain.read_model_dir(d)
    model = load_model(d, torch.float32, device="cpu", ops=TorchOps())
    specs = {m.cache_spec() for m in model.cache_layers().values()}
    windowed = next(s for s in specs if s.window is not None)
    cache = CacheManager(model, page_size=16, num_pages=12, max_requests=2, dtype=torch.float32, device="cpu",
                         max_tokens_per_step=9, group_sizes={windowed: GroupSizes(page_size=4)})
    by_window = {g.window: g for g in cache.groups}
    assert by_window[None].page_size == 16 and by_window[None].pool.num_pages == 12
    # 20 - 1 + 9 positions in pages of 4, wherever they start: 8 pages a request
    assert by_window[20].page_size == 4 and by_window[20].pool.num_pages == 2 * 8
    assert by_window[20].max_pages_per_request == 12 * 16 // 4  # the table still covers the longest request
    runner = ModelRunner(model, cache)
    tokens = random_tokens(150, cfg["vocab_size"], 17)
    want = plain.model_logits_fast(tokens, w, cfg)
    got = run_cut(runner, tokens, [9, 2, 7, 9, 1, 1, 8] + [9] * 12 + [5])
    assert (got.double() - want).abs().max().item() < 2e-5
    assert all(g.pool.num_held == 0 for g in cache.groups)

    # through the engine: the windowed pool is sized from the scheduler's budget
    engine = LLMEngine(model, page_size=8, num_pages=40, max_requests=3, max_tokens_per_step=12)
    sizes = {g.window: (g.page_size, g.pool.num_pages) for g in engine.cache.groups}
    assert sizes[None] == (8, 40) and sizes[20] == (8, 3 * (-(-(19 + 12) // 8) + 1))
    prompts = [random_tokens(n, cfg["vocab_size"], 80 + i) for i, n in enumerate((70, 33, 90))]
    out = engine.generate(prompts, 12)
    for p, o in zip(prompts, out):
        assert o == plain.generate_greedy(p, w, cfg, 12)
    assert engine.scheduler.num_preemptions == 0 and all(g.pool.num_held == 0 for g in engine.cache.groups)


def test_a_mixer_may_ask_for_its_own_page_size():
    from litellmengine_amd.parts.base import KVCacheSpec

    assert KVCacheSpec(2, 16, None, 32).page_size == 32
    assert KVCacheSpec(2, 16) != KVCacheSpec(2, 16, page_size=32)  # another page size: another group
    with pytest.raises(ValueError):
        KVCacheSpec(2, 16, page_size=0)


def test_a_step_that_fails_in_the_model_leaves_the_cache_as_it_was(tmp_path):
    """A kernel error in the second layer of a step (the first layer has written its K and V by
    then): pages, tables, lengths and what waits for the device table are what they were, and
    the same entries stepped again give the plain model's logits."""
    d = make_model_dir(tmp_path, "C")
    cfg, w = plain.read_model_dir(d)
    runner = make_runner(d, 4, 24)
    cache, ops = runner.cache, runner.model.ctx.ops
    a, b = random_tokens(30, cfg["vocab_size"], 3), random_tokens(11, cfg["vocab_size"], 4)
    sa, sb = runner.admit(), runner.admit()
    runner.step([StepEntry(sa, a[:13]), StepEntry(sb, b[:2])])

    def snapshot():
        return ([g.pool.num_free for g in cache.groups], [[g.tables[s] for s in (sa, sb)] for g in cache.groups],
                [cache.length(sa), cache.length(sb)], [g.native.lib.lle_pt_num_pending(g.native.handle) for g in cache.groups])

    before = snapshot()
    calls, real = [0], ops.paged_attention

    def failing(*args, **kw):
        calls[0] += 1
        if calls[0] == 2:
            raise RuntimeError("the kernel refuses its operands")
        return real(*args, **kw)

    ops.paged_attention = failing
    entries = [StepEntry(sa, a[13:30], list(range(17))), StepEntry(sb, b[2:11], list(range(9)))]
    with pytest.raises(RuntimeError, match="refuses"):
        runner.step(entries)
    ops.paged_attention = real
    assert snapshot() == before
    got = runner.step(entries)
    want = torch.cat([plain.model_logits_fast(a, w, cfg)[13:], plain.model_logits_fast(b, w, cfg)[2:]])
    assert (got.double() - want).abs().max().item() < 2e-5
    runner.release(sa)
    runner.release(sb)
    assert all(g.pool.num_held == 0 for g in cache.groups)
