"""Generation through the engine (scheduler + step + sampler): on the CPU with
substitute kernels, and on the GPU through the entry point."""
import pytest
import torch

from litellmengine_amd.engine import LLMEngine
from litellmengine_amd.models import load_model
from tests.plain import qwen3_plain as plain
from tests.tiny import CONFIGS, make_model_dir, random_tokens
from tests.torch_ops import TorchOps


RUN_AHEAD = False


@pytest.fixture(autouse=True, params=[False, True], ids=["step by step", "steps launched ahead"])
def both_ways_of_stepping(request):
    """Every test of this file runs twice: with each step's tokens read before the next step is
    laid out, and with decode steps launched ahead of that reading (the device feeds a
    request's pick to its next step; the host learns of an end-of-sequence token a step late)."""
    global RUN_AHEAD
    RUN_AHEAD = request.param
    yield
    RUN_AHEAD = False


def cpu_engine(d, **kw):
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    kw.setdefault("run_ahead", RUN_AHEAD)
    return LLMEngine(model, **kw)


@pytest.mark.parametrize("which,page_size", [("A", 4), ("C", 16)])
def test_greedy_generation_equals_full_recompute(tmp_path, which, page_size):
    """Workload of the tiny configuration A: prompts 5/9/17, 8 greedy steps, page size 4.  (With
    tied embeddings and random weights A mostly repeats a prompt's last token; C, with an output
    head of its own, goes through different tokens.)"""
    d = make_model_dir(tmp_path, which)
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, 256, i) for i, n in enumerate((5, 9, 17))]
    want = [plain.generate_greedy(p, w, cfg, 8) for p in prompts]
    if which == "C":
        assert len(set(sum(want, []))) >= 6
    eng = cpu_engine(d, page_size=page_size, num_pages=24, max_requests=3)
    assert eng.generate(prompts, 8) == want
    # each alone == among the others (tests/test_paged_generate_engine.cpp:428-552)
    for p, x in zip(prompts, want):
        assert cpu_engine(d, page_size=page_size, num_pages=24, max_requests=1).generate([p], 8) == [x]


def test_chunked_prefill_and_preemption_do_not_change_tokens(tmp_path):
    """Tiny configuration B: prompts 1/7/23/40, page size 8, prefill chunk 16; then
    the same with a pool so small that requests are preempted and recomputed."""
    d = make_model_dir(tmp_path, "B")
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, 503, 10 + i) for i, n in enumerate((1, 7, 23, 40))]
    want = [plain.generate_greedy(p, w, cfg, 6) for p in prompts]
    eng = cpu_engine(d, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16, max_tokens_per_step=24)
    assert eng.generate(prompts, 6) == want
    small = cpu_engine(d, page_size=8, num_pages=8, max_requests=4, prefill_chunk=16, max_tokens_per_step=24)
    assert small.generate(prompts, 6) == want
    assert all(g.pool.num_held == 0 for g in small.cache.groups)


def test_session_continues_from_its_cache_and_is_released(tmp_path):
    """Two turns as in tests/test_paged_generate_engine.cpp:555-663: the second turn keeps the
    history, counts its own new tokens only, runs only the new tokens, and generates what a
    fresh request over the whole history generates."""
    d = make_model_dir(tmp_path, "B")
    cfg, w = plain.read_model_dir(d)
    first, second = random_tokens(11, 503, 31), random_tokens(5, 503, 32)
    gen1 = plain.generate_greedy(first, w, cfg, 4)
    gen2 = plain.generate_greedy(first + gen1 + second, w, cfg, 3)
    eng = cpu_engine(d, page_size=8, num_pages=8, max_requests=2, prefill_chunk=4)
    r = eng.add_request(first, 4, keep_session=True)
    eng.run_until_finished()
    assert r.finished and r.generated == gen1 and r.slot >= 0
    held = eng.cache.groups[0].pool.num_held
    assert held > 0 and r.cached_len == len(first) + 3  # the last token drawn is not cached yet
    eng.append_input_tokens(r, second, 3)
    assert not r.finished and r.generated == [] and r.prompt_len == len(first) + 4 + len(second)
    assert r.cached_len == len(first) + 3 and r.extend_len == len(second) + 1
    steps_before = eng.num_steps
    eng.run_until_finished()
    assert r.finished and r.generated == gen2 and r.tokens == first + gen1 + second + gen2
    # 6 tokens in portions of 4 (two steps, the second draws), then two decode steps
    assert eng.num_steps - steps_before == 4
    eng.release_request(r)
    assert r.slot == -1 and all(g.pool.num_held == 0 for g in eng.cache.groups)
    # a request that was not kept is recomputed whole when it is continued
    r2 = eng.add_request(first, 4)
    eng.run_until_finished()
    assert r2.slot == -1 and r2.generated == gen1
    eng.append_input_tokens(r2, second, 3)
    assert r2.cached_len == 0
    eng.run_until_finished()
    assert r2.generated == gen2 and all(g.pool.num_held == 0 for g in eng.cache.groups)


def test_parked_sessions_lose_their_cache_before_running_requests_are_preempted(tmp_path):
    d = make_model_dir(tmp_path, "A")
    cfg, w = plain.read_model_dir(d)
    a, b, c = (random_tokens(n, 256, 40 + i) for i, n in enumerate((9, 10, 14)))
    eng = cpu_engine(d, page_size=4, num_pages=8, max_requests=3)
    ra = eng.add_request(a, 3, keep_session=True)
    eng.run_until_finished()
    rb = eng.add_request(b, 3, keep_session=True)
    eng.run_until_finished()
    assert eng.scheduler.parked == [ra, rb] and eng.cache.groups[0].pool.num_free == 2
    rc = eng.add_request(c, 4)  # needs 5 pages at its longest: the session parked longest goes first
    eng.run_until_finished()
    assert rc.generated == plain.generate_greedy(c, w, cfg, 4)
    assert eng.scheduler.num_evictions == 1 and eng.scheduler.num_preemptions == 0
    assert ra.slot == -1 and ra.cached_len == 0 and rb.slot >= 0 and eng.scheduler.parked == [rb]
    # the evicted session can still go on: from its first token
    more = random_tokens(2, 256, 50)
    eng.append_input_tokens(ra, more, 2)
    eng.run_until_finished()
    assert ra.generated == plain.generate_greedy(a + plain.generate_greedy(a, w, cfg, 3) + more, w, cfg, 2)
    eng.release_request(ra)
    eng.release_request(rb)
    assert all(g.pool.num_held == 0 for g in eng.cache.groups)


def test_eos_is_appended_and_ends_the_request(tmp_path):
    d = make_model_dir(tmp_path, "C")
    cfg, w = plain.read_model_dir(d)
    p = random_tokens(6, 256, 3)
    free = plain.generate_greedy(p, w, cfg, 8)
    at = next(i for i in range(2, 8) if free[i] not in free[:i])  # a token that is new where it stands
    eos = free[at]
    cut = free[: at + 1]
    assert cpu_engine(d, page_size=16, num_pages=8, max_requests=1).generate([p], 8, eos_token_id=eos) == [cut]


def test_steps_launched_ahead_learn_of_an_end_a_step_late_and_change_nothing(tmp_path):
    """Three greedy requests decode together; one meets its end-of-sequence token, one its token
    limit, one goes on.  With steps launched ahead the host reads a step's tokens while the next
    step is already on its way: the request that met its end ran one token too far (that token
    is dropped, its position counts as cached), the one at its limit was not scheduled again;
    the tokens are those of stepping one by one, a session goes on from there, a request that
    arrives in between is served, and a request that is released while a step is on its way
    takes no token any more."""
    d = make_model_dir(tmp_path, "C")
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, 311, 70 + i) for i, n in enumerate((6, 11, 3))]
    free = [plain.generate_greedy(p, w, cfg, 12) for p in prompts]
    eos = free[0][4]  # request 0 ends with its fifth token (or earlier, if the token came before)
    want0 = plain.generate_greedy(prompts[0], w, cfg, 12, eos=eos)
    assert 1 < len(want0) < 12
    outs = {}
    for ahead in (False, True):
        eng = cpu_engine(d, page_size=16, num_pages=12, max_requests=4, run_ahead=ahead)
        a = eng.add_request(prompts[0], 12, eos_token_id=eos, keep_session=True)
        b = eng.add_request(prompts[1], 7)
        c = eng.add_request(prompts[2], 30)
        late = None
        while not (a.finished and b.finished):
            eng.step()
            if late is None and len(c.generated) >= 3:
                late = eng.add_request(prompts[1][:5], 4)  # arrives while the others decode
        assert a.generated == want0 and b.generated == free[1][:7]
        # the session goes on: its history, more input, new tokens
        more = random_tokens(4, 311, 99)
        eng.append_input_tokens(a, more, 5)
        while not a.finished:
            eng.step()
        assert a.generated == plain.generate_greedy(prompts[0] + want0 + more, w, cfg, 5)
        eng.release_request(a)
        while len(c.generated) + c.pending < 20:
            eng.step()
        eng.release_request(c)  # perhaps with a step of it on its way
        eng.run_until_finished()
        assert late.finished and late.generated == plain.generate_greedy(prompts[1][:5], w, cfg, 4)
        assert c.generated == plain.generate_greedy(prompts[2], w, cfg, 30)[: len(c.generated)] and len(c.generated) >= 19
        assert all(g.pool.num_held == 0 for g in eng.cache.groups) and eng.cache.num_free_slots == 4
        outs[ahead] = (eng.num_steps_ahead, eng.num_steps)
    assert outs[False][0] == 0 and outs[True][0] > 10, outs


def test_temperature_draws_do_not_depend_on_the_batch(tmp_path):
    d = make_model_dir(tmp_path, "B")
    prompts = [random_tokens(n, 503, 20 + i) for i, n in enumerate((4, 9, 15))]
    together = cpu_engine(d, page_size=8, num_pages=16, max_requests=4)
    reqs = [together.add_request(p, 6, temperature=0.7, seed=42) for p in prompts]
    together.run_until_finished()
    for i, p in enumerate(prompts):
        alone = cpu_engine(d, page_size=8, num_pages=16, max_requests=4)
        for _ in range(i):  # same request id, so the same stream of draws
            alone.scheduler._next_id += 1
        r = alone.add_request(p, 6, temperature=0.7, seed=42)
        alone.run_until_finished()
        assert r.generated == reqs[i].generated
    greedy = cpu_engine(d, page_size=8, num_pages=16, max_requests=4).generate(prompts, 6)
    assert greedy != [r.generated for r in reqs]  # temperature is really used


class RecordedDraws:
    """Stands in for a request's generator: hands out its numbers and keeps them."""

    def __init__(self, rng):
        self.rng = rng
        self.drawn = []

    def random(self):
        self.drawn.append(self.rng.random())
        return self.drawn[-1]


def temperature_workload_matches_plain(d, eng):
    """Workload of the tiny configuration B: prompts 1/7/23/40, 6 tokens each at temperature
    0.7, page size 8, prompt portions of 16.  The uniform numbers that the engine draws are
    recorded; the plain model, fed the same numbers, must pick the same tokens from its own
    logits of the whole history."""
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, 503, 10 + i) for i, n in enumerate((1, 7, 23, 40))]
    reqs = [eng.add_request(p, 6, temperature=0.7, seed=9) for p in prompts]
    for r in reqs:
        r.rng = RecordedDraws(r.rng)
    eng.run_until_finished()
    for r, p in zip(reqs, prompts):
        assert len(r.generated) == 6 and len(r.rng.drawn) == 6
        history = list(p)
        for k, u in enumerate(r.rng.drawn):
            row = plain.model_logits_fast(history, w, cfg)[-1]
            assert r.generated[k] == plain.temperature_pick(row, 0.7, u), (r.request_id, k)
            history.append(r.generated[k])
    greedy = [plain.generate_greedy(p, w, cfg, 6) for p in prompts]
    assert greedy != [r.generated for r in reqs]  # the draws decide, not the maximum


def test_temperature_generation_matches_plain_draw_by_draw(tmp_path):
    d = make_model_dir(tmp_path, "B")
    temperature_workload_matches_plain(d, cpu_engine(d, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16,
                                                     max_tokens_per_step=24))


@pytest.mark.gpu
def test_temperature_generation_matches_plain_draw_by_draw_gpu(tmp_path):
    d = make_model_dir(tmp_path, "B", dtype=torch.bfloat16)
    model = load_model(d, "float32")
    temperature_workload_matches_plain(d, LLMEngine(model, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16,
                                                    max_tokens_per_step=24))


@pytest.mark.gpu
def test_temperature_generation_in_bfloat16_lands_where_the_plain_model_allows_gpu(tmp_path):
    """The same workload in bfloat16.  The engine's logits are within 2e-2 of the plain model's,
    so its running sum at temperature 0.7 is within 3 % of the plain one: the token it draws
    must be one whose share of the plain running sum lies within that margin of the target, and
    where the target is further than the margin from both ends of a token's share it must be
    that token.  (A draw taken from the wrong row, the wrong uniform number or a wrong running
    sum lands anywhere in the vocabulary: one chance in sixteen a draw to pass.)"""
    d = make_model_dir(tmp_path, "B", dtype=torch.bfloat16)
    model = load_model(d, "bfloat16")
    eng = LLMEngine(model, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16, max_tokens_per_step=24)
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, 503, 10 + i) for i, n in enumerate((1, 7, 23, 40))]
    reqs = [eng.add_request(p, 6, temperature=0.7, seed=9) for p in prompts]
    for r in reqs:
        r.rng = RecordedDraws(r.rng)
    eng.run_until_finished()
    margin, decided = 0.03, 0
    for r, p in zip(reqs, prompts):
        assert len(r.generated) == 6 and len(r.rng.drawn) == 6
        history = list(p)
        for k, u in enumerate(r.rng.drawn):
            row = plain.model_logits_fast(history, w, cfg)[-1]
            cdf = torch.cumsum(torch.softmax(row.double() / 0.7, dim=0), dim=0)
            got = r.generated[k]
            lo, hi = (float(cdf[got - 1]) if got else 0.0), float(cdf[got])
            assert lo - margin <= u <= hi + margin, (r.request_id, k, got, u, lo, hi)
            exact = plain.temperature_pick(row, 0.7, u)
            elo, ehi = (float(cdf[exact - 1]) if exact else 0.0), float(cdf[exact])
            if elo + margin < u < ehi - margin:
                decided += 1
                assert got == exact, (r.request_id, k)
            history.append(got)
    print(f"bfloat16 temperature: {decided} of 24 draws decided beyond the margin")


def test_a_draw_that_rounds_to_one_is_kept_below_one():
    from litellmengine_amd.sampling import Sampler

    class Ops:
        def sample(self, logits, temperature, uniform):
            self.uniform = uniform
            return torch.zeros(logits.shape[0], dtype=torch.int32)

    class Req:
        temperature = 0.7

        class rng:
            random = staticmethod(lambda: 1.0 - 2.0 ** -40)

    ops = Ops()
    Sampler(ops, "cpu").pick(torch.zeros((1, 5)), [Req()])
    assert ops.uniform.dtype == torch.float32 and float(ops.uniform[0]) < 1.0


@pytest.mark.gpu
@pytest.mark.parametrize("which,dtype", [("A", "float32"), ("B", "float32"), ("C", "float32"), ("B", "bfloat16")])
def test_greedy_generation_through_the_entry_point(tmp_path, which, dtype):
    from litellmengine_amd.entrypoints.generate import generate

    d = make_model_dir(tmp_path, which, dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, cfg["vocab_size"], 30 + i) for i, n in enumerate((5, 9, 17, 40))]
    want = [plain.generate_greedy(p, w, cfg, 8) for p in prompts]
    got = generate(d, prompts, max_tokens=8, temperature=0.0, dtype=dtype, page_size=4, prefill_chunk=16)
    if dtype == "float32":
        assert got == want
    else:  # rounding may flip a near-tie, after which the sequences part ways: near the maximum at every step
        assert all(len(g) == 8 and near_greedy(p, g, w, cfg, 8e-2) for p, g in zip(prompts, got)), (got, want)


@pytest.mark.gpu
def test_command_line_and_python_front(tmp_path, capsys):
    from litellmengine_amd.entrypoints import cli
    from litellmengine_amd.entrypoints.run_prompt import parse_new_token_ids

    d = make_model_dir(tmp_path, "A", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    want = plain.generate_greedy([5, 17, 3, 99], w, cfg, 5)
    assert cli.main(["--model", d, "--input-ids", "5, 17,3,99", "--max-tokens=5", "--temperature", "0",
                     "--dtype", "float32", "--page-size", "4"]) == 0
    out = capsys.readouterr().out
    assert parse_new_token_ids(out) == want
    assert "Generated token ids:\n  5,17,3,99," in out
    # random weights from a folder that holds a config.json only
    import os, json
    only = tmp_path / "only_config"
    os.makedirs(only)
    with open(only / "config.json", "w") as f:
        json.dump(CONFIGS["B"], f)
    assert cli.main(["--model", str(only), "--random-weights", "--seed", "3", "--input-ids", "1,2,3",
                     "--max-tokens", "4", "--temperature", "0.7"]) == 0
    ids = parse_new_token_ids(capsys.readouterr().out)
    assert len(ids) == 4 and all(0 <= i < 503 for i in ids)
    # the draws are the request's own (seeded): the same command gives the same tokens, another seed of the
    # draws others, and they are not the greedy ones
    assert cli.main(["--model", str(only), "--random-weights", "--seed", "3", "--input-ids", "1,2,3",
                     "--max-tokens", "4", "--temperature", "0.7"]) == 0
    assert parse_new_token_ids(capsys.readouterr().out) == ids
    assert cli.main(["--model", str(only), "--random-weights", "--seed", "3", "--input-ids", "1,2,3",
                     "--max-tokens", "4", "--temperature", "0"]) == 0
    assert parse_new_token_ids(capsys.readouterr().out) != ids
    assert cli.main(["--model", d, "--input-ids", "1,2", "--max-tokens", "0"]) == 1
    assert "--max-tokens must be greater than 0" in capsys.readouterr().err
    assert cli.main(["--model", d, "--input-ids", "1,x"]) == 1


@pytest.mark.gpu
def test_text_front_in_process_and_through_the_command_line(tmp_path, capsys):
    """run_prompt with a small word tokenizer written here: the chat template is applied, the
    prompt's ids go to the engine in-process and, with --engine, to the command line as a child
    process (whose `New token ids:` line is parsed); both print the plain model's greedy reply."""
    import os

    from tokenizers import Tokenizer, models, pre_tokenizers

    from litellmengine_amd.entrypoints import run_prompt
    from tests.trace_util import ROOT

    d = make_model_dir(tmp_path, "A", dtype=torch.bfloat16)
    words = ["[UNK]", "user", "assistant", "what", "is", "the", "capital", "of", "france"] + [f"w{i}" for i in range(200)]
    tok = Tokenizer(models.WordLevel({w: i for i, w in enumerate(words)}, unk_token="[UNK]"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.add_special_tokens(["<|im_start|>", "<|im_end|>"])
    tok.save(os.path.join(d, "tokenizer.json"))
    cfg, w = plain.read_model_dir(d)
    prompt = "what is the capital of france"
    start, end = tok.token_to_id("<|im_start|>"), tok.token_to_id("<|im_end|>")
    from litellmengine_amd.entrypoints.cli import templated_prompt

    # the architecture's template around the prompt (thinking off: an empty block of thoughts, unknown words here)
    ids = tok.encode(templated_prompt(d, prompt, enable_thinking=False), add_special_tokens=False).ids
    assert ids[:11] == [start, 1] + [3, 4, 5, 6, 7, 8] + [end, start, 2] and len(ids) > 11
    want = plain.generate_greedy(ids, w, cfg, 6, eos=end)
    text = tok.decode(want, skip_special_tokens=True)
    common = ["--model", d, "--prompt", prompt, "--max-tokens", "6", "--dtype", "float32", "--show-full-text"]
    assert run_prompt.main(common) == 0
    out = capsys.readouterr().out
    assert f"prompt: {len(ids)} tokens\n  " + ",".join(map(str, ids)) in out
    assert f"reply: {len(want)} tokens\n{text}\n" in out and "prompt and reply together:" in out
    assert run_prompt.main(common + ["--engine", os.path.join(ROOT, "bin", "litellmengine")]) == 0
    out = capsys.readouterr().out
    assert "New token ids:" in out and f"reply: {len(want)} tokens\n{text}\n" in out
    # without the template the words alone are the prompt
    assert run_prompt.main(common[:-1] + ["--no-chat-template", "--eos-token-id", "999"]) == 0
    out = capsys.readouterr().out
    bare = plain.generate_greedy([3, 4, 5, 6, 7, 8], w, cfg, 6)
    assert "prompt: 6 tokens\n  3,4,5,6,7,8" in out and tok.decode(bare, skip_special_tokens=True) in out
    # an engine that fails hands its exit code on
    assert run_prompt.main(common + ["--engine", "false"]) == 1


def test_token_id_grammar_and_output_parsing():
    # src/runtime/token_ids.cpp:64-109, scripts/run_prompt.py:9-27
    from litellmengine_amd.entrypoints.run_prompt import parse_new_token_ids
    from litellmengine_amd.entrypoints.token_ids import format_token_ids, parse_token_ids

    assert parse_token_ids(" 1, 2 ,3 ") == [1, 2, 3]
    assert format_token_ids([4, 5]) == "4,5"
    for bad in ("", "1,,2", "-1", "a", "1,2,", "99999999999"):
        with pytest.raises(ValueError):
            parse_token_ids(bad)
    assert parse_new_token_ids("x\nNew token ids:\n  7,8\n") == [7, 8]
    assert parse_new_token_ids("New token ids:\n  <none>\n") == []
    with pytest.raises(RuntimeError):
        parse_new_token_ids("nothing here")


def test_args_follow_the_reference():
    from litellmengine_amd.entrypoints.args import ArgsError, parse_args

    a = parse_args(["--model", "m"])
    assert (a.max_tokens, a.temperature, a.top_k, a.top_p, a.page_size) == (128, 0.7, 50, 0.9, 16)
    assert a.benchmark_requests == 32 and a.benchmark_warmup == 1 and a.eos_token_id is None
    assert parse_args(["--model=m", "--prompt-ids", "1,2"]).input_ids == "1,2"
    for bad in (["--max-tokens", "0"], ["--temperature", "-1"], ["--top-p", "0"], ["--top-k", "-1"],
                ["--eos-token-id", "-2"], ["--page-size", "0"], ["--use-kv-cache", "--use-paged-kv-cache"],
                ["--bogus"]):
        with pytest.raises(ArgsError):
            parse_args(["--model", "m"] + bad)
    with pytest.raises(ArgsError):
        parse_args([])


def near_greedy(history, generated, w, cfg, margin):
    """Every generated token is the plain model's maximum for the history before it, or within
    `margin` of it (reduced precision may flip a near-tie; the history is the engine's own)."""
    tokens = list(history) + list(generated)
    logits = plain.model_logits_fast(tokens[:-1], w, cfg)
    for k, tok in enumerate(generated):
        row = logits[len(history) + k - 1]
        if row[tok] < row.max() - margin:
            return False
    return True


def random_arrivals(eng, d, seed, page, exact):
    """Requests arrive at random steps into a pool too small for all of them, some are
    sessions that are continued once: whatever the scheduler decides (portions, preemption,
    eviction of parked sessions), every request generates what the plain model generates
    for its whole history, and in the end no page is held.  Lengths scale with the page size."""
    import random

    cfg, w = plain.read_model_dir(d)
    vocab, k = cfg["vocab_size"], page // 4
    rng = random.Random(seed)
    todo = []
    for i in range(9):
        prompt = random_tokens(rng.randint(1, 22 * k), vocab, 100 * seed + i)
        todo.append(dict(at=rng.randint(0, 25), prompt=prompt, new=rng.randint(1, 7), session=rng.random() < 0.4,
                         more=random_tokens(rng.randint(1, 6 * k), vocab, 900 + 100 * seed + i), new2=rng.randint(1, 5)))
    live, step = [], 0
    while todo or eng.has_work() or any(x["session"] and "turn2" not in x for x in live):
        for x in [x for x in todo if x["at"] <= step]:
            todo.remove(x)
            x["req"] = eng.add_request(x["prompt"], x["new"], keep_session=x["session"])
            live.append(x)
        for x in live:  # a finished session gets its second turn a few steps later
            if x["session"] and "turn2" not in x and x["req"].finished and rng.random() < 0.3:
                x["turn1"] = list(x["req"].generated)
                eng.append_input_tokens(x["req"], x["more"], x["new2"])
                x["turn2"] = True
        eng.step()
        step += 1
        assert step < 2000
    eng.run_until_finished()
    assert eng.scheduler.num_preemptions + eng.scheduler.num_evictions > 0, "the pool was meant to be too small"
    for x in live:
        if exact:
            first = plain.generate_greedy(x["prompt"], w, cfg, x["new"])
            if x["session"]:
                assert x["turn1"] == first
                assert x["req"].generated == plain.generate_greedy(x["prompt"] + first + x["more"], w, cfg, x["new2"])
            else:
                assert x["req"].generated == first
        elif x["session"]:
            assert len(x["turn1"]) == x["new"] and near_greedy(x["prompt"], x["turn1"], w, cfg, 8e-2)
            assert len(x["req"].generated) == x["new2"]
            assert near_greedy(x["prompt"] + x["turn1"] + x["more"], x["req"].generated, w, cfg, 8e-2)
        else:
            assert len(x["req"].generated) == x["new"] and near_greedy(x["prompt"], x["req"].generated, w, cfg, 8e-2)
        if x["session"]:
            eng.release_request(x["req"])
    assert all(g.pool.num_held == 0 for g in eng.cache.groups) and eng.cache.num_free_slots == 4
    return eng.scheduler.num_preemptions, eng.scheduler.num_evictions


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_arrivals_small_pool_sessions_match_plain(tmp_path, seed):
    d = make_model_dir(tmp_path, "A")
    eng = cpu_engine(d, page_size=4, num_pages=14, max_requests=4, prefill_chunk=7, max_tokens_per_step=12)
    random_arrivals(eng, d, seed, 4, exact=True)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [0, 1])
def test_random_arrivals_small_pool_sessions_match_plain_gpu(tmp_path, seed, dtype):
    """The same on the GPU, at the sizes whose small bfloat16 steps take the fused decode paths:
    preempted and evicted requests come back into slots and pages that others have used, decode
    steps run through captured graphs, and the device tables hold rows of requests long gone."""
    d = make_model_dir(tmp_path, "D", dtype=torch.bfloat16)
    model = load_model(d, dtype)
    eng = LLMEngine(model, page_size=16, num_pages=14, max_requests=4, prefill_chunk=28, max_tokens_per_step=48, run_ahead=RUN_AHEAD)
    assert eng.runner.use_graphs
    pre, ev = random_arrivals(eng, d, seed, 16, exact=dtype == "float32")
    print(f"random arrivals on the GPU, {dtype}, seed {seed}: {pre} preemptions, {ev} evictions")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sessions_on_the_gpu(tmp_path, dtype):
    """Two sessions and a plain request on the GPU (the sizes whose small bfloat16 steps take the
    fused decode paths): turns continued from the cache generate what the plain model generates
    for the whole history; nothing is held after release."""
    d = make_model_dir(tmp_path, "D", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    model = load_model(d, dtype)
    eng = LLMEngine(model, page_size=16, num_pages=24, max_requests=3, prefill_chunk=20, run_ahead=RUN_AHEAD)
    firsts = [random_tokens(n, 419, 70 + i) for i, n in enumerate((37, 9, 50))]
    mores = [random_tokens(n, 419, 80 + i) for i, n in enumerate((11, 3))]
    reqs = [eng.add_request(p, 6, keep_session=i < 2) for i, p in enumerate(firsts)]
    eng.run_until_finished()
    gen1 = [plain.generate_greedy(p, w, cfg, 6) for p in firsts]
    assert [r.generated for r in reqs] == gen1
    for r, more in zip(reqs[:2], mores):
        eng.append_input_tokens(r, more, 5)
    eng.run_until_finished()
    for r, p, g, more in zip(reqs[:2], firsts, gen1, mores):
        assert r.generated == plain.generate_greedy(p + g + more, w, cfg, 5)
        eng.release_request(r)
    assert all(g.pool.num_held == 0 for g in eng.cache.groups)


def test_chat_template_belongs_to_the_architecture(tmp_path):
    """The command line asks the registry entry of the folder's architecture for the template
    (src/tokenizer/qwen3_chat_template.cpp:7-24 for Qwen3); an architecture registered
    without one gets its prompts as they are."""
    import json
    import os

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.config.registry import get_architecture, register_architecture
    from litellmengine_amd.entrypoints.cli import templated_prompt

    qwen = tmp_path / "qwen"
    os.makedirs(qwen)
    with open(qwen / "config.json", "w") as f:
        json.dump(CONFIGS["A"], f)
    assert templated_prompt(str(qwen), "Hi") == (
        "<|im_start|>user\nHi<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n")
    assert templated_prompt(str(qwen), "Hi", enable_thinking=True).endswith("<|im_start|>assistant\n<think>\n")
    register_architecture("PlainPromptLM", Qwen3Config, get_architecture("Qwen3ForCausalLM").build)
    other = tmp_path / "other"
    os.makedirs(other)
    with open(other / "config.json", "w") as f:
        json.dump(dict(CONFIGS["A"], architectures=["PlainPromptLM"]), f)
    assert templated_prompt(str(other), "Hi") == "Hi"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,max_graphs", [("float32", 32), ("bfloat16", 32), ("float32", 2)])
def test_a_shrinking_batch_walks_through_few_graphs(tmp_path, dtype, max_graphs):
    """Thirteen requests that finish one after the other: the decode batch shrinks from 13 to 1,
    padded to 16, 8, 4, 2, 1 with rows that stand for nobody, so five graphs are captured, not
    thirteen; every request generates what the plain model generates.  A second wave finds the
    graphs again, unless only two may be kept: then the ones used least recently were dropped
    and are captured anew."""
    d = make_model_dir(tmp_path, "D", dtype=torch.bfloat16)
    cfg, w = plain.read_model_dir(d)
    model = load_model(d, dtype)
    eng = LLMEngine(model, page_size=16, num_pages=13 * 4, max_requests=13, max_tokens_per_step=512, run_ahead=RUN_AHEAD)
    eng.runner.MAX_GRAPHS = max_graphs
    for wave in range(2):
        prompts = [random_tokens(5 + 2 * i, 419, 300 + 20 * wave + i) for i in range(13)]
        reqs = [eng.add_request(p, 2 + i) for i, p in enumerate(prompts)]  # the i-th finishes after 2 + i tokens
        eng.run_until_finished()
        assert eng.runner.use_graphs and len(eng.runner._graphs) <= max_graphs
        assert eng.runner.num_captures == (5 if max_graphs >= 5 else 5 * (wave + 1)), eng.runner.num_captures
        if max_graphs >= 5:
            assert sorted(k[0] for k in eng.runner._graphs) == [1, 2, 4, 8, 16]
        for r, p in zip(reqs, prompts):
            if dtype == "float32":
                assert r.generated == plain.generate_greedy(p, w, cfg, r.max_new_tokens)
            else:
                assert len(r.generated) == r.max_new_tokens and near_greedy(p, r.generated, w, cfg, 8e-2)
        assert all(g.pool.num_held == 0 for g in eng.cache.groups)
