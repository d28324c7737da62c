#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen3-8B layer sizes, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

    python bench.py --dtype float32                               # the same in true 32-bit
    python bench.py --sizes 32b | --sizes 0p6b                    # the decode workload at other layer sizes
    python bench.py --workload reference-0p6b [--dtype float32]   # the reference's own benchmark shape
    python bench.py --workload mixed-32b [--layers L]             # a prompt chunk beside 63 decoded tokens
    python bench.py --workload serving                            # requests of many lengths arriving over time

A "step" is one decode step of the whole engine (scheduler, model step over the
paged cache, sampling) with `batch` live requests whose context ends at
`context` tokens.  Seeded random weights (bfloat16), uniform random token ids.
One JSON line is printed: `value` = decoded tokens per second, `prefill` = a
2048-token prompt in one step, `more` = the same measurements, shorter, of the true 32-bit
path, of the Qwen3-32B sizes and of the reference's own benchmark shape (default line only;
--no-more skips them), `roofline` = bytes the decode step has to read
(every weight it uses once + the cache of the live requests) / its time against
8 TB/s, `points` = decode at batch 1 and 64.  Both rooflines are also given against
what this machine reaches on kernels that do nothing else (`measured_peak`: a
read-only kernel over 4 GiB, a kernel of matrix instructions on registers).  The reference publishes nothing
for this configuration (its only table is Qwen3-0.6B in float32 on an unnamed
GPU, readme.md:62-66), so `vs_baseline` is null.
"""
import argparse
import json
import sys
import time

# Qwen3-8B layer sizes
SIZES = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36, hidden_size=4096,
    num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
)
# Qwen3-0.6B layer sizes: the model of the reference's published table (readme.md:62-66)
SIZES_0P6B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=28, hidden_size=1024,
    num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
)
# Qwen3-32B layer sizes
SIZES_32B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=64, hidden_size=5120,
    num_attention_heads=64, num_key_value_heads=8, head_dim=128, intermediate_size=25600, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
)
REFERENCE_TOK_S = 189.06  # readme.md:66: 32 requests x 64 new tokens, paged batch kernel, FP32, an unnamed CUDA GPU
HBM_PEAK = 8.0e12  # bytes/s
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
PAGE_SIZE = 16
PREFILL_TOKENS = 2048


def weight_bytes_per_step(cfg, elem=2):
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h  # qkv
    per_layer += h * cfg.num_attention_heads * d  # o
    per_layer += 3 * h * cfg.intermediate_size  # gate, up, down
    per_layer += 2 * h + 2 * d  # norms
    return (per_layer * cfg.num_hidden_layers + h + cfg.vocab_size * h) * elem


def kv_bytes_per_token(cfg, elem=2):
    return 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers * elem


def prefill_flops(cfg, tokens):
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h + h * cfg.num_attention_heads * d
    per_layer += 3 * h * cfg.intermediate_size
    linear = 2.0 * tokens * per_layer * cfg.num_hidden_layers + 2.0 * cfg.vocab_size * h  # head: one row
    attention = 4.0 * cfg.num_attention_heads * d * (tokens * (tokens + 1) / 2) * cfg.num_hidden_layers
    return linear + attention


def make_engine(model, batch, context, max_tokens_per_step=8192):
    from litellmengine_amd.engine import LLMEngine

    pages_each = (context + PAGE_SIZE - 1) // PAGE_SIZE + 1
    return LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * batch, max_requests=batch,
                     max_tokens_per_step=max_tokens_per_step, prefill_chunk=2048, max_pages_per_request=pages_each)


def random_prompts(n, length, vocab, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n, length), generator=g).tolist()


def time_decode(model, cfg, batch, context, steps, warmup):
    """`steps` timed decode steps of `batch` requests; the last one runs at a
    attends to `context` keys.  Returns seconds per step."""
    import torch

    engine = make_engine(model, batch, context)
    prompt_len = context - (steps + warmup)
    for p in random_prompts(batch, prompt_len, cfg.vocab_size, 100 + batch):
        engine.prefill(engine.add_request(p, steps + warmup + 1))  # each prompt alone, in portions
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    lens = [r.cached_len for r in engine.scheduler.requests.values()]
    assert all(n == context for n in lens), lens
    return dt


def time_prefill(model, cfg, tokens, repeats=3):
    import torch

    engine = make_engine(model, 1, tokens + 16, max_tokens_per_step=tokens)
    best = None
    for i in range(repeats + 1):
        req = engine.add_request(random_prompts(1, tokens, cfg.vocab_size, 7 + i)[0], 1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()  # the whole prompt in one step, one token drawn
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert req.finished and engine.num_steps == i + 1
        if i > 0:  # the first run warms up
            best = dt if best is None else min(best, dt)
    return best


def measure_peaks(dtype):
    """What this machine reaches on kernels that do nothing else: (bytes/s of a kernel that only
    reads 4 GiB from HBM, flops/s of a kernel that only issues matrix instructions of `dtype`
    on registers).  The rooflines are given against the published peaks and against these."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()

    def timed(launch, repeats=8):
        # by the wall clock around a run of launches (no timing events: recording one makes the runtime
        # keep time stamps of every later launch of the process, which costs the short kernels of a
        # decode step about a microsecond each)
        launch()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(repeats):
                launch()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / repeats
            best = dt if best is None else min(best, dt)
        return best

    data = torch.empty(1 << 30, dtype=torch.int32, device="cuda")  # 4 GiB: far more than the caches hold
    data.fill_(1)
    nbytes = data.numel() * 4
    read = max(nbytes / timed(lambda b=b: ops.probe_read_stream(data, b)) for b in (256, 16384, 65536))
    del data
    torch.cuda.empty_cache()
    tdtype = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    units = torch.cuda.get_device_properties(0).multi_processor_count
    flops = [0.0]

    def mfma():
        flops[0] = ops.probe_mfma(tdtype, 8 * units, 4000)

    seconds = timed(mfma, repeats=2)
    return read, flops[0] / seconds


def flat_config(cfg, full_layers, **more):
    d = {"layers": cfg.num_hidden_layers, "layers_of_full_model": full_layers, "hidden": cfg.hidden_size,
         "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
         "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "page_size": PAGE_SIZE,
         "parallelism": "none (1 GPU)"}
    d.update(more)
    return d


def time_reference_workload(dtype, runs, warmup):
    """The shape of the reference's benchmark (src/benchmark/generation_benchmark.cpp:259-315,
    :430-526): 32 requests, 64-token prompts, 64 new tokens each, greedy; warm-up runs, then
    the whole run is timed, prompts included.  Returns (config, requests, prompt length, new
    tokens, seconds a run)."""
    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.engine import LLMEngine
    from litellmengine_amd.models import random_model

    cfg = Qwen3Config.from_dict(SIZES_0P6B)
    model = random_model(cfg, seed=0, dtype=dtype)
    requests, prompt_len, new_tokens = 32, 64, 64
    pages_each = (prompt_len + new_tokens + PAGE_SIZE - 1) // PAGE_SIZE + 1
    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * requests, max_requests=requests,
                       max_tokens_per_step=requests * prompt_len, max_pages_per_request=pages_each)
    times = []
    for run in range(warmup + runs):
        prompts = random_prompts(requests, prompt_len, cfg.vocab_size, 1000 + run)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = engine.generate(prompts, new_tokens)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert all(len(o) == new_tokens for o in out)
        if run >= warmup:
            times.append(dt)
    return cfg, requests, prompt_len, new_tokens, sum(times) / len(times)


def reference_workload(args):
    cfg, requests, prompt_len, new_tokens, dt = time_reference_workload(args.dtype, args.steps, args.warmup)
    value = requests * new_tokens / dt
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "new tok/s of 32 requests x 64-token prompts x 64 new tokens, prompts included, Qwen3-0.6B sizes",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / REFERENCE_TOK_S, 2), "dtype": short,
        "data": "synthetic: seeded random weights, uniform random token ids; the reference's 189.06 tok/s is FP32 "
                "on an unnamed CUDA GPU with a real checkpoint and one text prompt",
        "config": flat_config(cfg, SIZES_0P6B["num_hidden_layers"], model="Qwen3-0.6B sizes (random weights)",
                              global_batch=requests, seq_len=prompt_len + new_tokens, new_tokens=new_tokens),
    }))
    return 0


def mixed_workload(args):
    """One 2048-token portion of a long prompt beside 63 decoded tokens at context 4096,
    Qwen3-32B layer sizes: the step a serving loop runs while a prompt comes in."""
    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    layers = args.layers if args.layers != SIZES["num_hidden_layers"] else SIZES_32B["num_hidden_layers"]
    cfg = Qwen3Config.from_dict(dict(SIZES_32B, num_hidden_layers=layers))
    model = random_model(cfg, seed=0, dtype=args.dtype)
    decoders, context, chunk = 63, 4096, PREFILL_TOKENS
    steps, warmup = args.steps, args.warmup
    long_prompt = chunk * (steps + warmup)
    pages_dec = (context + PAGE_SIZE - 1) // PAGE_SIZE + 1
    pages_long = (long_prompt + PAGE_SIZE - 1) // PAGE_SIZE + 2
    from litellmengine_amd.engine import LLMEngine

    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_dec * decoders + pages_long,
                       max_requests=decoders + 1, max_tokens_per_step=chunk + decoders, prefill_chunk=chunk,
                       max_pages_per_request=max(pages_dec, pages_long))
    prompt_len = context - (steps + warmup)
    for p in random_prompts(decoders, prompt_len, cfg.vocab_size, 300):
        engine.prefill(engine.add_request(p, steps + warmup + 1))
    long_req = engine.add_request(random_prompts(1, long_prompt, cfg.vocab_size, 301)[0], 1)
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    assert long_req.finished and long_req.cached_len == long_prompt, (long_req.cached_len, long_prompt)
    lens = [r.cached_len for r in engine.scheduler.requests.values() if r is not long_req]
    assert all(n == context for n in lens), lens
    tokens = chunk + decoders
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h + h * cfg.num_attention_heads * d
    per_layer += 3 * h * cfg.intermediate_size
    past_mean = chunk * (warmup + (steps - 1) / 2.0)  # keys before the timed portions, on average
    attn = 4.0 * cfg.num_attention_heads * d * (chunk * past_mean + chunk * (chunk + 1) / 2 + decoders * context)
    flops = (2.0 * tokens * per_layer + attn) * cfg.num_hidden_layers + 2.0 * (decoders + 1) * cfg.vocab_size * h
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "tokens/s of a mixed step: a 2048-token prompt portion beside 63 decoded tokens at context 4096, "
                  "Qwen3-32B sizes",
        "value": round(tokens / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: seeded random weights, uniform random token ids",
        "config": flat_config(cfg, SIZES_32B["num_hidden_layers"], model="Qwen3-32B sizes (random weights)",
                              global_batch=decoders + 1, seq_len=context, prompt_portion=chunk),
        "roofline": {"bound": "mfma", "achieved": round(flops / dt / 1e12, 1), "peak": MFMA_PEAK[short] / 1e12,
                     "unit": "TFLOP/s", "frac": round(flops / dt / MFMA_PEAK[short], 4)},
    }))
    return 0


def serving_workload(args):
    """Requests of many lengths arriving over time, through the engine's own scheduler, at the
    Qwen3-8B layer sizes: 200 requests, prompts of 30 to 3050 tokens, 16 to 256 new tokens each,
    one arriving every second step, at most 64 live, a budget of 2048 tokens a step.  The whole run
    is timed (prompt portions beside decoded tokens, graph captures included); all tokens / time."""
    import collections
    import random

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.engine import LLMEngine
    from litellmengine_amd.models import random_model

    cfg = Qwen3Config.from_dict(dict(SIZES, num_hidden_layers=args.layers))
    model = random_model(cfg, seed=0, dtype=args.dtype)
    rng = random.Random(5)
    requests, live, every = 200, 64, 2
    sizes = [(rng.choice([30, 100, 300, 700, 1500, 3000]) + rng.randint(0, 50), rng.choice([16, 64, 128, 256]))
             for _ in range(requests)]
    longest = max(p + g for p, g in sizes)
    pages_each = (longest + PAGE_SIZE - 1) // PAGE_SIZE + 1
    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * live, max_requests=live,
                       max_tokens_per_step=PREFILL_TOKENS, max_pages_per_request=pages_each)
    todo = [(random_prompts(1, p, cfg.vocab_size, 100 + i)[0], g) for i, (p, g) in enumerate(sizes)]
    kinds = collections.defaultdict(lambda: [0, 0.0])  # kind -> steps, seconds, then the tokens of every such step
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = 0
    while todo or engine.has_work():
        if todo and steps % every == 0:
            prompt, new = todo.pop(0)
            engine.add_request(prompt, new)
        before = sum(r.cached_len for r in engine.scheduler.requests.values())
        captures, graph_steps = engine.runner.num_captures, engine.runner.num_graph_steps
        ts = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - ts
        ran = sum(r.cached_len for r in engine.scheduler.requests.values()) - before
        kind = ("capture" if engine.runner.num_captures > captures else
                "decode_only_graph" if engine.runner.num_graph_steps > graph_steps else
                "le64" if ran <= 64 else "le256" if ran <= 256 else "le1024" if ran <= 1024 else "gt1024")
        kinds[kind][0] += 1
        kinds[kind][1] += dt
        kinds[kind].append(ran)
        steps += 1
    total = time.perf_counter() - t0
    new_tokens = sum(g for _, g in sizes)
    all_tokens = sum(p + g for p, g in sizes)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "tokens/s, prompts included, of 200 requests (prompts of 30-3050 tokens, 16-256 new tokens) "
                  "arriving one every second step, at most 64 live, Qwen3-8B sizes",
        "value": round(all_tokens / total, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 0,
        "ms_per_step": round(total / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: seeded random weights, uniform random token ids, seeded lengths",
        "config": flat_config(cfg, SIZES["num_hidden_layers"], model="Qwen3-8B sizes (random weights)",
                              global_batch=live, requests=requests, token_budget=PREFILL_TOKENS),
        "new_tokens_per_s": round(new_tokens / total, 1), "seconds": round(total, 3),
        "graph_captures": engine.runner.num_captures,
        "steps_by_tokens": {k: {"steps": v[0], "ms_each": round(v[1] / v[0] * 1e3, 2), "share": round(v[1] / total, 3),
                                "tokens_each": round(sum(v[2:]) / v[0], 1)}
                            for k, v in sorted(kinds.items())},
    }))
    return 0


def more_workloads(steps, warmup):
    """What else the default line carries, each measured like the headline but shorter: the true
    32-bit path at the Qwen3-8B sizes (decode at batch 8, a 2048-token prompt), decode at batch 8
    at the Qwen3-32B sizes, and the reference's own benchmark shape at the Qwen3-0.6B sizes.
    Flat: numbers, and for each workload one string that names its sizes."""
    import gc

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    def sizes_of(cfg, what):
        return (f"{what}: {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_attention_heads}/"
                f"{cfg.num_key_value_heads} heads of {cfg.head_dim}, intermediate {cfg.intermediate_size}, vocab "
                f"{cfg.vocab_size}, page {PAGE_SIZE}, random weights")

    def free():
        gc.collect()
        torch.cuda.empty_cache()

    more = {}
    steps, warmup = max(4, min(steps, 10)), max(1, min(warmup, 2))
    cfg = Qwen3Config.from_dict(SIZES)
    model = random_model(cfg, seed=0, dtype="float32")
    dt = time_decode(model, cfg, 8, 4096, steps, warmup)
    step_bytes = weight_bytes_per_step(cfg, 4) + 8 * (4096 - (steps - 1) / 2.0) * kv_bytes_per_token(cfg, 4)
    pt = time_prefill(model, cfg, PREFILL_TOKENS, repeats=1)
    more.update({
        "fp32_8b": sizes_of(cfg, "true 32-bit path, Qwen3-8B sizes, decode batch 8 at context 4096 and a 2048-token prompt"),
        "fp32_8b_decode_b8_tok_s": round(8 / dt, 2), "fp32_8b_decode_b8_ms": round(dt * 1e3, 3),
        "fp32_8b_decode_b8_hbm_frac": round(step_bytes / dt / HBM_PEAK, 4),
        "fp32_8b_prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "fp32_8b_prefill_ms": round(pt * 1e3, 2),
        "fp32_8b_prefill_frac": round(prefill_flops(cfg, PREFILL_TOKENS) / pt / MFMA_PEAK["fp32"], 4),
    })
    del model
    free()
    cfg = Qwen3Config.from_dict(SIZES_32B)
    model = random_model(cfg, seed=0, dtype="bfloat16")
    dt = time_decode(model, cfg, 8, 4096, steps, warmup)
    step_bytes = weight_bytes_per_step(cfg, 2) + 8 * (4096 - (steps - 1) / 2.0) * kv_bytes_per_token(cfg, 2)
    more.update({
        "bf16_32b": sizes_of(cfg, "Qwen3-32B sizes, bf16, decode batch 8 at context 4096"),
        "bf16_32b_decode_b8_tok_s": round(8 / dt, 2), "bf16_32b_decode_b8_ms": round(dt * 1e3, 3),
        "bf16_32b_decode_b8_hbm_frac": round(step_bytes / dt / HBM_PEAK, 4),
    })
    del model
    free()
    cfg, requests, prompt_len, new_tokens, dt = time_reference_workload("bfloat16", 3, 1)
    more.update({
        "bf16_0p6b_reference_shape": sizes_of(cfg, f"Qwen3-0.6B sizes, bf16, {requests} requests x {prompt_len}-token prompts x "
                                              f"{new_tokens} new tokens, prompts included (the shape of the reference's "
                                              f"{REFERENCE_TOK_S} tok/s, which is FP32 on an unnamed CUDA GPU)"),
        "bf16_0p6b_reference_shape_tok_s": round(requests * new_tokens / dt, 1),
        "bf16_0p6b_reference_shape_ms": round(dt * 1e3, 2),
    })
    free()
    return more


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=SIZES["num_hidden_layers"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--no-more", action="store_true", help="skip the other workloads that the default line carries")
    ap.add_argument("--sizes", default="8b", choices=["8b", "0p6b", "32b"],
                    help="layer sizes of the decode workload: Qwen3-8B (default, the headline), Qwen3-0.6B or Qwen3-32B")
    ap.add_argument("--workload", default="decode", choices=["decode", "reference-0p6b", "mixed-32b", "serving"],
                    help="decode (default: the headline line), the reference's own benchmark shape at Qwen3-0.6B "
                         "sizes, or a mixed prompt-portion + decode step at Qwen3-32B sizes")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported")
        return 2
    if args.workload != "decode":
        import torch

        torch.cuda.set_device(0)
        if args.workload == "reference-0p6b":
            args.steps, args.warmup = min(args.steps, 5), min(args.warmup, 1)
            return reference_workload(args)
        if args.workload == "serving":
            return serving_workload(args)
        args.steps, args.warmup = min(args.steps, 3), min(args.warmup, 1)
        return mixed_workload(args)

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    table = {"8b": SIZES, "0p6b": SIZES_0P6B, "32b": SIZES_32B}[args.sizes]
    layers = args.layers if args.layers != SIZES["num_hidden_layers"] or args.sizes == "8b" else table["num_hidden_layers"]
    sizes = dict(table, num_hidden_layers=layers)
    cfg = Qwen3Config.from_dict(sizes)
    name = {"8b": "Qwen3-8B", "0p6b": "Qwen3-0.6B", "32b": "Qwen3-32B"}[args.sizes]
    torch.cuda.set_device(0)
    model = random_model(cfg, seed=0, dtype=args.dtype)
    elem = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "fp32"

    dt = time_decode(model, cfg, args.batch, args.context, args.steps, args.warmup)
    value = args.batch / dt
    avg_ctx = args.context - (args.steps - 1) / 2.0
    step_bytes = weight_bytes_per_step(cfg, elem) + args.batch * avg_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / dt
    line = {
        "metric": f"decode tok/s @ batch {args.batch}, {name} sizes, context {args.context} (+ prefill tok/s @ 2048, % roofline)",
        "value": round(value, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {
            "model": f"{name} sizes (random weights)", "layers": cfg.num_hidden_layers,
            "layers_of_full_model": table["num_hidden_layers"], "hidden": cfg.hidden_size,
            "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "global_batch": args.batch,
            "seq_len": args.context, "page_size": PAGE_SIZE, "prefill_tokens": PREFILL_TOKENS, "parallelism": "none (1 GPU)",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        # The decode points come before the probes of the peaks (measured so, batch 1 came out 2 %
        # faster in three runs out of three; three seconds of matrix instructions or of reading
        # before a decode run, in one process, changed nothing: the cause is not known).
        points = {}
        s = max(8, args.steps // 2)
        points["decode_b1"] = round(1 / time_decode(model, cfg, 1, args.context, s, 4), 2)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line["prefill"] = {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS, "ms": round(pt * 1e3, 3),
                           "frac": round(prefill_flops(cfg, PREFILL_TOKENS) / pt / MFMA_PEAK[short], 4)}
        points["decode_b64"] = round(64 / time_decode(model, cfg, 64, args.context, s, 4), 2)
        read_peak, mfma_peak = measure_peaks(args.dtype)
        line["roofline"]["measured_peak"] = round(read_peak / 1e9, 1)
        line["roofline"]["frac_of_measured"] = round(achieved / read_peak, 4)
        line["prefill"]["measured_peak_tflops"] = round(mfma_peak / 1e12, 1)
        line["prefill"]["frac_of_measured"] = round(prefill_flops(cfg, PREFILL_TOKENS) / pt / mfma_peak, 4)
        line["points"] = points
        headline = (args.sizes == "8b" and args.dtype == "bfloat16" and layers == SIZES["num_hidden_layers"]
                    and args.batch == 8 and args.context == 4096)
        if headline and not args.no_more:
            del model
            line["more"] = more_workloads(args.steps, args.warmup)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
