"""The command line, in the manner of the reference's `main` (src/main.cpp:26-335):
same option names, same banner, and the same output contract — the lines
`Generated token ids:` and `New token ids:` followed by a comma list or
`<none>`, which the Python front (run_prompt) parses."""
from __future__ import annotations

import os
import sys
import time
from typing import List

from .args import ArgsError, build_parser, parse_args, resolve_device
from .token_ids import format_token_ids, parse_token_ids


def templated_prompt(model_dir: str, prompt: str, enable_thinking: bool = False) -> str:
    """The text to tokenise for a user prompt: the chat template of the architecture that the
    folder's config.json names (the reference applies Qwen3's to every model,
    src/main.cpp:115-121), or the prompt itself for an architecture without one."""
    from ..config.registry import architecture_of_model_dir

    template = architecture_of_model_dir(model_dir).chat_template
    return prompt if template is None else template(prompt, enable_thinking)


def _load_tokenizer(model_dir: str):
    path = os.path.join(model_dir, "tokenizer.json")
    if not os.path.isfile(path):
        raise ArgsError(f"--prompt needs {path}; pass --input-ids instead")
    from tokenizers import Tokenizer

    return Tokenizer.from_file(path)


def run(argv=None) -> int:
    args = parse_args(argv)
    device = resolve_device(args.device)
    out = sys.stdout
    print("litellmengine_amd (one MI355X)", file=out)
    print(f"Device: {device}", file=out)
    print("Config:", file=out)
    for label, value in (
        ("Model", args.model), ("Max tokens", args.max_tokens), ("Temperature", args.temperature),
        ("Top-k", args.top_k), ("Top-p", args.top_p), ("Eos Token Id", -1 if args.eos_token_id is None else args.eos_token_id),
        ("dtype", args.dtype), ("page_size", args.page_size), ("benchmark", int(args.benchmark)),
        ("random_weights", int(args.random_weights)), ("seed", args.seed),
    ):
        print(f"  {label + ':':<15}{value}", file=out)

    tokenizer = None
    if args.input_ids is not None:
        input_ids = parse_token_ids(args.input_ids)
        print("\nInput token ids:\n  " + format_token_ids(input_ids), file=out)
    else:
        tokenizer = _load_tokenizer(args.model)
        input_ids = tokenizer.encode(templated_prompt(args.model, args.prompt, False), add_special_tokens=False).ids
        print("\nInput prompt:\n" + args.prompt, file=out)
        print("\nEncoded input token ids:\n  " + format_token_ids(input_ids), file=out)
    print(f"Input length: {len(input_ids)}", file=out)

    from .generate import load_for_generation, make_engine

    print("\nLoading model...", file=out)
    model = load_for_generation(args.model, args.dtype, device, args.random_weights, args.seed)
    print("Model initialized.", file=out)
    if args.top_k != 50 or args.top_p != 0.9:
        print("\nWarning: top-k and top-p are not implemented; temperature sampling only.", file=out)
    eos = -1 if args.eos_token_id is None else args.eos_token_id

    if args.benchmark:
        return _benchmark(args, model, input_ids, eos, out)

    print("\nGenerating...", file=out)
    engine = make_engine(model, [len(input_ids) + args.max_tokens], args.page_size, args.max_tokens_per_step,
                         args.prefill_chunk, args.verbose)
    new_ids = engine.generate([input_ids], args.max_tokens, eos, args.temperature, args.seed)[0]
    print("\nGenerated token ids:\n  " + format_token_ids(list(input_ids) + new_ids), file=out)
    print("\nNew token ids:\n  " + (format_token_ids(new_ids) if new_ids else "<none>"), file=out)
    if tokenizer is not None:
        print("\nDecoded new text:\n" + tokenizer.decode(new_ids), file=out)
    return 0


def _benchmark(args, model, input_ids: List[int], eos: int, out) -> int:
    """Warm-up runs, then one timed run of --benchmark-requests copies of the
    prompt, device synchronised before and after, new tokens / wall time
    (src/benchmark/generation_benchmark.cpp:430-526; result text :531-578)."""
    import torch

    from .generate import make_engine

    n = args.benchmark_requests

    def one_run(requests: int):
        engine = make_engine(model, [len(input_ids) + args.max_tokens] * requests, args.page_size,
                             args.max_tokens_per_step, args.prefill_chunk, False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        new = engine.generate([input_ids] * requests, args.max_tokens, eos, args.temperature, args.seed)
        torch.cuda.synchronize()
        return sum(len(x) for x in new), (time.perf_counter() - t0) * 1e3

    print("\nRunning generation benchmark...", file=out)
    for _ in range(args.benchmark_warmup):
        one_run(n)
    total, ms = one_run(n)
    print("\nGeneration benchmark result", file=out)
    print("  Mode:             Paged KV cache batch decode", file=out)
    print(f"  Page size:        {args.page_size}", file=out)
    print(f"  Requests:         {n}", file=out)
    print(f"  Prompt tokens:    {len(input_ids)}", file=out)
    print(f"  Max new tokens:   {args.max_tokens}", file=out)
    print(f"  Total new tokens: {total}", file=out)
    print(f"  Total time:       {ms:.3f} ms", file=out)
    print(f"  Throughput:       {total / ms * 1e3:.3f} tok/s", file=out)
    print(f"  Latency/token:    {ms / max(total, 1):.4f} ms/token", file=out)
    return 0


def main(argv=None) -> int:
    try:
        return run(argv)
    except (ArgsError, ValueError, RuntimeError, OSError) as e:  # src/main.cpp:330-334
        print(f"Error: {e}\n", file=sys.stderr)
        build_parser().print_usage(sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
