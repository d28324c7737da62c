"""Command-line options, with the reference's names, meanings and defaults where
it has them (include/runtime/args.hpp:8-37, src/runtime/args.cpp:82-159); both
`--key value` and `--key=value` are taken.  Options of this engine's own:
--prompt-ids (alias of --input-ids), --random-weights, --seed, --dtype,
--prefill-chunk, --max-tokens-per-step."""
from __future__ import annotations

import argparse


class ArgsError(ValueError):
    pass


class _Parser(argparse.ArgumentParser):
    def error(self, message):
        raise ArgsError(message)


def build_parser() -> argparse.ArgumentParser:
    p = _Parser(prog="litellmengine", add_help=True, allow_abbrev=False,
                description="Generate tokens with the model in a folder (its config.json names the architecture) "
                            "on one MI355X.")
    p.add_argument("--model", required=True, help="local model folder (config.json + safetensors)")
    p.add_argument("--prompt", default="What is the capital of France?", help="input prompt (needs tokenizer.json)")
    p.add_argument("--input-ids", "--prompt-ids", dest="input_ids", default=None,
                   help='comma-separated token ids, e.g. "1,2,3"; bypasses the tokenizer')
    p.add_argument("--max-tokens", type=int, default=128, help="maximum generated tokens, default 128")
    p.add_argument("--temperature", type=float, default=0.7, help="sampling temperature, 0 = greedy, default 0.7")
    p.add_argument("--top-k", type=int, default=50, help="parsed and ignored, as in the reference")
    p.add_argument("--top-p", type=float, default=0.9, help="parsed and ignored, as in the reference")
    p.add_argument("--eos-token-id", type=int, default=None, help="stop when this token id is generated")
    p.add_argument("--device", default=None, help="cuda, cuda:0, gpu or auto (there is no CPU path)")
    p.add_argument("--verbose", action="store_true", help="per-step lines on stderr")
    p.add_argument("--benchmark", action="store_true", help="time generation instead of printing tokens")
    p.add_argument("--benchmark-requests", type=int, default=32)
    p.add_argument("--benchmark-warmup", type=int, default=1)
    p.add_argument("--use-kv-cache", action="store_true", help="accepted; the cache is always paged here")
    p.add_argument("--use-paged-kv-cache", action="store_true", help="accepted; the cache is always paged here")
    p.add_argument("--page-size", type=int, default=16, help="tokens per cache page, default 16")
    p.add_argument("--benchmark-interleaved", action="store_true", help="accepted; requests are always batched here")
    p.add_argument("--benchmark-batch-decode", action="store_true", help="accepted; requests are always batched here")
    # this engine's own
    p.add_argument("--random-weights", action="store_true",
                   help="seeded random weights for the sizes in MODEL/config.json (no safetensors needed)")
    p.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--prefill-chunk", type=int, default=None, help="most prompt tokens of one request in a step")
    p.add_argument("--max-tokens-per-step", type=int, default=2048, help="token budget of one step")
    return p


def parse_args(argv=None):
    args = build_parser().parse_args(argv)
    # src/runtime/args.cpp:135-157 and src/main.cpp:58-84
    if args.max_tokens <= 0:
        raise ArgsError("--max-tokens must be greater than 0")
    if args.temperature < 0.0:
        raise ArgsError("--temperature must be >= 0")
    if args.top_k < 0:
        raise ArgsError("--top-k must be >= 0")
    if not 0.0 < args.top_p <= 1.0:
        raise ArgsError("--top-p must be in range (0, 1]")
    if args.eos_token_id is not None and args.eos_token_id < 0:
        raise ArgsError("--eos-token-id must be >= 0")
    if args.use_kv_cache and args.use_paged_kv_cache:
        raise ArgsError("Cannot enable both --use-kv-cache and --use-paged-kv-cache")
    if args.page_size <= 0:
        raise ArgsError("--page-size must be positive")
    if args.benchmark_interleaved and args.benchmark_batch_decode:
        raise ArgsError("Cannot enable both --benchmark-interleaved and --benchmark-batch-decode")
    if args.benchmark_requests <= 0 or args.benchmark_warmup < 0:
        raise ArgsError("--benchmark-requests must be positive and --benchmark-warmup >= 0")
    return args


def resolve_device(name):
    """src/core/device.cpp:20-40 knows cpu / cuda / gpu / auto; this engine has no
    CPU path, so cpu is refused."""
    import torch

    name = (name or "auto").lower()
    if name == "cpu":
        raise ArgsError("--device cpu: this engine runs on the GPU only")
    if name in ("auto", "gpu", "cuda"):
        index = 0
    elif name.startswith("cuda:") and name[5:].isdigit():
        index = int(name[5:])
    else:
        raise ArgsError(f"Unknown device: {name}")
    if not torch.cuda.is_available():
        raise ArgsError("no GPU is visible")
    return torch.device("cuda", index)
