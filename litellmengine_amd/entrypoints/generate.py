"""Python entry: a model folder and prompts (token ids) in, new token ids out."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


def load_for_generation(model_dir: str, dtype="bfloat16", device=None, random_weights: bool = False, seed: int = 0):
    from ..config import load_config
    from ..models import load_model, random_model

    if device is not None:
        device = torch.device(device)
        if device.type == "cuda":
            if device.index is None:  # "cuda": the current device
                device = torch.device("cuda", torch.cuda.current_device())
            torch.cuda.set_device(device)
    if random_weights:
        return random_model(load_config(model_dir), seed, dtype, device)
    return load_model(model_dir, dtype, device)


def pages_for_requests(lengths: Sequence[int], page_size: int) -> int:
    """Pages so that every request can hold its longest length at once, plus one
    spare page each (the reference sizes its pool as prompt + max_tokens + 16,
    src/main.cpp:264-268)."""
    return sum((n + page_size - 1) // page_size + 1 for n in lengths)


def make_engine(model, total_lengths: Sequence[int], page_size: int = 16, max_tokens_per_step: int = 2048,
                prefill_chunk: Optional[int] = None, verbose: bool = False, num_pages: Optional[int] = None):
    from ..engine import LLMEngine

    pages = num_pages or pages_for_requests(total_lengths, page_size)
    longest = max(total_lengths)
    return LLMEngine(
        model, page_size=page_size, num_pages=pages, max_requests=max(1, len(total_lengths)),
        max_tokens_per_step=max_tokens_per_step, prefill_chunk=prefill_chunk,
        max_pages_per_request=(longest + page_size - 1) // page_size + 1, verbose=verbose,
    )


def generate(model_dir: str, prompts: Sequence[Sequence[int]], max_tokens: int = 128, temperature: float = 0.0,
             eos_token_id: int = -1, dtype="bfloat16", device=None, page_size: int = 16, seed: int = 0,
             random_weights: bool = False, max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None,
             verbose: bool = False, num_pages: Optional[int] = None) -> List[List[int]]:
    """Generate up to `max_tokens` new tokens for every prompt (lists of token
    ids), all requests batched.  Returns the new ids of each."""
    model = load_for_generation(model_dir, dtype, device, random_weights, seed)
    engine = make_engine(model, [len(p) + max_tokens for p in prompts], page_size, max_tokens_per_step,
                         prefill_chunk, verbose, num_pages)
    return engine.generate(prompts, max_tokens, eos_token_id, temperature, seed)
