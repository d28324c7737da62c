"""The generation engine: scheduler + step function + sampler.

Counterpart of PagedGenerateEngine (include/engine/paged_generate_engine.hpp:14-87,
src/engine/paged_generate_engine.cpp:17-608): add_request, then steps until
everything finished.  One `step()` here runs whatever the scheduler chose,
prompt portions beside decoded tokens.
"""
from __future__ import annotations

import sys
from typing import Dict, List, Optional, Sequence

from ..cache import CacheManager
from ..sampling import Sampler
from .batch import StepEntry
from .request import Request
from .runner import ModelRunner
from .scheduler import Scheduler


class LLMEngine:
    def __init__(self, model, *, page_size: int = 16, num_pages: int, max_requests: int = 64,
                 max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None,
                 max_pages_per_request: Optional[int] = None, verbose: bool = False):
        ctx = model.ctx
        self.model = model
        self.cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                                  max_pages_per_request=max_pages_per_request, dtype=ctx.dtype, device=ctx.device,
                                  max_tokens_per_step=max_tokens_per_step)
        self.runner = ModelRunner(model, self.cache)
        self.scheduler = Scheduler(self.cache, max_tokens_per_step, prefill_chunk)
        self.sampler = Sampler(ctx.ops, ctx.device)
        self.verbose = verbose
        self.num_steps = 0

    def _check_ids(self, token_ids: Sequence[int]) -> None:
        for t in token_ids:
            if not 0 <= int(t) < self.model.vocab_size:
                raise ValueError(f"token id {t} outside [0, {self.model.vocab_size})")

    def add_request(self, prompt_ids: Sequence[int], max_new_tokens: int, eos_token_id: int = -1,
                    temperature: float = 0.0, seed: int = 0, keep_session: bool = False) -> Request:
        """`keep_session`: the request keeps its cache when it finishes, for
        append_input_tokens; release_request ends it."""
        self._check_ids(prompt_ids)
        return self.scheduler.add_request(prompt_ids, max_new_tokens, eos_token_id, temperature, seed, keep_session)

    def append_input_tokens(self, request: Request, token_ids: Sequence[int], max_new_tokens: int,
                            eos_token_id: int = -1) -> Request:
        """A further turn of a finished request: its history, then `token_ids`, then up to
        `max_new_tokens` new ones (src/engine/paged_generate_engine.cpp:81-97)."""
        self._check_ids(token_ids)
        return self.scheduler.append_input_tokens(request.request_id, token_ids, max_new_tokens, eos_token_id)

    def release_request(self, request: Request) -> None:
        self.scheduler.release_request(request.request_id)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def step(self, only: Optional[Sequence[int]] = None) -> List[Request]:
        """One scheduled step (of the requests with the ids in `only`, if given).
        Returns the requests that finished in it."""
        plan = self.scheduler.schedule(only)
        if not plan:
            return []
        entries = [
            StepEntry(p.request.slot, p.request.tokens[p.start : p.start + p.num_tokens],
                      [p.num_tokens - 1] if p.samples else [])
            for p in plan
        ]
        logits = self.runner.step(entries, borrow=True)
        sampled = self.sampler.pick(logits, [p.request for p in plan if p.samples])
        done = self.scheduler.update(plan, sampled)
        self.num_steps += 1
        if self.verbose:  # per-step lines on stderr, src/engine/paged_generate_engine.cpp:578-595
            parts = ", ".join(f"req {p.request.request_id}: {p.num_tokens} tok" for p in plan)
            print(f"[step {self.num_steps}] {parts}; sampled {sampled}", file=sys.stderr)
        return done

    def prefill(self, request: Request) -> None:
        """Run `request` alone until its prompt is cached and its first token drawn
        (PagedGenerateEngine::prefill, src/engine/paged_generate_engine.cpp:99-149)."""
        while not request.finished and (request.cached_len == 0 or request.extend_len > 1):
            self.step(only=[request.request_id])

    def run_until_finished(self) -> None:
        while self.has_work():
            self.step()

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, eos_token_id: int = -1,
                 temperature: float = 0.0, seed: int = 0) -> List[List[int]]:
        """New token ids of every prompt (EOS included when it ended the request)."""
        reqs = [self.add_request(p, max_new_tokens, eos_token_id, temperature, seed) for p in prompts]
        self.run_until_finished()
        return [list(r.generated) for r in reqs]
