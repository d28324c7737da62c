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
from .request import Request, RequestStatus
from .runner import ModelRunner
from .scheduler import Scheduler


class LLMEngine:
    def __init__(self, model, *, page_size: int = 16, num_pages: int, max_requests: int = 64,
                 max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None,
                 max_pages_per_request: Optional[int] = None, verbose: bool = False,
                 run_ahead: Optional[bool] = None):
        """`run_ahead`: steps in which every running request decodes greedily are launched before
        the tokens of the step before them have been read (default: on a GPU).  The device keeps
        each request's last pick and feeds it to the next step itself, so the GPU does not wait
        for the host between steps; what the host learns a step late is only that a request met
        its end-of-sequence token, and the one token it then ran too far is dropped."""
        ctx = model.ctx
        self.model = model
        self.cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                                  max_pages_per_request=max_pages_per_request, dtype=ctx.dtype, device=ctx.device,
                                  max_tokens_per_step=max_tokens_per_step)
        self.run_ahead = ctx.device.type == "cuda" if run_ahead is None else bool(run_ahead)
        self.runner = ModelRunner(model, self.cache, pick_tokens=self.run_ahead)
        self._ahead = None  # (plan, PendingTokens) of a step that is on its way
        self.num_steps_ahead = 0  # steps that were launched before the step before them had been read
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

    # -- steps launched ahead ---------------------------------------------------------------
    def _may_run_ahead(self, only) -> bool:
        """Whether the next step can be launched without the tokens of the one on its way: every
        running request decodes greedily (its one pending token is, or will be, on the device),
        nobody waits to be admitted, and the pages are there without taking anybody's."""
        s = self.scheduler
        if not self.run_ahead or only is not None or self.verbose or s.waiting or not s.running:
            return False
        runs = []
        for r in s.running:
            if r.temperature > 0.0 or r.extend_len != 1:
                return False
            if not r.awaits_last_token:
                runs.append((r.slot, r.cached_len + 1))
        if len(runs) > min(s.max_tokens_per_step, self.runner.MAX_GRAPH_BATCH):
            return False
        return not runs or self.cache.can_extend(runs)

    def finish_steps(self) -> List[Request]:
        """Read the tokens of the step that is on its way, if there is one; the requests that
        finished in it.  (Every path that needs the host's view up to date starts here.)"""
        if self._ahead is None:
            return []
        plan, pending = self._ahead
        self._ahead = None
        return self.scheduler.resolved(plan, pending.wait())

    def _step_ahead(self) -> List[Request]:
        plan = self.scheduler.schedule(None)
        if not plan:  # everybody waits for a last token
            return self.finish_steps()
        entries = [StepEntry(p.request.slot, [-1] if p.request.pending else p.request.tokens[p.start : p.start + 1], [0])
                   for p in plan]
        pending = self.runner.step_ahead(entries)
        self.scheduler.launched(plan)
        done = self.finish_steps()  # the step before: by now the GPU has this one to go on with
        for p in plan:
            if p.request.status is RequestStatus.RUNNING:
                p.request.pending = 1
        self._ahead = (plan, pending)
        self.num_steps += 1
        self.num_steps_ahead += 1
        return done

    def step(self, only: Optional[Sequence[int]] = None) -> List[Request]:
        """One scheduled step (of the requests with the ids in `only`, if given).
        Returns the requests that finished in it (with steps launched ahead: the requests whose
        end the host learnt of in it)."""
        if self._may_run_ahead(only):
            return self._step_ahead()
        early = self.finish_steps()
        plan = self.scheduler.schedule(only)
        if not plan:
            return early
        entries = [
            StepEntry(p.request.slot, p.request.tokens[p.start : p.start + p.num_tokens],
                      [p.num_tokens - 1] if p.samples else [])
            for p in plan
        ]
        logits = self.runner.step(entries, borrow=True)
        samplers = [p.request for p in plan if p.samples]
        picks = self.runner.last_picks
        if picks is not None and len(samplers) == len(plan) and all(r.temperature <= 0.0 for r in samplers):
            sampled = picks.tolist()  # the graph picked the first maxima itself
        else:
            sampled = self.sampler.pick(logits, samplers)
        done = early + self.scheduler.update(plan, sampled)
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
        self.finish_steps()

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, eos_token_id: int = -1,
                 temperature: float = 0.0, seed: int = 0) -> List[List[int]]:
        """New token ids of every prompt (EOS included when it ended the request)."""
        reqs = [self.add_request(p, max_new_tokens, eos_token_id, temperature, seed) for p in prompts]
        self.run_until_finished()
        return [list(r.generated) for r in reqs]
