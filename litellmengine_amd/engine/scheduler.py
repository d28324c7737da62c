"""The scheduler: which tokens of which requests run in the next step.

The reference has no scheduler object: callers prefill every request alone and
whole, then loop `decode_batch` over the unfinished ones, with a pool sized for
the worst case so that pages never run out
(src/benchmark/generation_benchmark.cpp:259-315); a shortage throws from
`ensure_blocks` up to `main` (src/engine/block_table_manager.cpp:82-84).

Here, every step:
 1. requests that are decoding (one pending token) come first, the one that was
    served longest ago first (with a budget below the number of decoders they
    take turns), then requests with prompt tokens left, oldest first; each gets
    min(pending, prefill_chunk, what is left of max_tokens_per_step) tokens;
 2. if the pages for that are not there, the YOUNGEST running request is
    preempted: its pages and slot are given back, its cache is forgotten
    (cached_len = 0) and it waits at the FRONT of the queue to be recomputed
    (prompt and what it generated so far); repeated until the step fits.  No
    request is admitted in a step that preempted;
 3. otherwise waiting requests are admitted in order while a slot, budget and
    the pages for their first portion are there.
A request that could never fit (its last cached position needs more pages than
a group has, or than a request may hold) is refused when it is added.  Finished
requests give their pages back at once, unless they were added as a session
(`keep_session`): a finished session is PARKED with its slot and pages until
`append_input_tokens` continues it (only the new tokens are run then, in
portions like any prompt; the reference feeds them one by one,
src/engine/paged_generate_engine.cpp:133-141) or `release_request` ends it.
Parked sessions come before running requests when pages run out: the one
parked longest loses its cache first (it is recomputed whole if it is ever
continued).  A waiting request takes a parked session's cache only if that
makes it fit: when the free pages and those of all parked sessions together
are too few, nothing is evicted and the request goes on waiting.
"""
from __future__ import annotations

import collections
from typing import Deque, Dict, List, NamedTuple, Optional, Sequence

from ..cache import CacheManager, OutOfPages
from .request import Request, RequestStatus


class Portion(NamedTuple):
    """`num_tokens` tokens of `request` from its `cached_len` on; `samples` when
    the portion reaches the end of what the request has, so a token is drawn."""

    request: Request
    start: int
    num_tokens: int
    samples: bool


class Scheduler:
    def __init__(self, cache: CacheManager, max_tokens_per_step: int = 2048, prefill_chunk: Optional[int] = None):
        if max_tokens_per_step <= 0:
            raise ValueError("max_tokens_per_step must be positive")
        if prefill_chunk is not None and prefill_chunk <= 0:
            raise ValueError("prefill_chunk must be positive")
        self.cache = cache
        self.max_tokens_per_step = max_tokens_per_step
        self.prefill_chunk = prefill_chunk or max_tokens_per_step
        self.waiting: Deque[Request] = collections.deque()
        self.running: List[Request] = []
        self.requests: Dict[int, Request] = {}
        self.parked: List[Request] = []  # finished sessions that still hold their cache, oldest first
        self._next_id = 0
        self._admissions = 0
        self.num_preemptions = 0
        self.num_evictions = 0  # parked sessions whose cache was taken
        self._serve_clock = 0
        self._last_served: Dict[int, int] = {}  # request id -> when tokens of it last ran (ticks of the clock)

    # -- adding ---------------------------------------------------------------------
    def add_request(self, prompt_ids: Sequence[int], max_new_tokens: int, eos_token_id: int = -1,
                    temperature: float = 0.0, seed: int = 0, keep_session: bool = False) -> Request:
        """src/engine/paged_generate_engine.cpp:57-79: a prompt must not be empty,
        max_new_tokens >= 0; 0 finishes at once."""
        if len(prompt_ids) == 0:
            raise ValueError("a request needs a non-empty prompt")
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        if temperature < 0:
            raise ValueError("temperature must be >= 0")
        self._check_fits(len(prompt_ids), max_new_tokens)
        req = Request(self._next_id, [int(t) for t in prompt_ids], len(prompt_ids), max_new_tokens,
                      int(eos_token_id), float(temperature), int(seed), keep_session=bool(keep_session))
        self._next_id += 1
        self.requests[req.request_id] = req
        if max_new_tokens == 0:
            req.status = RequestStatus.FINISHED
            return req
        self.waiting.append(req)
        return req

    def _check_fits(self, prompt_len: int, max_new_tokens: int) -> None:
        longest = prompt_len + max_new_tokens - 1  # the last token drawn is never cached
        for group in self.cache.groups:
            pages = group.pages_for(longest)
            if group.window is None and pages > group.pool.num_pages:
                raise ValueError(
                    f"request of {prompt_len} prompt + {max_new_tokens} new tokens needs {pages} pages, "
                    f"the cache has {group.pool.num_pages}"
                )
            if pages > group.max_pages_per_request:
                raise ValueError(
                    f"request needs {pages} pages, a request may hold {group.max_pages_per_request}"
                )

    def append_input_tokens(self, request_id: int, token_ids: Sequence[int], max_new_tokens: int,
                            eos_token_id: int = -1) -> Request:
        """Continue a finished request with more input (PagedGenerateEngine::append_input_tokens,
        src/engine/paged_generate_engine.cpp:81-97).  A parked session runs on from its cache;
        a request whose cache is gone waits to be recomputed from its first token."""
        r = self.requests[request_id]
        if not r.finished:
            raise RuntimeError("append_input_tokens expects a finished request")
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens must be >= 0")
        self._check_fits(len(r.tokens) + len(token_ids), max_new_tokens)
        r.append_input_tokens(token_ids, max_new_tokens, eos_token_id)
        if max_new_tokens == 0 or r.extend_len == 0:
            return r  # nothing to run: it stays finished (and parked, if it was)
        if r in self.parked:
            self.parked.remove(r)
            r.status = RequestStatus.RUNNING
            self.running.append(r)
        else:
            r.cached_len = 0
            r.status = RequestStatus.WAITING
            self.waiting.append(r)
        return r

    def release_request(self, request_id: int) -> None:
        """Give back whatever the request still holds and end it
        (PagedGenerateEngine::release_request, src/engine/paged_generate_engine.cpp:386-395)."""
        r = self.requests[request_id]
        if r in self.parked:
            self.parked.remove(r)
        if r in self.running:
            self.running.remove(r)
        if r in self.waiting:
            self.waiting.remove(r)
        if r.slot >= 0:
            self.cache.release(r.slot)
            r.slot = -1
        r.cached_len = 0
        r.keep_session = False
        r.status = RequestStatus.FINISHED
        self._last_served.pop(request_id, None)

    def _evict_parked(self) -> bool:
        """Take the cache of the session parked longest; False if none is parked."""
        if not self.parked:
            return False
        r = self.parked.pop(0)
        self.cache.release(r.slot)
        r.slot = -1
        r.cached_len = 0
        self.num_evictions += 1
        return True

    def _parked_pages_cover(self, short: Sequence[int]) -> bool:
        """Whether the pages of all parked sessions make up for `short` (per group: pages
        needed minus pages free)."""
        if all(x <= 0 for x in short):
            return True
        have = [0] * len(short)
        for r in self.parked:
            have = [a + b for a, b in zip(have, self.cache.pages_held(r.slot))]
        return all(x <= h for x, h in zip(short, have))

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # -- one step ---------------------------------------------------------------------
    def schedule(self, only: Optional[Sequence[int]] = None) -> List[Portion]:
        """The portions of the next step.  `only` (request ids) restricts the step to
        those requests, the way the reference's callers prefill one request alone
        or decode a chosen set (src/engine/paged_generate_engine.cpp:99-149, :182-341)."""
        budget = self.max_tokens_per_step
        chosen = None if only is None else set(only)
        mine = [r for r in self.running if (chosen is None or r.request_id in chosen) and not r.awaits_last_token]
        turn = lambda r: self._last_served.get(r.request_id, -1)
        decoding = sorted((r for r in mine if r.extend_len == 1), key=turn)
        prompts = [r for r in mine if r.extend_len > 1]
        # Decoders that alone fill the budget, step after step, would leave prompt tokens (of running
        # requests and of waiting ones) standing until they finish: then a quarter of the budget is
        # kept back from them (a budget of one token cannot be shared: decoders first).
        others = bool(prompts) or any(chosen is None or w.request_id in chosen for w in self.waiting)
        kept_back = max(1, budget // 4) if others and len(decoding) >= budget > 1 else 0
        plan: List[Portion] = []
        for r in decoding + prompts:
            left = budget - kept_back if r.extend_len == 1 else budget
            if left <= 0:
                continue
            n = min(r.extend_len, self.prefill_chunk, left)
            plan.append(Portion(r, r.cached_len, n, n == r.extend_len))
            budget -= n

        preempted = False
        while plan and not self.cache.can_extend([(p.request.slot, p.start + p.num_tokens) for p in plan]):
            if len(self.running) == 1 and not self._parked_pages_cover(
                    self.cache.shortfall([(p.request.slot, p.start + p.num_tokens) for p in plan])):
                raise OutOfPages("the only running request does not fit into the cache")  # nothing was evicted
            if self._evict_parked():
                continue
            # the youngest of ALL running requests, whether this step runs it or not (`only`)
            victim = max(self.running, key=lambda r: r.admitted_at)
            self._preempt(victim)
            preempted = True
            budget += sum(p.num_tokens for p in plan if p.request is victim)
            plan = [p for p in plan if p.request is not victim]

        while not preempted and budget > 0:
            r = next((w for w in self.waiting if chosen is None or w.request_id in chosen), None)
            if r is None:
                break
            need_slot = self.cache.num_free_slots == 0
            if need_slot and not self.parked:
                break
            n = min(r.extend_len, self.prefill_chunk, budget)
            planned = [(p.request.slot, p.start + p.num_tokens) for p in plan]
            short = [a + b for a, b in zip(self.cache.shortfall(planned), self.cache.pages_needed(None, n))]
            if not self._parked_pages_cover(short):
                # evicting every parked session would not make room: they keep their caches
                if not self.running:
                    raise OutOfPages("the first waiting request does not fit into the empty cache")
                break
            if need_slot:
                self._evict_parked()
            slot = self.cache.admit()
            wants = planned + [(slot, n)]
            while not self.cache.can_extend(wants):
                if not self._evict_parked():
                    raise RuntimeError("the pages of parked sessions were counted but are not there")
            self.waiting.remove(r)
            r.slot = slot
            r.status = RequestStatus.RUNNING
            r.admitted_at = self._admissions
            self._admissions += 1
            self.running.append(r)
            plan.append(Portion(r, 0, n, n == r.extend_len))
            budget -= n
        for p in plan:  # a clock that ticks per portion: requests of one step keep their order for the next turn
            self._serve_clock += 1
            self._last_served[p.request.request_id] = self._serve_clock
        return plan

    def _preempt(self, r: Request) -> None:
        self.cache.release(r.slot)
        self._last_served.pop(r.request_id, None)  # when it runs again it counts as newly served
        r.slot = -1
        r.cached_len = 0
        r.status = RequestStatus.WAITING
        r.preemptions += 1
        self.num_preemptions += 1
        self.running.remove(r)
        self.waiting.appendleft(r)

    def update(self, plan: Sequence[Portion], sampled: Sequence[int]) -> List[Request]:
        """After the step ran: advance the caches' lengths, append the drawn tokens
        (one per portion with `samples`, in plan order), finish and free.
        Returns the requests that finished in this step."""
        self.launched(plan)
        return self.resolved(plan, sampled)

    def launched(self, plan: Sequence[Portion]) -> None:
        """The step of `plan` is on its way: its tokens count as cached."""
        for p in plan:
            p.request.mark_forward_done(p.num_tokens)

    def resolved(self, plan: Sequence[Portion], sampled: Sequence[int]) -> List[Request]:
        """The tokens that the step of `plan` drew are known (one per portion with `samples`, in
        plan order): append them, finish and free.  A request that has finished or been released
        since the step was launched (it ran one token past its end: the host learnt of the end a
        step late) takes no token any more.  Returns the requests that finished."""
        done: List[Request] = []
        it = iter(sampled)
        for p in plan:
            if not p.samples:
                continue
            r, token = p.request, next(it)
            if r.status is not RequestStatus.RUNNING:
                continue
            r.pending = 0
            r.append_token(token)
            if r.finished:
                self.running.remove(r)
                self._last_served.pop(r.request_id, None)
                if r.keep_session:
                    self.parked.append(r)
                else:
                    self.cache.release(r.slot)
                    r.slot = -1
                done.append(r)
        return done
