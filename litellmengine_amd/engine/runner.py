"""The step function: one batch of (request, its next tokens) through the model.

The reference's nearest piece is `forward_uncached_chunk_and_sample`
(src/engine/paged_generate_engine.cpp:475-598) for one request and
`decode_batch` (:182-341) for single tokens of several; both return logits of
every row.  `ModelRunner.step` takes any mix, runs only the tokens it is given
from the cache that earlier steps left, and returns float32 logits at the
wanted places only.  Order inside a step as in the reference: the step's K/V
are written to their pages first, then every token attends through the block
table (src/model/qwen3.cpp:464-481 before :498-557).

Steps that hold single tokens only (decoding) are launch-bound, so they are
captured into HIP graphs and replayed: the step's integer arrays are copied
into the graph's fixed buffer, the block tables are updated outside the graph,
and the same kernels run.  There is one graph per (batch bucket, context
bucket): a batch is filled up to the next of a few sizes with rows that stand
for nobody (they read one key of a page that is never written, write nothing,
and their logits are dropped), so a batch whose requests finish one by one
walks through a handful of graphs instead of one per size; the graphs used
least recently are dropped beyond MAX_GRAPHS.  Models whose mixers need the
host-side view of the batch are stepped without graphs.
"""
from __future__ import annotations

import collections
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache import CacheManager
from . import batch as _batch
from .batch import StepEntry, StepLayout, StepState, apply_table_updates, build_step, layout_step, state_on


class _DecodeGraph:
    def __init__(self, graph, buf, logits, sampled=None):
        self.graph = graph
        self.buf = buf
        self.logits = logits
        self.sampled = sampled  # int32 [batch bucket]: the first maximum of every row, picked inside the graph


class PendingTokens:
    """The tokens that a step picked, on their way from the device: `wait()` returns them once
    the step has run (one id per entry, in the entries' order)."""

    def __init__(self, host: torch.Tensor, count: int, event=None):
        self._host, self._count, self._event = host, count, event

    def wait(self) -> List[int]:
        if self._event is not None:
            self._event.synchronize()
        return self._host[: self._count].tolist()


class ModelRunner:
    MAX_GRAPH_BATCH = 256
    MIN_CONTEXT_BUCKET = 256
    BATCH_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 192, 256)
    MAX_GRAPHS = 32  # each keeps float32 logits [batch bucket, vocabulary] alive

    def __init__(self, model, cache: CacheManager, use_graphs: Optional[bool] = None, pick_tokens: bool = False):
        """`pick_tokens`: decode graphs also pick every row's first maximum (the greedy token) and
        leave it on the device for the request's next step, so that a caller may launch that step
        before it has read this one's tokens (step_ahead)."""
        self.model = model
        self.cache = cache
        self.device = cache.device
        self.vocab_size = model.vocab_size
        self.last_step: Optional[StepState] = None
        self.pick_tokens = bool(pick_tokens)
        # by request slot (and the spare one of padding rows): the token picked for it last
        self.token_feedback = torch.zeros(cache.max_requests + 1, dtype=torch.int32, device=self.device)
        self.last_picks: Optional[torch.Tensor] = None  # the picks of the last step(), where a graph made them
        self._results = [None, None, None]  # pinned host buffers that picks are copied to, in turn
        self._result_turn = 0
        graph_safe = all(getattr(b.mixer, "graph_safe", False) for b in model.blocks)
        if use_graphs is None:
            use_graphs = self.device.type == "cuda"
        self.use_graphs = bool(use_graphs) and graph_safe and self.device.type == "cuda"
        self._graphs: "collections.OrderedDict[Tuple[int, int], _DecodeGraph]" = collections.OrderedDict()
        self._graph_pool = None
        self.num_captures = 0
        self.num_graph_steps = 0  # steps that ran as a graph (decode steps), captures included
        if self.use_graphs:
            self._first_graph_of_the_process(self.device)

    _graphs_woken = set()

    @classmethod
    def _first_graph_of_the_process(cls, device) -> None:
        """Capture and replay a toy graph once per process and device, when the first runner is
        made.  Measured on MI355X: for about 115 ms after the first graph that a process
        captures, every launch is some 5 % slower (decode steps of 4.47 ms for the first 25
        replays at batch 8, 3.57 ms for the first 31 at batch 1, then 4.27 and 3.41; the clocks
        are up all the while, a pause before the capture changes nothing, a pause after it, or
        a graph captured earlier, takes the phase away, and no later graph shows it).  Paid
        here, it is over before the first request decodes."""
        key = torch.device(device).index or 0
        if key in cls._graphs_woken:
            return
        cls._graphs_woken.add(key)
        x = torch.zeros(64, device=device)
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            x.add_(1.0)
        graph.replay()
        torch.cuda.synchronize(device)

    # requests ------------------------------------------------------------------
    def admit(self) -> int:
        return self.cache.admit()

    def release(self, slot: int) -> None:
        self.cache.release(slot)

    # one step -----------------------------------------------------------------------
    def check(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise ValueError("a step needs at least one entry")
        slots = [e.slot for e in entries]
        if len(set(slots)) != len(slots):
            twice = next(s for i, s in enumerate(slots) if s in slots[:i])
            raise ValueError(f"request slot {twice} appears twice in one step")
        self.cache.lengths_of(slots)  # (every slot is in use)
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise ValueError("an entry needs at least one token")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"wanted place {w} outside the entry's {n} tokens")

    def check_tokens(self, entries: Sequence[StepEntry], allow_deferred: bool = False) -> None:
        """Token ids outside the vocabulary are refused before anything is changed
        (src/layers/embedding.cu:75-87).  min and max run in C.  `allow_deferred`: -1 stands
        for the token that the device still holds for the request (step_ahead)."""
        low = -1 if allow_deferred else 0
        for e in entries:
            if min(e.tokens) < low or max(e.tokens) >= self.vocab_size:
                bad = next(t for t in e.tokens if not low <= int(t) < self.vocab_size)
                raise ValueError(f"token id {bad} outside [0, {self.vocab_size})")

    def step(self, entries: Sequence[StepEntry], borrow: bool = False) -> torch.Tensor:
        """Run the entries as one batch.  Returns float32 logits [wanted, vocab] in
        the order of the entries and of their `want`.  Raises cache.OutOfPages,
        with nothing changed, when the pages for this step are not there.  With
        `borrow` the result may alias memory that the next step overwrites.
        If the model raises (a kernel that refuses its operands), the step did not
        happen: the pages it took go back and no length moves, so the same entries
        can be stepped again (what a mixer keeps as state of its own is its own to mend)."""
        logits, _ = self._run(entries, borrow, ahead=False)
        return logits

    def step_ahead(self, entries: Sequence[StepEntry]) -> PendingTokens:
        """A decode step whose greedy picks are not waited for: every entry is one token wanting
        its logits' first maximum, and a token id of -1 stands for the pick that the step before
        made for the same request (it never left the device).  The step is put on the stream and
        the picks follow it to the host; `wait()` of what is returned hands them out.  The cache's
        lengths move at once: the next step may be laid out, and launched, before this one has run."""
        for e in entries:
            if len(e.tokens) != 1 or list(e.want) != [0]:
                raise ValueError("step_ahead takes single tokens whose logits are wanted")
        _, picks = self._run(entries, True, ahead=True)
        n = len(entries)
        if self.device.type != "cuda":
            return PendingTokens(picks[:n].clone(), n)
        turn = self._result_turn = (self._result_turn + 1) % len(self._results)
        host = self._results[turn]
        if host is None or host.numel() < n:
            host = self._results[turn] = torch.empty(max(256, n), dtype=torch.int32, pin_memory=True)
        host[:n].copy_(picks[:n], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return PendingTokens(host, n, event)

    def _run(self, entries: Sequence[StepEntry], borrow: bool, ahead: bool):
        """(logits, picks): the step itself; `picks` (int32 on the device, one per entry) where the
        step picked tokens (a graph that does, or `ahead`)."""
        self.check(entries)
        cache = self.cache
        before = [(e.slot, cache.length(e.slot)) for e in entries]
        wants = [(slot, length + len(e.tokens)) for (slot, length), e in zip(before, entries)]
        self.check_tokens(entries, allow_deferred=ahead)
        cache.extend_many(wants)
        picks = None
        try:
            if self.use_graphs and len(entries) <= self.MAX_GRAPH_BATCH and all(len(e.tokens) == 1 for e in entries):
                logits, picks = self._graph_step(entries, borrow, ahead)
            else:
                state = build_step(entries, cache, self.device, self.vocab_size, all_rows=ahead,
                                   token_feedback=self.token_feedback if ahead else None)
                self.last_step = state
                logits = self.model.forward(state, cache)
                if ahead:
                    picks = self.model.ctx.ops.argmax(logits, scatter=(self.token_feedback, state.seq_slots))
        except BaseException:
            cache.shrink_many(before)
            raise
        cache.commit_many(wants)
        self.last_picks = picks
        return logits, picks

    # decoding through a captured graph ---------------------------------------------------
    def _graph_step(self, entries: Sequence[StepEntry], borrow: bool, ahead: bool = False):
        cache = self.cache
        self.num_graph_steps += 1
        if ahead and not self.pick_tokens:
            raise RuntimeError("step_ahead needs a runner that picks tokens inside its graphs (pick_tokens)")
        batch = next(b for b in self.BATCH_BUCKETS if b >= len(entries))
        layout = layout_step(entries, cache, all_rows=True, vocab_size=self.vocab_size, device=self.device,
                             pad_to=batch, with_seqs=False, allow_deferred=ahead)
        apply_table_updates(cache, self.device)
        bucket = self.MIN_CONTEXT_BUCKET
        while bucket < layout.max_kv_len:
            bucket *= 2
        host = layout.host
        key = (batch, bucket)
        g = self._graphs.get(key)
        if g is None:
            while len(self._graphs) >= self.MAX_GRAPHS:
                self._graphs.popitem(last=False)  # the one used least recently
            g = self._capture(layout, host, bucket)
            self._graphs[key] = g
            self.num_captures += 1
        else:
            self._graphs.move_to_end(key)
            g.buf.copy_(host, non_blocking=True)  # (behind what is on the stream already, not waited for)
            _batch._staging.copy_enqueued()
        g.graph.replay()  # its kernels read the buffer that the capture saw: g.buf
        logits = g.logits
        picks = None if g.sampled is None else g.sampled[: len(entries)]
        rows = [i for i, e in enumerate(entries) if len(e.want) > 0]
        if len(rows) != len(entries):
            some = logits[torch.tensor(rows, dtype=torch.long, device=self.device)] if rows else logits[:0].clone()
            return some, None
        logits = logits[: len(entries)]
        return (logits if borrow else logits.clone()), picks

    def _capture(self, layout: StepLayout, host: torch.Tensor, bucket: int) -> _DecodeGraph:
        buf = host.to(self.device)  # (a blocking copy: the staging buffer behind `host` is free again)
        # Before a capture the same kernels run for real once (the library picks its products for these
        # sizes and takes its workspaces, kernels set themselves up: none of that may happen under
        # capture; the very first capture runs them twice).  They run on a batch of the same size
        # whose rows all stand for nobody: the cache's spare table row and page, the spare row of
        # every mixer's state, nothing written.  So no request's cache or state moves before the
        # graph's first replay, whatever the mixers keep.
        warm = layout_step([], self.cache, all_rows=True, vocab_size=self.vocab_size, device=self.device,
                           pad_to=layout.num_seqs, with_seqs=False)
        feedback = self.token_feedback if self.pick_tokens else None
        pick = lambda logits, st: self.model.ctx.ops.argmax(logits, scatter=(self.token_feedback, st.seq_slots))
        warm_state = state_on(warm.host.to(self.device), warm, self.cache, max_kv_len=bucket, with_seqs=False,
                              token_feedback=feedback)
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            for _ in range(2 if self.num_captures == 0 else 1):
                warm_logits = self.model.forward(warm_state, self.cache)
                if self.pick_tokens:
                    pick(warm_logits, warm_state)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        state = state_on(buf, layout, self.cache, max_kv_len=bucket, with_seqs=False, token_feedback=feedback)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self.model.forward(state, self.cache)
            sampled = pick(logits, state) if self.pick_tokens else None
        if self._graph_pool is None:
            self._graph_pool = graph.pool()
        return _DecodeGraph(graph, buf, logits, sampled)
