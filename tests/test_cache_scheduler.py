"""The cache manager's bookkeeping and the scheduler's decisions (CPU)."""
import random

import pytest
import torch

from litellmengine_amd.cache import CacheManager, OutOfPages, PagePool
from litellmengine_amd.config import Qwen3Config, get_architecture
from litellmengine_amd.engine import Scheduler
from litellmengine_amd.engine.request import RequestStatus
from tests.tiny import CONFIGS


def structure(which):
    cfg = Qwen3Config.from_dict(CONFIGS[which])
    return get_architecture(cfg.architecture).build(cfg)


def manager(which="A", page_size=4, num_pages=8, max_requests=4, **kw):
    return CacheManager(structure(which), page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                        dtype=torch.float32, device="cpu", **kw)


# -- page pool: pinned by tests/test_block_table_manager.cpp:279-326 -------------------
def test_pool_order_and_lifo_reuse():
    pool = PagePool(6)
    assert pool.allocate(3) == [0, 1, 2]
    assert pool.allocate(1) == [3]
    pool.release([0, 1])  # given back in table order: the last one is used again first
    assert pool.allocate(1) == [1]
    assert pool.allocate(1) == [0]
    assert pool.num_free == 2


def test_pool_all_or_nothing_and_double_free():
    pool = PagePool(4)
    pool.allocate(3)
    with pytest.raises(OutOfPages, match="not enough free physical blocks"):
        pool.allocate(2)
    assert pool.num_free == 1  # nothing was taken
    pool.release([2])
    with pytest.raises(ValueError, match="twice"):
        pool.release([2])
    with pytest.raises(ValueError, match="twice"):
        pool.release([1, 1])
    assert pool.num_free == 2  # the failed call changed nothing
    with pytest.raises(ValueError, match="does not exist"):
        pool.release([9])


# -- manager ---------------------------------------------------------------------------
def test_growth_address_map_and_release():
    m = manager(page_size=4, num_pages=8)
    assert len(m.groups) == 1 and m.groups[0].kv.shape == (2, 8 + 1, 2, 2, 4, 16)  # one spare page that is never handed out
    a, b = m.admit(), m.admit()
    m.extend(a, 5)
    m.extend(b, 3)
    m.extend(a, 9)
    g = m.groups[0]
    assert g.tables[a] == [0, 1, 3] and g.tables[b] == [2]
    # token slot = table[pos / P] * P + pos % P  (src/engine/block_table_manager.cpp:91-122)
    assert g.token_slot(a, 9 - 1) == 3 * 4 + 0 and g.token_slot(a, 6) == 1 * 4 + 2
    with pytest.raises(IndexError):
        g.token_slot(b, 4)  # an unallocated logical page
    m.commit(a, 9)
    assert m.length(a) == 9
    m.release(a)
    assert g.pool.num_free == 7 and not m.is_live(a)
    with pytest.raises(ValueError, match="not in use"):
        m.release(a)
    c = m.admit()
    assert c == a and m.length(c) == 0  # slot and pages are used again
    m.extend(c, 1)
    assert g.tables[c] == [3]  # last page given back first


def test_extend_is_all_or_nothing_across_requests():
    m = manager(page_size=4, num_pages=4)
    a, b = m.admit(), m.admit()
    m.extend(a, 8)
    before = [list(t) for t in m.groups[0].tables]
    assert not m.can_extend([(a, 12), (b, 8)])
    with pytest.raises(OutOfPages):
        m.extend_many([(a, 12), (b, 8)])
    assert [list(t) for t in m.groups[0].tables] == before and m.groups[0].pool.num_free == 2
    m.extend_many([(a, 12), (b, 4)])
    assert m.groups[0].pool.num_free == 0
    with pytest.raises(ValueError, match="shrink"):
        m.commit(a, 12) or m.extend(a, 3)


def test_request_page_limit():
    m = manager(page_size=4, num_pages=8, max_pages_per_request=2)
    a = m.admit()
    assert m.can_extend([(a, 8)]) and not m.can_extend([(a, 9)])


def test_device_table_gets_only_new_entries():
    m = manager(page_size=4, num_pages=8)
    a = m.admit()
    m.extend(a, 6)
    ups = m.take_table_updates()
    assert ups == [(0, [a * 8 + 0, a * 8 + 1], [0, 1])]
    assert m.take_table_updates() == []
    m.extend(a, 7)
    assert m.take_table_updates() == []
    m.extend(a, 9)
    assert m.take_table_updates() == [(0, [a * 8 + 2], [2])]


def test_window_group_gives_pages_back_as_the_window_passes():
    m = manager("C", page_size=4, num_pages=16)
    assert len(m.groups) == 2
    win = next(g for g in m.groups if g.window == 20)
    full = next(g for g in m.groups if g.window is None)
    assert win.cache_ids == [0, 2, 3] and full.cache_ids == [1]
    a = m.admit()
    m.extend(a, 30)
    m.commit(a, 30)
    # next query is position 30 and sees keys >= 11: pages 0 and 1 (keys 0..7) are passed
    assert win.tables[a][:3] == [-1, -1, 2] and win.pool.num_held == 6
    assert full.pool.num_held == 8
    with pytest.raises(IndexError):
        win.token_slot(a, 7)
    m.extend(a, 31)
    m.commit(a, 31)  # sees keys >= 12: page 2 (keys 8..11) is passed too
    assert win.pool.num_held == 5 and win.tables[a][:4] == [-1, -1, -1, 3]
    m.extend(a, 33)
    m.commit(a, 33)  # sees keys >= 14: page 3 (12..15) is still needed; one new page for position 32
    assert win.tables[a][:4] == [-1, -1, -1, 3] and win.pool.num_held == 6
    m.release(a)
    assert win.pool.num_held == 0 and full.pool.num_held == 0


def test_state_rows_are_zeroed_at_admission():
    from litellmengine_amd.parts import StateSpec

    model = structure("A")
    model.blocks[1].mixer.state_spec = lambda: StateSpec((3,), torch.float32)
    m = CacheManager(model, page_size=4, num_pages=4, max_requests=2, dtype=torch.float32, device="cpu")
    # a row for each request slot and a spare one, which the rows that pad a graph's batch name
    assert m.layer(0).state is None and m.layer(1).state.shape == (2 + 1, 3) and m.pad_slot == 2
    a = m.admit()
    m.layer(1).state[a] += 5.0
    m.release(a)
    assert m.admit() == a and float(m.layer(1).state[a].abs().sum()) == 0.0


def test_padding_rows_stay_inside_every_per_slot_tensor():
    """A decode batch filled up to a graph's size names the spare slot for its padding rows:
    inside the block table of every group and inside every mixer's state rows."""
    from litellmengine_amd.engine.batch import StepEntry, layout_step, views_of
    from litellmengine_amd.parts import StateSpec

    model = structure("C")
    model.blocks[0].mixer.state_spec = lambda: StateSpec((5,), torch.float32)
    m = CacheManager(model, page_size=4, num_pages=8, max_requests=3, dtype=torch.float32, device="cpu")
    slots = [m.admit() for _ in range(3)]
    m.extend_many([(s, 1) for s in slots])
    for pad_to, entries in ((8, [StepEntry(s, [1], [0]) for s in slots]), (4, [])):  # the second: a warm-up batch
        layout = layout_step(entries, m, all_rows=True, pad_to=pad_to)
        v = views_of(layout.host, layout.sizes())
        seq_slots, kv_lens = v[3], v[5]
        assert layout.num_seqs == pad_to and int(seq_slots.max()) == m.pad_slot
        assert all(int(seq_slots.max()) < g.block_table.shape[0] for g in m.groups)
        assert all(int(seq_slots.max()) < state.shape[0] for state in m.states.values())
        pads = seq_slots == m.pad_slot
        assert int(pads.sum()) == pad_to - len(entries) and bool((kv_lens[pads] == 1).all())
        for g, mapping in zip(m.groups, v[7:]):
            assert bool((mapping[len(entries):] == -1).all())  # nothing is written for them
            assert int(g.block_table[m.pad_slot, 0]) == g.pool.num_pages  # the page that is never handed out


@pytest.mark.parametrize("which,seed", [("A", 0), ("A", 1), ("C", 2), ("C", 3)])
def test_random_orders_lose_no_page(which, seed):
    """Admit, grow, commit and release in random order: every page is either
    free or in exactly one live table, and in the end all are free."""
    rng = random.Random(seed)
    m = manager(which, page_size=4, num_pages=12, max_requests=5)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.num_free_slots:
            live[m.admit()] = 0
        elif op < 0.8 and live:
            slot = rng.choice(list(live))
            new_len = live[slot] + rng.randint(1, 9)
            if m.can_extend([(slot, new_len)]):
                if rng.random() < 0.3:
                    # a step that does not happen after all: grown with another request, then given back
                    other = rng.choice(list(live))
                    wants = [(slot, new_len)] + ([(other, live[other] + 5)] if other != slot else [])
                    if m.can_extend(wants):
                        stacks = [(g.pool.num_free, [g.tables[s] for s in live]) for g in m.groups]
                        m.extend_many(wants)
                        m.shrink_many([(s, live[s]) for s, _ in wants])
                        assert [(g.pool.num_free, [g.tables[s] for s in live]) for g in m.groups] == stacks
                        again = [g.pool.num_free for g in m.groups]
                        m.extend_many(wants)  # ... and the pages come in the same order when it is tried again
                        took = [[g.tables[s] for s, _ in wants] for g in m.groups]
                        m.shrink_many([(s, live[s]) for s, _ in wants])
                        m.extend_many(wants)
                        assert [[g.tables[s] for s, _ in wants] for g in m.groups] == took
                        m.shrink_many([(s, live[s]) for s, _ in wants])
                        assert [g.pool.num_free for g in m.groups] == again
                m.extend(slot, new_len)
                m.commit(slot, new_len)
                live[slot] = new_len
            else:
                with pytest.raises(OutOfPages):
                    m.extend(slot, new_len)
        elif live:
            slot = rng.choice(list(live))
            m.release(slot)
            del live[slot]
        for g in m.groups:
            held = [p for s in range(5) for p in g.held_pages(s)]
            assert len(held) == len(set(held)), "a page is held twice"
            assert len(held) == g.pool.num_held, "a page is lost"
            assert all(g.pool.is_held(p) for p in held)
            for s, n in live.items():
                lo = 0 if g.window is None else max(0, n - g.window + 1)
                for pos in range(lo, n):
                    g.token_slot(s, pos)  # every key a later query may see has a page
    for slot in list(live):
        m.release(slot)
    assert all(g.pool.num_free == 12 for g in m.groups)


# -- scheduler ----------------------------------------------------------------------------
def drive(s, tokens_of=lambda r: 7):
    """Run the scheduler with a fake model (every sampled token is 7) and the
    real cache bookkeeping; returns the plans as [(request id, start, n, samples)]."""
    log = []
    while s.has_work():
        plan = s.schedule()
        assert plan, "the scheduler must make progress"
        s.cache.extend_many([(p.request.slot, p.start + p.num_tokens) for p in plan])
        for p in plan:
            s.cache.commit(p.request.slot, p.start + p.num_tokens)
        s.update(plan, [tokens_of(p.request) for p in plan if p.samples])
        log.append([(p.request.request_id, p.start, p.num_tokens, p.samples) for p in plan])
    return log


def test_portions_under_a_token_budget():
    s = Scheduler(manager(page_size=4, num_pages=32), max_tokens_per_step=16, prefill_chunk=10)
    a = s.add_request(list(range(23)), 3)
    b = s.add_request(list(range(5)), 2)
    log = drive(s)
    assert log[0] == [(0, 0, 10, False), (1, 0, 5, True)]  # chunk limit, then the next request in the rest
    assert log[1] == [(1, 5, 1, True), (0, 10, 10, False)]  # decoding rows first
    assert log[2] == [(0, 20, 3, True)]
    assert log[3] == [(0, 23, 1, True)] and log[4] == [(0, 24, 1, True)]
    assert a.generated == [7, 7, 7] and b.generated == [7, 7]
    assert a.cached_len == 25 and len(a.tokens) == 26  # the last token drawn is never run
    assert all(g.pool.num_held == 0 for g in s.cache.groups)


def test_budget_cuts_a_prompt_anywhere():
    s = Scheduler(manager(page_size=4, num_pages=32), max_tokens_per_step=7)
    s.add_request(list(range(9)), 1)
    s.add_request(list(range(9)), 1)
    log = drive(s)
    assert log[0] == [(0, 0, 7, False)]
    assert log[1] == [(0, 7, 2, True), (1, 0, 5, False)]
    assert log[2] == [(1, 5, 4, True)]


def test_finish_on_eos_and_zero_new_tokens():
    s = Scheduler(manager(page_size=4, num_pages=8))
    a = s.add_request([1, 2, 3], 5, eos_token_id=7)
    z = s.add_request([1], 0)
    assert z.status is RequestStatus.FINISHED and not z.generated  # src/engine/request_manager.cpp:30-34
    drive(s)
    assert a.generated == [7] and a.finished  # eos is appended, then the request ends (:140-148)
    with pytest.raises(ValueError, match="non-empty"):
        s.add_request([], 3)
    with pytest.raises(ValueError, match=">= 0"):
        s.add_request([1], -1)


def test_request_that_can_never_fit_is_refused():
    s = Scheduler(manager(page_size=4, num_pages=4))
    s.add_request(list(range(10)), 7)  # 16 positions cached at most: fits exactly
    with pytest.raises(ValueError, match="needs 5 pages"):
        s.add_request(list(range(10)), 8)


def test_waiting_request_is_admitted_only_when_its_pages_are_free():
    s = Scheduler(manager(page_size=4, num_pages=4), max_tokens_per_step=64)
    a = s.add_request(list(range(9)), 2)  # 3 pages
    b = s.add_request(list(range(6)), 2)  # 2 pages: must wait
    plan = s.schedule()
    assert [p.request.request_id for p in plan] == [0]
    assert b.status is RequestStatus.WAITING and s.cache.num_free_slots == 3
    log = drive(s)
    # b starts in the step after a finished and freed its pages
    first_b = next(i for i, step in enumerate(log) if any(r == 1 for r, *_ in step))
    last_a = max(i for i, step in enumerate(log) if any(r == 0 for r, *_ in step))
    assert first_b == last_a + 1
    assert s.num_preemptions == 0


def test_out_of_pages_preempts_the_youngest_and_recomputes_it():
    s = Scheduler(manager(page_size=4, num_pages=4), max_tokens_per_step=64)
    a = s.add_request(list(range(7)), 6)  # grows to 12 cached: 3 pages
    b = s.add_request(list(range(4)), 8)  # grows to 11 cached: 3 pages; together 6 > 4
    log = drive(s)
    assert s.num_preemptions >= 1 and b.preemptions >= 1 and a.preemptions == 0
    assert a.generated == [7] * 6 and b.generated == [7] * 8
    # after a preemption b is recomputed from position 0 with what it had generated
    restarts = [step for step in log for (r, start, n, _) in step if r == 1 and start == 0]
    assert len(restarts) == 1 + b.preemptions
    redo = [(start, n) for step in log for (r, start, n, _) in step if r == 1 and start == 0][-1]
    assert redo[1] > 4  # prompt plus generated tokens in one portion
    assert all(g.pool.num_held == 0 for g in s.cache.groups) and s.cache.num_free_slots == 4


def test_no_admission_in_a_step_that_preempted():
    s = Scheduler(manager(page_size=4, num_pages=3), max_tokens_per_step=64)
    s.add_request(list(range(4)), 6)
    s.add_request(list(range(4)), 6)
    seen_preempt = False
    while s.has_work():
        before = s.num_preemptions
        waiting_before = len(s.waiting)
        plan = s.schedule()
        if s.num_preemptions > before:
            seen_preempt = True
            assert len(s.waiting) == waiting_before + (s.num_preemptions - before)
        s.cache.extend_many([(p.request.slot, p.start + p.num_tokens) for p in plan])
        for p in plan:
            s.cache.commit(p.request.slot, p.start + p.num_tokens)
        s.update(plan, [7 for p in plan if p.samples])
    assert seen_preempt


def run_plan(s, plan, token=7):
    s.cache.extend_many([(p.request.slot, p.start + p.num_tokens) for p in plan])
    for p in plan:
        s.cache.commit(p.request.slot, p.start + p.num_tokens)
    return s.update(plan, [token for p in plan if p.samples])


def test_decoders_take_turns_when_the_budget_is_below_their_number():
    s = Scheduler(manager(page_size=4, num_pages=32, max_requests=5), max_tokens_per_step=16)
    reqs = [s.add_request([1, 2], 5) for _ in range(5)]
    run_plan(s, s.schedule())  # all prompts in one step
    assert all(r.extend_len == 1 for r in reqs)
    s.max_tokens_per_step = 2
    served = []
    for _ in range(10):
        plan = s.schedule()
        assert len(plan) == 2 and all(p.num_tokens == 1 for p in plan)
        served.append(sorted(p.request.request_id for p in plan))
        run_plan(s, plan)
        if not s.has_work():
            break
    # nobody waits for the head of the list to finish: within any three steps everyone ran
    ids = [r.request_id for r in reqs]
    for i in range(len(served) - 2):
        window = set(served[i] + served[i + 1] + served[i + 2])
        assert window >= {r for r in ids if not s.requests[r].finished or r in window}
    counts = {r: sum(r in step for step in served[:5]) for r in ids}
    assert max(counts.values()) - min(counts.values()) <= 1, counts


def test_prompts_are_not_starved_by_decoders_that_fill_the_budget():
    """Six decoders and a budget of four tokens: a request that arrives with a prompt of ten
    tokens is admitted at once and gets a share of every step, beside decoders that still take
    turns; and what is released or preempted leaves nothing behind in the turn-taking record."""
    s = Scheduler(manager(page_size=4, num_pages=64, max_requests=8), max_tokens_per_step=32)
    decoders = [s.add_request([1, 2, 3], 30) for _ in range(6)]
    run_plan(s, s.schedule())
    assert all(r.extend_len == 1 for r in decoders)
    s.max_tokens_per_step = 4
    late = s.add_request(list(range(10)), 2)
    seen = []
    for step in range(16):
        plan = s.schedule()
        assert sum(p.num_tokens for p in plan) <= 4
        seen.append([(p.request.request_id, p.num_tokens) for p in plan])
        run_plan(s, plan)
        if late.finished:
            break
    assert late.finished and step <= 12, seen  # ten steps for its prompt (a token each), two decoding
    assert any(rid == late.request_id for rid, _ in seen[0]), "a share of the first step already"
    assert all(sum(1 for rid, _ in plan if rid != late.request_id) >= 2 for plan in seen)  # decoders go on
    # nothing of a released or a preempted request stays in the record
    victim = decoders[0]
    s.release_request(victim.request_id)
    assert victim.request_id not in s._last_served
    s._preempt(decoders[1])
    assert decoders[1].request_id not in s._last_served and decoders[1].status is RequestStatus.WAITING


def test_a_request_that_does_not_fit_leaves_parked_sessions_alone():
    s = Scheduler(manager(page_size=4, num_pages=8, max_requests=4), max_tokens_per_step=64)
    a = s.add_request(list(range(7)), 2, keep_session=True)   # parks with 2 pages
    b = s.add_request(list(range(5)), 8)                      # runs on: up to 3 pages
    while not a.finished:
        run_plan(s, s.schedule())
    assert s.parked == [a] and not b.finished
    big = s.add_request(list(range(27)), 1)  # 7 pages: free + parked pages are too few while b runs
    held_a = s.cache.pages_held(a.slot)
    plan = s.schedule()
    assert [p.request for p in plan] == [b]
    assert s.num_evictions == 0 and s.parked == [a] and s.cache.pages_held(a.slot) == held_a
    assert big.status is RequestStatus.WAITING
    while not b.finished:
        run_plan(s, s.schedule())
    # now evicting the session makes room: it is evicted, and only now
    while not big.finished:
        run_plan(s, s.schedule())
    assert s.num_evictions == 1 and a.slot == -1 and a.cached_len == 0


def test_the_only_running_request_that_cannot_fit_raises_without_evicting():
    s = Scheduler(manager("C", page_size=4, num_pages=6, max_requests=3), max_tokens_per_step=64, prefill_chunk=4)
    a = s.add_request(list(range(6)), 1, keep_session=True)
    while not a.finished:
        run_plan(s, s.schedule())
    assert s.parked == [a]
    held = s.cache.pages_held(a.slot)
    # fits the group with a window as far as add_request can tell, never the whole-cache group's pool:
    # refused at once, the parked session untouched
    with pytest.raises(ValueError, match="pages"):
        s.add_request(list(range(40)), 1)
    assert s.parked == [a] and s.cache.pages_held(a.slot) == held and s.num_evictions == 0


def test_only_restricts_the_step_but_not_the_choice_of_the_victim():
    s = Scheduler(manager(page_size=4, num_pages=4), max_tokens_per_step=64)
    a = s.add_request(list(range(7)), 10)
    b = s.add_request(list(range(4)), 8)
    run_plan(s, s.schedule())  # both prompts: 2 + 1 pages of 4
    assert a.slot >= 0 and b.slot >= 0
    while s.cache.can_extend([(a.slot, a.cached_len + 1)]):
        run_plan(s, s.schedule(only=[a.request_id]))
        assert b.status is RequestStatus.RUNNING
    plan = s.schedule(only=[a.request_id])  # a needs a page; b, the youngest, gives its pages although it does not run
    assert [p.request for p in plan] == [a] and b.status is RequestStatus.WAITING and b.preemptions == 1


# -- the step layout (csrc/host.cpp) ------------------------------------------------------
def test_step_layout_matches_the_address_map():
    """Token ids, positions, requests, lengths, wanted rows and every token's page slot in
    every group, as one flat array: against the same computed here from the tables."""
    from litellmengine_amd.engine.batch import StepEntry, layout_step

    m = manager("C", page_size=4, num_pages=16, max_requests=4)  # two groups: a window and all keys
    a, b, c = m.admit(), m.admit(), m.admit()
    m.extend(a, 7)
    m.commit(a, 7)
    m.extend(b, 30)
    m.commit(b, 30)  # the window group has given pages of b back
    entries = [StepEntry(b, [9, 8, 7], [2]), StepEntry(a, [1], []), StepEntry(c, [4, 5, 6, 7, 8], [0, 4])]
    m.extend_many([(b, 33), (a, 8), (c, 5)])
    lay = layout_step(entries, m, vocab_size=10)
    N, S, R, G = 9, 3, 3, len(m.groups)
    assert (lay.num_tokens, lay.num_seqs, lay.num_logit_rows, lay.num_groups, lay.max_kv_len) == (N, S, R, G, 33)
    flat = lay.host.tolist()
    assert len(flat) == 3 * N + 3 * S + 1 + R + G * N
    want = [9, 8, 7, 1, 4, 5, 6, 7, 8] + [30, 31, 32, 7, 0, 1, 2, 3, 4] + [0, 0, 0, 1, 2, 2, 2, 2, 2]
    want += [b, a, c] + [0, 3, 4, 9] + [33, 8, 5] + [2, 4, 8]
    for g in m.groups:
        want += [g.token_slot(s, p) for s, p in [(b, 30), (b, 31), (b, 32), (a, 7)] + [(c, i) for i in range(5)]]
    assert flat == want
    assert [(q.slot, q.q_start, q.q_len, q.past_len) for q in lay.seqs] == [(b, 0, 3, 30), (a, 3, 1, 7), (c, 4, 5, 0)]
    every = layout_step(entries, m, all_rows=True)
    assert every.host.tolist()[3 * N + 3 * S + 1:3 * N + 3 * S + 1 + N] == list(range(N))


def test_step_layout_refuses_bad_tokens_and_missing_pages():
    from litellmengine_amd.engine.batch import StepEntry, layout_step

    m = manager(page_size=4, num_pages=8)
    a = m.admit()
    m.extend(a, 4)
    with pytest.raises(ValueError, match="token id 300 outside"):
        layout_step([StepEntry(a, [1, 300], [])], m, vocab_size=256)
    with pytest.raises(ValueError, match="token id -1 outside"):
        layout_step([StepEntry(a, [-1], [])], m, vocab_size=256)
    with pytest.raises(IndexError, match="has no page"):
        layout_step([StepEntry(a, [1, 2, 3, 4, 5], [])], m, vocab_size=256)  # the fifth position was never extended to
