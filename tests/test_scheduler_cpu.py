"""The scheduler's decisions on the CPU, with a toy "model" that maps a history to its next token."""
import random

import pytest

from vosti_amd.cache.manager import CacheManager, GroupSpec, OutOfPages
from vosti_amd.engine.scheduler import Scheduler


def make(pages=8, page=4, seqs=4, budget=64, max_len=256, prefix=False, windows=(0,)):
    cache = CacheManager(page, [GroupSpec(w, pages) for w in windows], seqs + 1, prefix)
    return cache, Scheduler(cache, seqs, budget, max_len)


def toy_next(history):
    """A deterministic stand-in for the model: the next token depends on the whole history."""
    h = 17
    for t in history:
        h = (h * 31 + t + 1) % 1009
    return h % 97


def drive(sched, cache, histories, max_steps=10_000, on_step=None):
    """Runs plan/commit until nothing is live.  histories: {rid: prompt list}, extended in place."""
    outputs = {rid: [] for rid in histories}
    steps = 0
    while True:
        rows = sched.plan()
        if not rows:
            break
        sampled = []
        for r in rows:
            # The row's tokens are the request's tokens from `start` on.
            assert histories[r.request_id][r.start:r.start + len(r.tokens)] == r.tokens
            if r.sample:
                assert r.start + len(r.tokens) == len(histories[r.request_id])
                sampled.append(toy_next(histories[r.request_id]))
        if on_step:
            on_step(rows)
        for e in sched.commit(sampled):
            histories[e.request_id].append(e.token)
            outputs[e.request_id].append(e.token)
        assert cache.check() == ""
        steps += 1
        assert steps < max_steps
    return outputs, steps


def expected(prompt, n, eos=()):
    h, out = list(prompt), []
    for _ in range(n):
        t = toy_next(h)
        h.append(t); out.append(t)
        if t in eos:
            break
    return out


def test_one_request_prefill_then_decode():
    # tests/engine_step.rs:27-60, 201-209: prompt [1, 2, 3], max_tokens 1: one step, one token, queues empty.
    cache, s = make()
    assert s.add_request(0, [1, 2, 3], 1) == "Accepted"
    rows = s.plan()
    assert len(rows) == 1 and rows[0].tokens == [1, 2, 3] and rows[0].start == 0 and rows[0].sample
    out = s.commit([42])
    assert [(e.request_id, e.token, e.finished) for e in out] == [(0, 42, True)]
    assert s.plan() == [] and s.num_waiting() == 0 and s.num_running() == 0 and cache.free_pages() == 8


def test_decode_rows_feed_the_last_token():
    # tests/engine_step.rs:278-300: after the prefill of 3 tokens the decode row holds the sampled
    # token at position 3; the next one position 4 (a new page with pages of 4).
    cache, s = make()
    s.add_request(0, [1, 2, 3], 3)
    s.plan(); s.commit([10])
    rows = s.plan()
    assert (rows[0].tokens, rows[0].start, rows[0].output_index) == ([10], 3, 1)
    assert cache.slots(0, 0, 3, 1).tolist() == [3]
    s.commit([11])
    rows = s.plan()
    assert (rows[0].tokens, rows[0].start) == ([11], 4) and cache.slots(0, 0, 4, 1).tolist() == [4]
    assert s.commit([12])[0].finished


def test_admission_status():
    # src/exec/request_state.rs:203-211; tests/engine_dynamic_arrival.rs:98-158.
    cache, s = make(max_len=16)
    assert s.add_request(1, [1], 1) == "Accepted"
    assert s.add_request(1, [1], 1) == "DuplicateRequestId"
    assert s.add_request(2, [], 1) == "EmptyPrompt"
    assert s.add_request(3, [1], 0) == "ZeroMaxTokens"
    assert s.add_request(4, [1], 1, eos_token_ids=(1, 2, 3, 4)) == "TooManyEosTokenIds"
    assert s.add_request(5, [1] * 10, 7) == "HistoryCapacityOverflow"
    # src/exec/engine.rs:2718-2720: end tokens that count need at least one id.
    assert s.add_request(6, [1], 1, eos_token_ids=(), ignore_eos=False) == "EmptyEosTokenIds"
    assert s.add_request(6, [1], 1, eos_token_ids=(), ignore_eos=True) == "Accepted"
    s.plan(); s.commit([5, 5])
    assert s.add_request(1, [1], 1) == "DuplicateRequestId"      # ids are never reused


def test_long_prompt_is_cut_at_page_boundaries_under_the_budget():
    # tests/engine_step.rs:211-243: a 3-page prompt under a one-page budget takes three steps and
    # emits on the third; tests/cache_scheduler_plan.rs:168-197: a non-final portion is not sampled.
    cache, s = make(page=4, budget=4)
    s.add_request(0, list(range(12)), 1)
    seen = []
    for _ in range(3):
        rows = s.plan()
        seen.append((rows[0].start, len(rows[0].tokens), rows[0].sample))
        out = s.commit([7] if rows[0].sample else [])
    assert seen == [(0, 4, False), (4, 4, False), (8, 4, True)] and out[0].token == 7
    # All pages of the prompt are taken at admission (planning.rs:992-998).
    cache, s = make(page=4, budget=6)
    s.add_request(0, list(range(12)), 1)
    rows = s.plan()
    assert len(rows[0].tokens) == 4 and cache.num_logical_pages(0, 0) == 3     # floor(6 / 4) * 4


def test_mixed_step_and_token_budget():
    # tests/engine_step.rs:245-276 and cache_scheduler_plan.rs:75-166: decode rows come first and count
    # one token each; the head of the queue is admitted with what is left of the budget.
    cache, s = make(page=4, budget=5, pages=16)
    s.add_request(0, [1, 2], 4)
    s.plan(); s.commit([9])
    s.add_request(1, [1, 2, 3, 4, 5, 6, 7, 8, 9], 2)
    s.add_request(2, [4, 5], 2)
    rows = s.plan()
    assert [(r.request_id, len(r.tokens), r.sample) for r in rows] == [(0, 1, True), (1, 4, False)]
    assert s.num_waiting() == 1           # request 2 waits behind the cut prompt
    s.commit([9])
    rows = s.plan()
    assert [(r.request_id, len(r.tokens)) for r in rows] == [(0, 1), (1, 4)]
    s.commit([9])
    rows = s.plan()                       # request 1's last token, then request 2 with the rest
    assert [(r.request_id, len(r.tokens), r.sample) for r in rows] == [(0, 1, True), (1, 1, True), (2, 2, True)]


def test_max_num_seqs_bounds_rows():
    cache, s = make(seqs=2, pages=16)
    for i in range(4):
        s.add_request(i, [1, 2], 2)
    assert [r.request_id for r in s.plan()] == [0, 1] and s.num_waiting() == 2
    s.commit([1, 1])
    assert [r.request_id for r in s.plan()] == [0, 1]
    s.commit([1, 1])                      # both finish
    assert [r.request_id for r in s.plan()] == [2, 3]


def test_end_tokens():
    # src/exec/request_state.rs:482-501: the end token is emitted, then the request is over.
    cache, s = make()
    s.add_request(0, [1], 5, eos_token_ids=(7, 8))
    s.add_request(1, [1], 3, eos_token_ids=(7,), ignore_eos=True)
    s.plan()
    out = s.commit([8, 7])
    assert [(e.token, e.finished) for e in out] == [(8, True), (7, False)]
    assert not s.is_live(0) and s.is_live(1)


def test_pages_run_out_decode_waits_prefill_waits():
    # src/exec/cache_scheduler/planning.rs:241-246: no swap; who cannot get a page is left out of the step.
    cache, s = make(page=4, pages=3, seqs=4)
    s.add_request(0, [1, 2, 3, 4], 8)       # 1 page, the next token opens another
    s.add_request(1, [1, 2, 3], 8)          # 1 page
    s.add_request(2, [1, 2, 3, 4, 5], 8)    # 2 pages: does not fit beside the others
    rows = s.plan()
    # Request 1 is admitted only while a page of headroom stays for request 0's next token.
    assert [r.request_id for r in rows] == [0, 1] and s.num_waiting() == 1
    s.commit([5, 5])
    rows = s.plan()
    assert [r.request_id for r in rows] == [0, 1] and cache.free_pages() == 0
    s.commit([5, 5])
    h = {0: [1, 2, 3, 4, 5, 5], 1: [1, 2, 3, 5, 5], 2: [1, 2, 3, 4, 5]}
    # From here on the toy model drives; everything finishes, with preemption if it has to be.
    outputs, _ = drive(s, cache, h)
    assert cache.free_pages() == 3 and cache.num_requests() == 0
    assert len(outputs[2]) == 8


def test_preemption_recomputes_and_gives_the_same_tokens():
    prompts = {i: [i + 1, i + 2, i + 3] for i in range(4)}
    want = {i: expected(p, 12) for i, p in prompts.items()}
    cache, s = make(page=4, pages=6, seqs=4, budget=64)     # 4 requests of 15 tokens need 16 pages
    h = {i: list(p) for i, p in prompts.items()}
    for i, p in prompts.items():
        s.add_request(i, p, 12)
    outputs, _ = drive(s, cache, h)
    assert outputs == want and s.preemptions() > 0 and cache.free_pages() == 6


def test_request_larger_than_the_pool_is_an_error():
    cache, s = make(page=4, pages=2)
    s.add_request(0, list(range(9)), 1)
    with pytest.raises(OutOfPages):
        s.plan()
    cache, s = make(page=4, pages=2)
    s.add_request(0, list(range(7)), 8)     # fits at first, then outgrows the pool alone
    h = {0: list(range(7))}
    with pytest.raises(OutOfPages):
        drive(s, cache, h)


def test_budget_below_a_page_still_progresses():
    cache, s = make(page=8, budget=3, pages=8)
    h = {0: list(range(20))}
    s.add_request(0, h[0], 2)
    outputs, steps = drive(s, cache, h)
    assert outputs[0] == expected(list(range(20)), 2) and steps >= 7


def test_prefix_reuse_through_the_scheduler():
    cache, s = make(page=4, pages=16, prefix=True)
    shared = list(range(50, 62))
    h = {0: shared + [1, 2], 1: shared + [3]}
    s.add_request(0, h[0], 2)
    rows = s.plan()
    assert rows[0].start == 0
    s.commit([toy_next(h[0])]); h[0].append(toy_next(h[0][:14]))
    s.add_request(1, h[1], 2)
    rows = s.plan()
    by_id = {r.request_id: r for r in rows}
    assert by_id[1].start == 12 and by_id[1].tokens == [3]       # three pages found in the cache
    assert cache.prefix_hits() == 3


def test_reuse_is_counted_once_for_an_admission_that_had_to_wait():
    """A request whose prompt finds cached pages but no pages for the rest waits; each step tries its
    admission again, and only the one that stands counts as a reuse."""
    cache, s = make(page=4, pages=7, prefix=True)
    shared = list(range(50, 58))                                   # two pages
    h = {0: shared + list(range(8)), 1: shared + list(range(20, 32))}
    s.add_request(0, h[0], 6)                                      # 4 pages for its prompt, 2 more while decoding
    s.plan(); s.commit([toy_next(h[0])]); h[0].append(toy_next(h[0][:16]))
    s.add_request(1, h[1], 2)                                      # 3 pages of its own and one to decode into: 7 - 4 do not hold them
    waited = 0
    while s.num_waiting():
        rows = s.plan()
        assert cache.check() == ""
        waited += 1
        s.commit([toy_next(h[r.request_id]) for r in rows if r.sample])
        for r in rows:
            if r.sample:
                h[r.request_id].append(toy_next(h[r.request_id]))
    assert waited > 2
    assert cache.prefix_hits() == 2 and cache.prefix_hit_requests() == 1


@pytest.mark.parametrize("seed", range(6))
def test_outputs_do_not_depend_on_the_schedule(seed):
    """Staggered arrivals, small budgets, few pages, windows: every request still gets the tokens it
    would get alone (the reference's schedule stress, scripts/determinism_tests/schedule_stress.py:20-106,
    with a toy model)."""
    rng = random.Random(seed)
    n = 8
    prompts = {i: [rng.randrange(50) for _ in range(rng.choice([1, 3, 4, 5, 9, 17, 31]))] for i in range(n)}
    max_new = {i: rng.randrange(1, 12) for i in range(n)}
    want = {i: expected(prompts[i], max_new[i], eos=(13,)) for i in range(n)}
    arrivals = sorted(rng.randrange(0, 20) for _ in range(n))
    cache, s = make(page=4, pages=rng.choice([12, 16, 40]), seqs=rng.choice([2, 3, 4]), budget=rng.choice([4, 7, 16, 64]),
                    prefix=rng.random() < 0.5, windows=rng.choice([(0,), (0, 8)]))
    h = {i: list(p) for i, p in prompts.items()}
    outputs = {i: [] for i in range(n)}
    step, arrived = 0, 0
    while arrived < n or s.num_waiting() or s.num_running():
        while arrived < n and arrivals[arrived] <= step:
            assert s.add_request(arrived, prompts[arrived], max_new[arrived], eos_token_ids=(13,)) == "Accepted"
            arrived += 1
        rows = s.plan()
        sampled = [toy_next(h[r.request_id]) for r in rows if r.sample]
        for r in rows:
            assert h[r.request_id][r.start:r.start + len(r.tokens)] == r.tokens
        for e in s.commit(sampled):
            h[e.request_id].append(e.token)
            outputs[e.request_id].append(e.token)
        assert cache.check() == ""
        step += 1
        assert step < 5000
    assert outputs == want
    assert cache.num_requests() == 0 and cache.available_pages(0) == cache.groups[0].num_pages


def test_a_step_that_did_not_run_is_planned_again():
    """plan, give up, plan: the same rows, nothing lost, and the outputs of the whole run unchanged."""
    from vosti_amd.engine.scheduler import SchedulerError
    cache, s = make(pages=12, page=4, seqs=3, budget=8)
    hist = {0: list(range(10)), 1: [7, 7, 7], 2: list(range(20, 26))}
    for rid, p in hist.items():
        s.add_request(rid, list(p), 5)
    key = lambda rows: [(r.request_id, r.start, tuple(r.tokens), r.sample, r.state_slot, r.output_index) for r in rows]
    first = s.plan()
    assert first and cache.pending(first[0].request_id) == len(first[0].tokens)
    with pytest.raises(SchedulerError, match="before the step planned last"):
        s.plan()
    with pytest.raises(SchedulerError, match="nothing was committed"):
        s.commit([1] * (sum(r.sample for r in first) + 1))
    s.abort_step()
    assert all(cache.pending(r.request_id) == 0 for r in first) and cache.check() == ""
    again = s.plan()
    assert key(again) == key(first)
    s.abort_step()
    # Given up twice, then run to the end: what comes out is what an undisturbed run gives.
    outs, _ = drive(s, cache, hist)
    assert outs == {0: expected(range(10), 5), 1: expected([7, 7, 7], 5), 2: expected(range(20, 26), 5)}
    assert cache.num_requests() == 0 and cache.check() == ""
    # Giving up when nothing is planned is harmless.
    s.abort_step()
    assert s.plan() == []
