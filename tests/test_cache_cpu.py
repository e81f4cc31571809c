"""The cache manager on the CPU: pages, block tables, windows, state slots, prefix reuse."""
import random

import pytest
from hypothesis import given, settings, strategies as st

from vosti_amd.cache.manager import CacheError, CacheManager, GroupSpec, OutOfPages


def mgr(page=4, pages=8, slots=4, windows=(0,), prefix=False):
    return CacheManager(page, [GroupSpec(w, pages) for w in windows], slots, prefix)


def feed(m, rid, tokens):
    m.extend(rid, tokens)
    m.commit(rid)


def test_slot_arithmetic_and_growth():
    # Reference: slot = block_ids[i / P] * P + i % P, pages needed (n-1)/P + 1
    # (src/exec/cache_scheduler/admission.rs:1166-1174); the free queue hands out pages 0, 1, 2, ...
    # (admission.rs:37-52); tests/engine_step.rs:278-312 holds the same vectors with P = 64.
    m = mgr(page=4, pages=8)
    m.add_request(7)
    m.extend(7, [1, 2, 3])
    assert m.slots(7, 0, 0, 3).tolist() == [0, 1, 2] and m.num_logical_pages(7, 0) == 1
    m.commit(7)
    assert m.length(7) == 3
    feed(m, 7, [9])                       # the tail page has room
    assert m.num_logical_pages(7, 0) == 1
    feed(m, 7, [9])                       # position 4 opens page 1
    assert m.slots(7, 0, 4, 1).tolist() == [4] and m.num_logical_pages(7, 0) == 2
    assert m.block_table_row(7, 0, 3).tolist() == [0, 1, 0]     # padded with page 0
    m.finish(7)
    assert m.free_pages() == 8 and m.check() == ""


def test_released_pages_are_used_first():
    m = mgr(page=4, pages=6)
    m.add_request(1); feed(m, 1, list(range(8)))       # pages 0, 1
    m.add_request(2); feed(m, 2, list(range(4)))       # page 2
    m.finish(1)
    m.add_request(3); feed(m, 3, list(range(4)))
    assert m.block_table_row(3, 0, 1).tolist()[0] in (0, 1)      # a page request 1 gave back, not page 3
    assert m.check() == ""


def test_out_of_pages_changes_nothing():
    m = mgr(page=4, pages=2)
    m.add_request(1); feed(m, 1, list(range(5)))
    m.add_request(2)
    with pytest.raises(OutOfPages):
        m.extend(2, [1])
    assert not m.try_extend(1, [1, 2, 3, 4])            # would need a third page
    assert m.pending(1) == 0 and m.length(1) == 5 and m.check() == ""
    assert m.try_extend(1, [1, 2, 3])
    m.commit(1)
    m.finish(1); m.finish(2)
    assert m.free_pages() == 2 and m.free_slots() == 4


def test_state_slots_and_errors():
    m = mgr(slots=2)
    m.add_request(1); m.add_request(2)
    assert {m.state_slot(1), m.state_slot(2)} == {0, 1}
    with pytest.raises(CacheError, match="slots"):
        m.add_request(3)
    with pytest.raises(CacheError, match="duplicate"):
        m.add_request(1)
    with pytest.raises(CacheError, match="unknown"):
        m.finish(9)
    m.extend(1, [1])
    with pytest.raises(CacheError, match="pending"):
        m.extend(1, [2])
    m.abort_step(1)
    assert m.pending(1) == 0
    m.finish(1)
    m.add_request(3)
    assert m.state_slot(3) in (0, 1) and m.check() == ""


def test_window_group_gives_pages_back():
    # Group 0 keeps all keys, group 1 the last 6.  The next query at position L sees keys >= L - 5:
    # a page goes back once all of its positions lie below that.
    m = mgr(page=4, pages=8, windows=(0, 6))
    m.add_request(1)
    feed(m, 1, list(range(9)))            # L = 9: first needed key 4 -> page 0 (keys 0..3) goes back
    assert m.free_pages(0) == 8 - 3 and m.free_pages(1) == 8 - 2
    assert m.block_table_row(1, 1, 3).tolist()[0] == 0        # the released entry reads as page 0
    feed(m, 1, list(range(20)))           # L = 29: first needed 24 -> pages 0..5 gone, 6, 7 live
    assert m.free_pages(1) == 8 - 2 and m.free_pages(0) == 0
    with pytest.raises(CacheError):       # a position the window has passed has no slot any more
        m.slots(1, 1, 0, 1)
    assert m.slots(1, 1, 28, 1).size == 1
    m.finish(1)
    assert m.free_pages(0) == 8 and m.free_pages(1) == 8 and m.check() == ""


def test_window_pool_is_reused_within_one_request():
    # 3 pages of 4 suffice for a window of 4 fed in portions of 4, however long the request is.
    m = CacheManager(4, [GroupSpec(4, 3)], 2, False)
    m.add_request(1)
    for i in range(50):
        feed(m, 1, [i] * 4)
        assert m.check() == ""
    assert m.length(1) == 200


# ------------------------------------------------------------------ prefix reuse
def test_prefix_reuse_basics():
    # Reference behaviours: a later request finds the published pages of an earlier one
    # (tests/cache_scheduler_plan.rs:199-255); at least one prompt token stays uncached
    # (src/exec/cache_scheduler/prefix_cache.rs:3187); pages survive their last holder
    # (tests/prefix_cache.rs:184-217).
    m = mgr(page=4, pages=8, prefix=True)
    prompt = list(range(10, 22))                     # 3 full pages
    assert m.add_request(1, prompt) == 0
    feed(m, 1, prompt)
    assert m.add_request(2, prompt) == 8             # (12 - 1) // 4 = 2 pages, the last token is computed
    assert m.block_table_row(2, 0, 2).tolist() == m.block_table_row(1, 0, 3).tolist()[:2]
    feed(m, 2, prompt[8:])
    m.finish(1); m.finish(2)
    assert m.cached_blocks() == 3 and m.free_pages() == 5 and m.available_pages() == 8
    assert m.add_request(3, prompt + [1]) == 12      # all three pages, after both holders left
    assert m.prefix_hits() == 5 and m.check() == ""
    m.finish(3)
    # A prompt that differs inside the second page matches the first page only.
    other = prompt[:5] + [999] + prompt[6:]
    assert m.add_request(4, other) == 4
    m.finish(4)
    assert m.check() == ""


def test_prefix_chain_continues_through_generated_pages():
    # tests/prefix_cache.rs:16-44: the hash of a page chains through its predecessor's.
    m = mgr(page=4, pages=8, prefix=True)
    m.add_request(1, [1, 2, 3])
    feed(m, 1, [1, 2, 3])
    for t in (4, 5, 6, 7, 8):                        # decoding fills page 0, then page 1
        feed(m, 1, [t])
    m.finish(1)
    assert m.cached_blocks() == 2
    assert m.add_request(2, [1, 2, 3, 4, 5, 6, 7, 8, 9]) == 8
    m.finish(2)
    assert m.add_request(3, [9, 2, 3, 4, 5, 6, 7, 8, 9]) == 0     # second page alone does not match
    m.finish(3)


def test_eviction_takes_children_before_parents():
    # tests/prefix_cache.rs:220-260, 292-340.
    m = mgr(page=4, pages=4, prefix=True)
    prompt = list(range(16))
    m.add_request(1, prompt); feed(m, 1, prompt); m.finish(1)
    assert m.cached_blocks() == 4 and m.free_pages() == 0
    m.add_request(2, [100, 101, 102, 103, 104])      # needs 2 pages: evicts the two deepest pages
    feed(m, 2, [100, 101, 102, 103, 104])
    assert m.evictions() == 2 and m.check() == ""
    m.finish(2)
    assert m.add_request(3, prompt) == 8             # the first two pages of the chain are still there
    m.finish(3)
    assert m.check() == ""


def test_first_writer_of_a_hash_wins():
    # src/exec/cache_scheduler/prefix_cache.rs:264-272: two requests computing the same page in the
    # same period do not share it; the second one's copy stays private and is freed at once.
    m = mgr(page=4, pages=8, prefix=True)
    p = [5, 6, 7, 8, 9]
    m.add_request(1, p); m.add_request(2, p)
    feed(m, 1, p); feed(m, 2, p)
    assert m.block_table_row(1, 0, 2).tolist() != m.block_table_row(2, 0, 2).tolist()
    m.finish(2)
    assert m.cached_blocks() == 0
    m.finish(1)
    assert m.cached_blocks() == 1 and m.check() == ""


def test_prefix_needs_all_keys_groups():
    m = mgr(page=4, pages=8, windows=(0, 8), prefix=True)
    assert not m.prefix_cache
    p = list(range(12))
    m.add_request(1, p); feed(m, 1, p); m.finish(1)
    assert m.add_request(2, p) == 0


@settings(max_examples=60, deadline=None)
@given(seed=st.integers(0, 10_000), prefix=st.booleans(), windows=st.sampled_from([(0,), (0, 6), (5,), (0, 0)]))
def test_no_page_lost_or_held_twice_under_random_orders(seed, prefix, windows):
    rng = random.Random(seed)
    m = mgr(page=4, pages=12, slots=5, windows=windows, prefix=prefix)
    live, next_id = {}, 0
    for _ in range(200):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            prompt = [rng.randrange(3) for _ in range(rng.randrange(1, 14))]
            cached = m.add_request(next_id, prompt)
            live[next_id] = prompt[cached:]
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            todo = live[rid]
            n = rng.randrange(1, 7)
            chunk = todo[:n] if todo else [rng.randrange(3) for _ in range(n)]
            if m.try_extend(rid, chunk):
                if rng.random() < 0.1:
                    m.abort_step(rid)
                else:
                    m.commit(rid)
                    live[rid] = todo[n:]
        elif live:
            rid = rng.choice(list(live))
            m.finish(rid)
            del live[rid]
        assert m.check() == "", m.check()
    for rid in live:
        m.finish(rid)
    assert m.check() == ""
    assert all(m.available_pages(g) == 12 for g in range(len(windows)))
    assert m.free_slots() == 5


def test_drop_cached_gives_every_unheld_page_back():
    m = CacheManager(4, [GroupSpec(0, 8)], 4, True)
    a, b = list(range(12)), list(range(100, 109))
    m.add_request(1, a); feed(m, 1, a)
    m.add_request(2, b); feed(m, 2, b); m.finish(2)             # two cached pages, one private tail freed
    assert m.cached_blocks() == 2 and m.free_pages(0) == 8 - 3 - 2
    assert m.drop_cached() == 2 and m.cached_blocks() == 0 and m.free_pages(0) == 5 and m.check() == ""
    assert m.add_request(3, b) == 0                              # nothing left to reuse
    m.finish(3); m.finish(1)
    assert m.drop_cached() == 3 and m.free_pages(0) == 8 and m.check() == ""
