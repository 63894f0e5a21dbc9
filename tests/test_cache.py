"""The page pool and the cache manager (no GPU): nothing lost, nothing held twice, nothing freed
twice, under scripted cases and under random orders of requests."""
import random

import pytest

from dinfer_amd.cache import CacheManager, GroupSpec
from page_pool_front import BlockPool


def test_alloc_free_roundtrip():
    """The reference's vector, crates/core/src/kv/block_pool.rs:239-250."""
    p = BlockPool(4)
    a = p.allocate(3)
    assert a == [0, 1, 2] and p.num_free == 1
    assert p.allocate(2) is None and p.num_free == 1      # all or nothing
    p.free(a)
    assert p.num_free == 4 and p.free_list() == [0, 1, 2, 3]   # back at the head, order kept
    p.check()


def test_freed_pages_are_reused_first():
    p = BlockPool(6)
    a, b = p.allocate(2), p.allocate(2)
    p.free(a)
    assert p.allocate(3) == [0, 1, 4]
    p.check()


def test_double_free_and_foreign_page_raise():
    p = BlockPool(3)
    a = p.allocate(1)
    p.free(a)
    with pytest.raises(RuntimeError, match="not held"):
        p.free(a)
    with pytest.raises(RuntimeError, match="not held"):
        p.free([7])
    p.check()


def mgr(blocks=8, page=16, window=None, seqs=4):
    return CacheManager([GroupSpec(page, blocks, window)], seqs)


def test_out_of_blocks_returns_false_and_keeps_state():
    """kv/manager.rs:453-484: a failed allocation changes nothing; chunks allocate incrementally."""
    m = mgr(blocks=4)
    m.admit("a")
    assert m.allocate("a", 0, 33) and m.block_table("a", 0) == [0, 1, 2]
    m.admit("b")
    assert not m.allocate("b", 0, 17)
    assert m.block_table("b", 0) == [] and m.num_free() == 1
    assert m.allocate("b", 0, 16) and m.num_free() == 0
    assert m.allocate("a", 33, 15) and m.block_table("a", 0) == [0, 1, 2]   # stays inside its last page
    assert not m.allocate("a", 48, 1)
    m.check()


def test_chunked_prefill_allocates_incrementally_and_slots_follow_pages():
    m = mgr(blocks=8, page=16)
    m.admit("a")
    m.allocate("a", 0, 10)
    assert m.pages_needed("a", 10, 6) == [0] and m.pages_needed("a", 10, 7) == [1]
    m.allocate("a", 10, 30)
    assert m.block_table("a", 0) == [0, 1, 2]
    # slot = page * page_size + position % page_size (crates/core/src/runner.rs:830-834)
    assert m.slot_mapping("a", 0, 14, 4) == [14, 15, 16, 17]
    m.free("a")
    m.admit("b")
    m.allocate("b", 0, 20)
    assert m.block_table("b", 0) == [2, 1]       # the tail of the freed request is taken first
    assert m.slot_mapping("b", 0, 15, 2) == [2 * 16 + 15, 16]
    m.check()


def test_window_pages_are_given_back_while_the_request_lives():
    m = mgr(blocks=8, page=4, window=6)
    m.admit("a")
    assert m.allocate("a", 0, 10)                 # pages 0..2
    assert m.release_passed("a", 10) == 1         # next position 10 sees keys 5..10: page 0 (keys 0..3) is dead
    assert m.block_table("a", 0) == [-1, 1, 2] and m.num_free() == 6
    assert m.allocate("a", 10, 3)                 # position 12 needs page 3: the freed page is used again
    assert m.block_table("a", 0) == [-1, 1, 2, 0]
    assert m.release_passed("a", 13) == 1         # next position 13 sees 8..13: page 1 (keys 4..7) is dead
    with pytest.raises(RuntimeError, match="given back"):
        m.slot_mapping("a", 0, 5, 1)
    m.check()
    m.free("a")
    assert m.num_free() == 8
    m.check()


def test_groups_have_pages_of_their_own():
    m = CacheManager([GroupSpec(4, 10, None), GroupSpec(4, 3, 8)], 2)
    m.admit("a")
    assert not m.allocate("a", 0, 16)             # the window group has only 3 pages: nothing is taken anywhere
    assert m.num_free(0) == 10 and m.num_free(1) == 3
    assert m.allocate("a", 0, 12)
    m.release_passed("a", 12)                     # window 8: next position 12 sees 5..12 -> page 0 dead
    assert m.block_table("a", 1)[0] == -1 and m.block_table("a", 0)[0] >= 0
    assert m.allocate("a", 12, 4)
    m.check()


def test_state_slots():
    m = mgr(seqs=2)
    assert m.admit("a") == 0 and m.admit("b") == 1
    assert m.take_fresh_slots() == [0, 1] and m.take_fresh_slots() == []
    assert not m.can_admit()
    with pytest.raises(RuntimeError, match="slots"):
        m.admit("c")
    with pytest.raises(KeyError):
        m.admit("a")
    m.free("a")
    assert m.admit("c") == 0 and m.take_fresh_slots() == [0]    # a reused slot is reported for zeroing again
    m.check()


@pytest.mark.parametrize("window", [None, 24])
@pytest.mark.parametrize("seed", range(5))
def test_random_orders_keep_the_invariants(seed, window):
    rng = random.Random(seed)
    m = CacheManager([GroupSpec(8, 40, None), GroupSpec(8, 40, window)], 5)
    live = {}
    for step in range(600):
        r = rng.random()
        if r < 0.25 and m.can_admit():
            rid = f"r{step}"
            m.admit(rid)
            live[rid] = 0
        elif r < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 7, 8, 9, 30])
            free_before = [m.num_free(0), m.num_free(1)]
            if m.allocate(rid, live[rid], n):
                live[rid] += n
                m.release_passed(rid, live[rid])
                # every position the next token may read still has a page
                lo = max(0, live[rid] - window + 1) if window else 0
                m.slot_mapping(rid, 1, lo, live[rid] - lo)
                m.slot_mapping(rid, 0, 0, live[rid])
            else:
                assert [m.num_free(0), m.num_free(1)] == free_before
        elif live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free(rid)
    m.check()
    assert m.num_free(0) == 40 and m.num_free(1) == 40


# ---- prefix cache ----------------------------------------------------------------------------------
def pmgr(blocks=8, page=4, seqs=4):
    return CacheManager([GroupSpec(page, blocks)], seqs, prefix_caching=True)


def run_request(m, rid, tokens, keep=False):
    """Admits, looks the prefix up, allocates and commits the rest; returns the tokens found cached."""
    m.admit(rid)
    got = m.lookup(rid, tokens)
    assert m.allocate(rid, got, len(tokens) - got)
    m.commit(rid, tokens, len(tokens))
    if not keep:
        m.free(rid)
    m.check()
    return got


def test_prefix_is_found_again_but_never_the_whole_prompt():
    """kv/manager.rs:150-199: full pages only, and at most (n - 1) / page of them."""
    m = pmgr()
    a = list(range(100, 110))                       # 10 tokens: two full pages and a half
    assert run_request(m, "a", a) == 0
    assert run_request(m, "b", a) == 8              # both full pages
    assert run_request(m, "c", a[:8]) == 4          # 8 tokens: the last one must be computed, so one page
    assert run_request(m, "d", a[:5] + [7] + a[6:]) == 4   # differs inside the second page
    assert run_request(m, "e", [1] + a[1:]) == 0    # differs in the first page: nothing, though later pages match


def test_shared_pages_have_two_holders():
    m = pmgr()
    a = list(range(20))
    run_request(m, "a", a, keep=True)
    assert run_request(m, "b", a[:13] + [99], keep=True) == 12
    ta, tb = m.block_table("a", 0), m.block_table("b", 0)
    assert ta[:3] == tb[:3] and ta[3] != tb[3]
    m.free("a")
    m.check()
    assert m.block_table("b", 0) == tb and m.num_free() == 8 - 4   # b still holds the shared pages
    m.free("b")
    m.check()
    assert m.num_free() == 8


def test_named_pages_are_evicted_last_and_oldest_first():
    """kv/block_pool.rs:160-182: nameless pages return to the head, named ones to the tail; a request is
    freed last page first, so its tail is evicted before its head (kv/manager.rs:338-345)."""
    m = pmgr(blocks=6)
    a = list(range(50, 62))                         # three full pages: 0, 1, 2
    run_request(m, "a", a + [1])                    # and one token in page 3 (nameless)
    assert m.pools[0].free_list() == [3, 4, 5, 2, 1, 0]
    m.admit("x")
    assert m.allocate("x", 0, 16)                   # takes 3, 4, 5 and the youngest-freed named page, 2
    assert m.block_table("x", 0) == [3, 4, 5, 2]
    m.free("x")                                     # nameless now: back at the head, last page first
    assert m.pools[0].free_list() == [2, 5, 4, 3, 1, 0]
    assert run_request(m, "b", a + [1], keep=True) == 8     # pages 0 and 1 are still named, 2 is not
    m.check()


def test_random_prefix_traffic_keeps_the_invariants():
    rng = random.Random(3)
    m = CacheManager([GroupSpec(4, 24), GroupSpec(4, 30)], 4, prefix_caching=True)
    stems = [[rng.randrange(50) for _ in range(40)] for _ in range(3)]
    live, hits = {}, 0
    for step in range(500):
        if live and (len(live) == 4 or rng.random() < 0.4):
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        else:
            toks = rng.choice(stems)[:rng.randrange(1, 40)] + [rng.randrange(50) for _ in range(rng.randrange(0, 6))]
            rid = f"r{step}"
            m.admit(rid)
            got = m.lookup(rid, toks)
            assert got % 4 == 0 and got < len(toks)
            hits += got
            if m.allocate(rid, got, len(toks) - got):
                m.commit(rid, toks, len(toks))
                assert m.slot_mapping(rid, 0, 0, len(toks)) and m.slot_mapping(rid, 1, 0, len(toks))
                live[rid] = toks
            else:
                m.free(rid)
        m.check()
    assert hits > 500
    for rid in list(live):
        m.free(rid)
    m.check()
    assert m.num_free(0) == 24 and m.num_free(1) == 30


def test_prefix_cache_refuses_window_groups():
    with pytest.raises(ValueError, match="every key"):
        CacheManager([GroupSpec(4, 8, 6)], 2, prefix_caching=True)
