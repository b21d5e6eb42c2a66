"""The cache manager: no page lost, held twice or freed twice, under random orders of requests;
prefix reuse; windows; state slots. No GPU."""
import random

import pytest

from mini_engine_amd.cache.manager import CacheManager, PrefixHit, page_hash


def test_allocate_grows_by_pages_and_is_all_or_nothing():
    m = CacheManager(4, 8)
    assert m.allocate("a", 0, 5) and m.block_table("a") == [0]
    assert m.allocate("a", 5, 3) and m.block_table("a") == [0]          # still inside the first page
    assert m.allocate("a", 8, 1) and m.block_table("a") == [0, 1]
    assert not m.allocate("b", 0, 17)                                   # needs 3, only 2 free
    assert not m.holds("b") and m.num_free_pages() == 2
    assert m.allocate("b", 0, 16)
    assert m.num_free_pages() == 0 and not m.allocate("a", 9, 8)
    m.check_invariants()
    m.free("a"); m.free("b")
    assert m.num_free_pages() == 4
    with pytest.raises(KeyError):
        m.free("a")                                                     # freeing twice is an error, not a leak
    m.check_invariants()


def test_freed_pages_are_used_again_oldest_first():
    m = CacheManager(3, 4)
    m.allocate("a", 0, 8)            # pages 0, 1
    m.free("a")                      # returned in reverse: 1 then 0 -> free = [2, 1, 0]
    m.allocate("b", 0, 12)
    assert m.block_table("b") == [2, 1, 0]


def test_random_traffic_keeps_invariants():
    rng = random.Random(0)
    for page, windows, slots in ((4, [None], 0), (8, [None, 16], 3), (4, [12, None, 40], 0)):
        m = CacheManager([rng.randint(6, 20) for _ in windows], page, windows, num_state_slots=slots)
        live = {}
        for it in range(3000):
            r = rng.random()
            if live and r < 0.25:
                rid = rng.choice(list(live))
                m.free(rid); del live[rid]
            elif live and r < 0.8:
                rid = rng.choice(list(live))
                n = rng.randint(1, 3 * page)
                if m.allocate(rid, live[rid], n):
                    live[rid] += n
            else:
                rid = f"r{it}"
                n = rng.randint(1, 4 * page)
                if m.allocate(rid, 0, n):
                    live[rid] = n
                else:
                    assert not m.holds(rid)
            m.check_invariants()
            for rid, n in live.items():
                for g, w in enumerate(windows):
                    t = m.block_table(rid, g)
                    assert len(t) == -(-n // page)
                    # every key the next token may see still has a page
                    lo = 0 if w is None else max(0, n - w + 1)
                    assert all(p >= 0 for p in t[lo // page:])
                if slots:
                    assert 0 <= m.state_slot(rid) < slots
        for rid in list(live):
            m.free(rid)
        m.check_invariants()
        assert all(m.num_free_pages(g) == m.num_pages(g) for g in range(len(windows)))


def test_window_pages_are_given_back_when_passed():
    m = CacheManager(4, 4, [6])
    assert m.allocate("a", 0, 4)
    for pos in range(4, 40):          # one token at a time: never more than 3 pages are needed
        assert m.allocate("a", pos, 1), pos
        held = [p for p in m.block_table("a") if p >= 0]
        assert len(held) <= 3
        first_needed = max(0, pos - 6 + 1)
        assert all(p >= 0 for p in m.block_table("a")[first_needed // 4:])
        assert all(p == -1 for p in m.block_table("a")[:first_needed // 4])
    m.check_invariants()
    m.free("a")
    assert m.num_free_pages() == 4


def test_state_slots():
    m = CacheManager(8, 4, [None], num_state_slots=2)
    assert m.allocate("a", 0, 1) and m.allocate("b", 0, 1)
    assert {m.state_slot("a"), m.state_slot("b")} == {0, 1}
    assert not m.allocate("c", 0, 1) and not m.holds("c")      # no slot left
    m.free("a")
    assert m.allocate("c", 0, 1) and m.state_slot("c") == 0
    assert not m.prefix_caching                                # state cannot be rebuilt from cached pages
    m.check_invariants()


def test_prefix_hash_chain_and_hits():
    assert page_hash([1, 2, 3]) != page_hash([1, 2, 3], prefix=5)
    m = CacheManager(8, 4)
    toks = list(range(10, 23))                 # 13 tokens: 3 full pages + 1
    assert m.find_prefix_hit(toks).num_pages == 0
    m.allocate("a", 0, 13)
    m.publish_full_pages("a", toks, 6)         # only the first page is complete so far
    assert m.find_prefix_hit(toks).num_pages == 1
    m.publish_full_pages("a", toks, 13)
    hit = m.find_prefix_hit(toks)
    assert hit.num_pages == 3 and hit.pages[0] == m.block_table("a")[:3]
    # never the page that holds the last token: 12 tokens = 3 full pages, but only 2 may hit
    assert m.find_prefix_hit(toks[:12]).num_pages == 2
    # a different token in page 1 stops the chain there
    other = toks[:5] + [999] + toks[6:]
    assert m.find_prefix_hit(other).num_pages == 1
    # sharing: the hit pages are held twice
    hb = m.find_prefix_hit(toks)
    assert m.allocate("b", 0, 13 - 12, hb) and m.block_table("b")[:3] == m.block_table("a")[:3]
    m.check_invariants()
    m.free("a")
    m.check_invariants()
    assert m.find_prefix_hit(toks).num_pages == 3          # still held by b
    m.free("b")
    assert m.find_prefix_hit(toks).num_pages == 3          # freed pages stay hittable until reused
    hc = m.find_prefix_hit(toks)
    assert m.allocate("c", 0, 1, hc)                       # free hit pages are taken out of the free list
    m.check_invariants()
    m.free("c")
    # reuse evicts: fill the pool with other content
    m.allocate("d", 0, 32)
    assert m.find_prefix_hit(toks).num_pages == 0
    m.check_invariants()


def test_hit_counts_free_hit_pages_against_the_free_list():
    m = CacheManager(3, 4)
    toks = list(range(9))
    m.allocate("a", 0, 9); m.publish_full_pages("a", toks, 9); m.free("a")
    hit = m.find_prefix_hit(toks)
    assert hit.num_pages == 2 and m.num_free_pages() == 3
    # 2 hit pages (sitting in the free list) + 2 fresh pages > 3 free pages: refused, nothing changes
    assert not m.allocate("b", 0, 8, hit)
    assert m.num_free_pages() == 3 and not m.holds("b")
    assert m.allocate("b", 0, 1, hit) and m.num_free_pages() == 0
    m.check_invariants()


def test_prefix_caching_is_off_with_windows():
    m = CacheManager(8, 4, [None, 8])
    m.allocate("a", 0, 12)
    m.publish_full_pages("a", list(range(12)), 12)
    assert m.find_prefix_hit(list(range(12))).num_pages == 0
