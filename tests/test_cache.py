"""The cache manager: pools, block tables, windowed groups, prefix cache, slots (no GPU)."""

import random

import pytest

from qwen25vl_lite_amd.cache import CacheGroupSpec, CacheManager, OutOfPages, OutOfSlots, PagePool, RadixPrefixCache
from qwen25vl_lite_amd.parts import CacheNeed


def test_pool_refcounts():
    # reference tests/test_components.py:154-170
    pool = PagePool(4)
    a = pool.allocate(2)
    assert pool.in_use() == 2
    pool.fork(a)
    pool.free(a)
    assert pool.in_use() == 2, "a page with two holders survives one free"
    pool.free(a)
    assert pool.in_use() == 0 and pool.num_free == 4
    pool.allocate(4)
    with pytest.raises(OutOfPages):
        pool.allocate(1)
    assert isinstance(OutOfPages("x"), MemoryError)


def test_pool_rejects_bogus_frees():
    # reference tests/test_components.py:663-676
    pool = PagePool(4)
    pool.allocate(2)
    for bad in ([9999], [-1]):
        with pytest.raises(ValueError):
            pool.free(bad)
    a = pool.allocate(1)
    pool.free(a)
    with pytest.raises(ValueError):
        pool.free(a)
    with pytest.raises(ValueError):
        pool.fork(a)
    pool.check({0: 1, 1: 1})


def test_freed_pages_are_handed_out_again():
    pool = PagePool(3)
    a = pool.allocate(3)
    pool.free([a[1]])
    assert pool.allocate(1) == [a[1]]


def _manager(windows=(None,), pages=8, page_size=4, seqs=3, prefix=True):
    groups = [CacheGroupSpec(CacheNeed(2, 8, w), 1 + i) for i, w in enumerate(windows)]
    return CacheManager(groups, pages, page_size, seqs, enable_prefix_cache=prefix)


def test_slot_mapping_vector():
    # reference tests/test_components.py:250-253: table [7, 3, 5], 16 per page, positions 15..17
    cm = CacheManager([CacheGroupSpec(CacheNeed(1, 8), 1)], 8, 16, 2, enable_prefix_cache=False)
    cm.admit("s")
    cm.requests["s"].tables[0] = [7, 3, 5]
    assert cm.slot_mapping("s", 0, 15, 18) == [7 * 16 + 15, 3 * 16 + 0, 3 * 16 + 1]


def test_reserve_is_all_or_nothing_across_groups():
    cm = _manager(windows=(None, None), pages=4, page_size=4)
    cm.admit("a")
    cm.reserve("a", 9)   # 3 pages in each group
    cm.admit("b")
    with pytest.raises(OutOfPages):
        cm.reserve("b", 5)  # 2 pages wanted, 1 free
    assert cm.free_pages() == [1, 1] and cm.table("b", 0) == [] and cm.table("b", 1) == []
    cm.check()
    cm.release("a")
    cm.reserve("b", 5)
    cm.check()
    cm.release("b")
    assert cm.pages_in_use() == [0, 0]


def test_windowed_group_gives_pages_back_as_the_window_passes():
    cm = _manager(windows=(None, 6), pages=16, page_size=4, prefix=False)
    cm.admit("a")
    n = 0
    for step in (5, 4, 1, 1, 1, 9, 1):
        cm.reserve("a", n + step)
        # pages the portion's first query can still see are there while it runs
        first_visible = max(0, n - 6 + 1)
        assert all(p >= 0 for p in cm.table("a", 1)[first_visible // 4:])
        n += step
        cm.commit("a", n)
        table = cm.table("a", 1)
        next_lo = max(0, n - 6 + 1)                    # first key the next token sees
        for i, page in enumerate(table):
            gone = (i + 1) * 4 <= next_lo
            assert (page < 0) == gone, (n, i, table)
        assert all(p >= 0 for p in cm.table("a", 0))   # the full group keeps everything
        cm.check()
    assert cm.pages_in_use()[1] <= (6 + 4 - 1) // 4 + 1
    with pytest.raises(RuntimeError):
        cm.slot_mapping("a", 1, 0, 1)                  # that page is gone
    cm.release("a")
    assert cm.pages_in_use() == [0, 0]


def test_prefix_cache_is_off_when_a_group_is_windowed():
    assert _manager(windows=(None, 6)).prefix_cache is None
    assert _manager(windows=(None, None)).prefix_cache is not None


def test_prefix_match_insert_release():
    # reference tests/test_components.py:228-236: 12 tokens, 3 pages of 4
    pools = [PagePool(32)]
    pc = RadixPrefixCache(pools, 4)
    pages = pools[0].allocate(3)
    pc.insert(list(range(12)), [pages], extra_keys=["k"] * 3)
    matched, nodes, got = pc.match(list(range(12)) + [99], extra_keys=["k"] * 3)
    assert matched == 12 and got == [pages]
    assert pc.match(list(range(12)), extra_keys=["other"] * 3)[0] == 0
    assert all(pc.nodes[n].users == 1 for n in nodes)
    pc.release(nodes)
    assert all(pc.nodes[n].users == 0 for n in nodes)
    # a shared beginning matches although the tails differ (reference tests/test_prefix_block_keys.py:44-55)
    matched, _, got = pc.match(list(range(8)) + [50, 51, 52, 53, 54])
    assert matched == 0   # those nodes carry the extra key
    pc.insert(list(range(8)), [pages[:2]])
    assert pc.match(list(range(8)) + [50, 51, 52, 53, 54])[0] == 8
    assert pc.match(list(range(12)), max_tokens=11)[0] == 8


def test_prefix_eviction_returns_pages():
    # reference tests/test_components.py:679-698
    pools = [PagePool(64)]
    pc = RadixPrefixCache(pools, 4, max_nodes=3)
    for i in range(6):
        pages = pools[0].allocate(1)
        pc.insert(list(range(i * 4, i * 4 + 4)), [pages])
        pools[0].free(pages)  # the request that computed them is done
    assert len(pc) <= 3 and pools[0].in_use() <= 3
    pc.evict(64)
    assert len(pc) == 0 and pools[0].in_use() == 0


def test_clearing_the_prefix_cache_keeps_what_is_in_use():
    cm = _manager(windows=(None,), pages=8, page_size=4, seqs=3)
    toks = list(range(100, 112))
    cm.admit("a")
    cm.reserve("a", 12)
    cm.commit("a", 12)
    assert cm.register_prefix("a", toks) == 3
    cm.release("a")
    cm.admit("b")
    assert cm.adopt_prefix("b", toks[:8] + [1, 2]) == 8        # b uses the first two nodes
    assert cm.prefix_cache.clear() == 1 and len(cm.prefix_cache) == 2
    cm.check()
    cm.release("b")
    assert cm.prefix_cache.clear() == 2 and len(cm.prefix_cache) == 0
    assert cm.pages_in_use() == [0]
    cm.check()


def test_pressure_evicts_unused_prefixes_but_not_used_ones():
    cm = _manager(windows=(None,), pages=4, page_size=4, seqs=3)
    toks = list(range(100, 112))
    cm.admit("a")
    cm.reserve("a", 12)
    cm.commit("a", 12)
    assert cm.register_prefix("a", toks) == 3
    cm.release("a")
    assert cm.pages_in_use() == [3], "the cache keeps the pages"
    cm.admit("b")
    assert cm.adopt_prefix("b", toks[:9] + [1, 2, 3]) == 8      # at least one token stays to compute
    cm.admit("c")
    cm.reserve("c", 8)                                        # needs 2: evicts the unused third node
    assert len(cm.prefix_cache) == 2
    with pytest.raises(OutOfPages):
        cm.reserve("c", 12)                                   # the other two are in use by b
    cm.check()
    cm.release("b")
    cm.reserve("c", 12)
    cm.check()
    cm.release("c")
    assert cm.pages_in_use() == [len(cm.prefix_cache)] == [1], "what is left belongs to the cache"
    cm.prefix_cache.evict(4)
    assert cm.pages_in_use() == [0]


def test_pressure_keeps_entries_whose_pages_would_not_come_back():
    """A running request's registered prefix has no user, but evicting it frees nothing (the
    request still holds the pages): under pressure it stays, so that a later request can find it."""
    cm = _manager(windows=(None,), pages=5, page_size=4, seqs=3)
    toks = list(range(200, 212))
    cm.admit("a")
    cm.reserve("a", 12)
    cm.commit("a", 12)
    assert cm.register_prefix("a", toks) == 3        # a keeps running and holding its three pages
    cm.admit("b")
    with pytest.raises(OutOfPages):
        cm.reserve("b", 12)                           # 2 free pages, 3 wanted: nothing to gain by evicting
    assert len(cm.prefix_cache) == 3, "the entries are still there"
    cm.release("b")
    cm.admit("c")
    assert cm.adopt_prefix("c", toks + [7]) == 12     # and are found
    cm.release("a")
    cm.release("c")
    cm.check()
    cm.prefix_cache.evict(5)                          # now the cache alone holds them: they come back
    assert cm.pages_in_use() == [0] and len(cm.prefix_cache) == 0


def test_fork_shares_full_pages_and_copies_the_one_being_filled():
    cm = _manager(windows=(None, 6), pages=8, page_size=4, seqs=3)
    cm.admit("a")
    cm.reserve("a", 10)
    cm.commit("a", 10)                                  # pages 0..1 full, page 2 half full; window 6 gave page 0 back
    assert cm.table("a", 1)[0] == -1
    copies = cm.fork("a", "b")
    assert [(g, src) for g, src, _ in copies] == [(0, cm.table("a", 0)[2]), (1, cm.table("a", 1)[2])]
    for g, src, dst in copies:
        assert dst != src and cm.table("b", g)[2] == dst
    assert cm.table("b", 0)[:2] == cm.table("a", 0)[:2] and cm.table("b", 1)[:2] == cm.table("a", 1)[:2]
    assert cm.num_tokens("b") == 10 and cm.slot_of("b") != cm.slot_of("a")
    cm.check()
    for req in ("a", "b"):                               # both go on, each into its own pages
        cm.reserve(req, 14)
        cm.commit(req, 14)
    assert cm.table("a", 0)[3] != cm.table("b", 0)[3]
    cm.check()
    cm.release("a")
    cm.check()
    cm.release("b")
    assert cm.pages_in_use() == [0, 0]
    # no room for the copy: nothing changes
    cm.admit("c")
    cm.reserve("c", 30)
    cm.commit("c", 30)
    with pytest.raises(OutOfPages):
        cm.fork("c", "d")
    assert "d" not in cm.requests
    cm.check()
    # at a page boundary nothing is copied
    cm.release("c")
    cm.admit("e")
    cm.reserve("e", 8)
    cm.commit("e", 8)
    assert cm.fork("e", "f") == []
    cm.check()


def test_slots():
    cm = _manager(seqs=2)
    s0, s1 = cm.admit("a"), cm.admit("b")
    assert {s0, s1} == {0, 1}
    with pytest.raises(OutOfSlots):
        cm.admit("c")
    with pytest.raises(ValueError):
        cm.admit("a")
    assert cm.take_fresh("a") and not cm.take_fresh("a")
    cm.release("a")
    assert cm.admit("c") == s0 and cm.take_fresh("c")
    cm.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_lifetimes_lose_nothing(seed):
    """Requests come, grow by portions and single tokens, are preempted or finish, in random
    order, over a full and a windowed group: no page lost, held twice or freed twice."""
    rng = random.Random(seed)
    windowed = seed % 2 == 1
    cm = _manager(windows=(None, 7) if windowed else (None, None), pages=24, page_size=4, seqs=4)
    live = {}
    next_id = 0
    prompts = [[rng.randrange(5) for _ in range(rng.randrange(1, 30))] for _ in range(6)]
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = next_id
            next_id += 1
            toks = list(rng.choice(prompts))
            cm.admit(rid)
            got = cm.adopt_prefix(rid, toks)
            live[rid] = {"toks": toks, "n": got}
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            st = live[rid]
            grow = rng.choice([1, 1, 2, 5, 11])
            upto = st["n"] + grow
            try:
                cm.reserve(rid, upto)
            except OutOfPages:
                victim = rng.choice(list(live))
                cm.release(victim)
                del live[victim]
                cm.check()
                continue
            while len(st["toks"]) < upto:
                st["toks"].append(rng.randrange(5))
            had = st["n"]
            st["n"] = upto
            cm.commit(rid, upto)
            if had < len(prompts[0]) and rng.random() < 0.5:
                cm.register_prefix(rid, st["toks"])
        elif live:
            rid = rng.choice(list(live))
            cm.release(rid)
            del live[rid]
        cm.check()
    for rid in list(live):
        cm.release(rid)
    cm.check()
    if cm.prefix_cache is not None:
        cm.prefix_cache.evict(10 ** 9)
    assert cm.pages_in_use() == [0, 0]
