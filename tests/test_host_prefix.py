"""Host-side prefix tree (page-granular reuse of cached prefixes) on host-only pools: sharing
by refcount, page-aligned matching, least-recently-used eviction, pinned chains, eviction under
allocation pressure, allocator invariants.  No GPU."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, Pool


def host_pool(n_pages=64, max_seqs=8, per_seq=None):
    return Pool(n_pages=n_pages, max_seqs=max_seqs, max_pages_per_seq=per_seq or n_pages, host_only=True)


def toks(seed, n):
    return np.random.Generator(np.random.PCG64(seed)).integers(0, 50000, size=n).astype(np.int32)


def test_publish_then_adopt_shares_pages_by_refcount():
    with host_pool() as pool:
        prompt = toks(1, 100)                         # 6 complete pages + 4 tokens
        a = pool.seq_create()
        pool.seq_reserve(a, 100)
        assert pool.prefix_match(prompt) == 0
        assert pool.prefix_insert(a, prompt) == 6
        assert pool.prefix_stats() == (6, 0, 0)       # held by the tree AND by a: nothing evictable
        ta = pool.block_table(a)
        assert [pool.page_refcount(int(p)) for p in ta[:6]] == [2] * 6 and pool.page_refcount(int(ta[6])) == 1
        # a longer request with the same head: 96 tokens = 6 pages are adopted, never the partial page
        longer = np.concatenate([prompt, toks(2, 50)])
        assert pool.prefix_match(longer) == 96
        b, matched = pool.seq_create_from_prefix(longer)
        assert matched == 96 and pool.seq_len(b) == 96
        assert np.array_equal(pool.block_table(b)[:6], ta[:6])
        assert [pool.page_refcount(int(p)) for p in ta[:6]] == [3] * 6
        # the rest starts on a fresh page: no copy-on-write pair for a page-aligned share
        assert pool.seq_reserve(b, 150) == []
        tb = pool.block_table(b)
        assert len(set(tb[6:10].tolist()) & set(ta.tolist())) == 0
        # a request that diverges inside page 3 shares 3 pages only
        fork = longer.copy()
        fork[3 * 16 + 5] += 1
        assert pool.prefix_match(fork) == 48
        # too short for one page: nothing
        assert pool.prefix_match(prompt[:15]) == 0
        c, m = pool.seq_create_from_prefix(prompt[:15])
        assert m == 0 and pool.seq_len(c) == 0
        pool.check()


def test_first_publisher_wins_and_branches():
    with host_pool() as pool:
        common = toks(3, 48)
        p1 = np.concatenate([common, toks(4, 32)])
        p2 = np.concatenate([common, toks(5, 32)])
        a, b = pool.seq_create(), pool.seq_create()
        pool.seq_reserve(a, 80)
        pool.seq_reserve(b, 80)
        assert pool.prefix_insert(a, p1) == 5
        # b computed the same first 3 pages itself: the tree keeps a's, adds b's two branch pages
        assert pool.prefix_insert(b, p2) == 2
        assert pool.prefix_stats()[0] == 7
        ta, tb = pool.block_table(a), pool.block_table(b)
        assert [pool.page_refcount(int(p)) for p in tb[:3]] == [1] * 3
        assert [pool.page_refcount(int(p)) for p in tb[3:5]] == [2] * 2
        c, m = pool.seq_create_from_prefix(p2)
        assert m == 80
        assert np.array_equal(pool.block_table(c)[:3], ta[:3]) and np.array_equal(pool.block_table(c)[3:5], tb[3:5])
        # listing more tokens than the sequence holds is refused
        with pytest.raises(BkvError) as ei:
            pool.prefix_insert(a, np.concatenate([p1, toks(6, 16)]))
        assert ei.value.status == L.ERR_RANGE
        pool.check()


def test_cached_prefix_outlives_its_sequence_and_lru_eviction_order():
    with host_pool(n_pages=32) as pool:
        prompts = [toks(10 + i, 64) for i in range(3)]          # 4 pages each
        for pr in prompts:
            s = pool.seq_create()
            pool.seq_reserve(s, 64)
            pool.prefix_insert(s, pr)
            pool.seq_free(s)
        assert pool.free_pages() == 32 - 12 and pool.prefix_stats() == (12, 12, 0)
        # use prompt 0 again: it becomes the most recently used
        s0, m = pool.seq_create_from_prefix(prompts[0])
        assert m == 64
        pool.seq_free(s0)
        # evicting 4 pages takes prompt 1 (the oldest), leaf first, whole chain
        assert pool.prefix_evict(4) == 4
        assert pool.prefix_match(prompts[1]) == 0 and pool.prefix_match(prompts[0]) == 64
        assert pool.prefix_match(prompts[2]) == 64
        # evicting 2 more shortens prompt 2 from its end
        assert pool.prefix_evict(2) == 2
        assert pool.prefix_match(prompts[2]) == 32
        assert pool.free_pages() == 32 - 6
        # asking for more than there is frees what is evictable and stops
        assert pool.prefix_evict(100) == 6
        assert pool.prefix_stats() == (0, 0, 0) and pool.free_pages() == 32
        pool.check()


def test_pages_in_use_and_pinned_chains_are_not_evicted():
    with host_pool(n_pages=32) as pool:
        sys_prompt, other = toks(20, 48), toks(21, 48)
        for pr in (sys_prompt, other):
            s = pool.seq_create()
            pool.seq_reserve(s, 48)
            pool.prefix_insert(s, pr)
            pool.seq_free(s)
        assert pool.prefix_pin(sys_prompt) == 48
        assert pool.prefix_stats() == (6, 3, 3)
        user, m = pool.seq_create_from_prefix(other[:32])      # holds 2 of other's 3 pages
        assert m == 32
        assert pool.prefix_evict(10) == 1                      # only other's last page can go
        assert pool.prefix_match(other) == 32 and pool.prefix_match(sys_prompt) == 48
        pool.seq_free(user)
        assert pool.prefix_evict(10) == 2
        assert pool.prefix_match(sys_prompt) == 48             # pinned: still there
        assert pool.prefix_pin(sys_prompt, pin=False) == 48
        assert pool.prefix_evict(10) == 3
        assert pool.free_pages() == 32
        pool.check()


def test_reserve_evicts_cached_prefixes_before_it_reports_no_pages():
    with host_pool(n_pages=16) as pool:
        cached = toks(30, 160)                                 # 10 pages
        s = pool.seq_create()
        pool.seq_reserve(s, 160)
        pool.prefix_insert(s, cached)
        pool.seq_free(s)
        assert pool.free_pages() == 6
        big = pool.seq_create()
        pool.seq_reserve(big, 12 * 16)                         # needs 12 pages: 6 come from the cache
        assert pool.seq_len(big) == 192 and pool.prefix_stats()[0] <= 4
        assert pool.prefix_match(cached) == 16 * pool.prefix_stats()[0]
        # when even that is not enough the error stays what it was
        with pytest.raises(BkvError) as ei:
            pool.seq_reserve(big, 17 * 16)
        assert ei.value.status in (L.ERR_NO_PAGES, L.ERR_RANGE)
        pool.check()


def test_reset_and_clear_drop_every_reference():
    with host_pool(n_pages=16) as pool:
        s = pool.seq_create()
        pool.seq_reserve(s, 64)
        pool.prefix_insert(s, toks(40, 64))
        pool.prefix_clear()
        assert pool.prefix_stats() == (0, 0, 0)
        assert [pool.page_refcount(int(p)) for p in pool.block_table(s)] == [1] * 4
        pool.prefix_insert(s, toks(40, 64))
        pool.reset()
        assert pool.free_pages() == 16 and pool.prefix_stats() == (0, 0, 0)
        pool.check()


def test_randomised_tree_keeps_allocator_invariants():
    rng = np.random.Generator(np.random.PCG64(50))
    base = [toks(60 + i, 16 * 12) for i in range(4)]
    with host_pool(n_pages=96, max_seqs=12, per_seq=24) as pool:
        live = []
        for step in range(400):
            op = rng.integers(0, 6)
            try:
                if op == 0 and len(live) < 10:
                    pr = base[rng.integers(0, 4)][:int(rng.integers(1, 12 * 16))].copy()
                    if rng.integers(0, 3) == 0:
                        pr[int(rng.integers(0, pr.size))] ^= 1           # diverge somewhere
                    s, m = pool.seq_create_from_prefix(pr)
                    assert m % 16 == 0 and m <= pr.size
                    pool.seq_reserve(s, pr.size)
                    live.append((s, pr))
                elif op == 1 and live:
                    s, pr = live[rng.integers(0, len(live))]
                    pool.prefix_insert(s, pr)
                elif op == 2 and live:
                    s, _ = live.pop(rng.integers(0, len(live)))
                    pool.seq_free(s)
                elif op == 3:
                    pool.prefix_evict(int(rng.integers(0, 8)))
                elif op == 4:
                    pool.prefix_pin(base[rng.integers(0, 4)][:64], pin=bool(rng.integers(0, 2)))
                elif op == 5 and live:
                    s, pr = live[rng.integers(0, len(live))]
                    pool.seq_reserve(s, min(pool.seq_len(s) + int(rng.integers(1, 40)), 24 * 16))
            except BkvError as e:
                assert e.status in (L.ERR_NO_PAGES, L.ERR_RANGE), e
            pool.check()
        nodes, evictable, pinned = pool.prefix_stats()
        assert 0 <= evictable <= nodes and 0 <= pinned <= nodes


# ---- lower tiers: on a host-only pool the policy keeps its books, no bytes move ------------------
def publish(pool, prompt):
    s = pool.seq_create()
    pool.seq_reserve(s, prompt.size)
    pool.prefix_insert(s, prompt)
    pool.seq_free(s)


def test_evicted_pages_are_demoted_leaf_first_and_promoted_on_adoption(tmp_path):
    with host_pool(n_pages=32) as pool:
        slab = pool.swap_page_bytes()
        pool.prefix_tiers(6 * slab, str(tmp_path / "t3.bin"), 4 * slab)
        a, b = toks(70, 64), toks(71, 64)                       # 4 pages each
        publish(pool, a)
        publish(pool, b)
        assert pool.prefix_tier_stats() == ((8, 0, 0), (0, 0, 0, 0))
        # 4 pages go: a is the older chain, it goes to host memory from its end -- and stays listed
        assert pool.prefix_evict(4) == 4
        assert pool.free_pages() == 32 - 4
        assert pool.prefix_tier_stats() == ((4, 4, 0), (4, 0, 0, 0))
        assert pool.prefix_match(a) == 64 and pool.prefix_match(b) == 64
        # 3 of b: the arena holds 6, so a's oldest page makes room by going to the file
        assert pool.prefix_evict(3) == 3
        nodes, moved = pool.prefix_tier_stats()
        assert nodes == (1, 6, 1) and moved == (7, 1, 0, 0)
        pool.check()
        # adopting a brings its 4 pages back (3 from host memory, 1 from the file) onto fresh pages
        s, m = pool.seq_create_from_prefix(a)
        assert m == 64 and pool.seq_len(s) == 64
        nodes, moved = pool.prefix_tier_stats()
        assert nodes == (5, 3, 0) and moved == (7, 1, 4, 0)
        assert len(set(pool.block_table(s)[:4].tolist())) == 4
        assert [pool.page_refcount(int(p)) for p in pool.block_table(s)[:4]] == [2] * 4
        pool.check()
        # pages in use stay on the device: only b's last device page can leave
        assert pool.prefix_evict(10) == 1
        assert pool.prefix_tier_stats()[0] == (4, 4, 0)
        pool.seq_free(s)
        pool.check()


def test_lower_tiers_fill_up_and_the_oldest_leaves_are_dropped(tmp_path):
    with host_pool(n_pages=64) as pool:
        slab = pool.swap_page_bytes()
        pool.prefix_tiers(2 * slab, str(tmp_path / "t3.bin"), 3 * slab)
        prompts = [toks(80 + i, 32) for i in range(4)]          # 2 pages each
        for pr in prompts:
            publish(pool, pr)
        assert pool.prefix_evict(8) == 8                        # 8 pages into 2 + 3 slots
        nodes, moved = pool.prefix_tier_stats()
        assert nodes[0] == 0 and nodes[1] == 2 and nodes[2] == 3 and moved[3] == 3
        assert sum(nodes) == 5
        # what is left are heads of chains (a page never outlives its parent)
        left = [pool.prefix_match(pr) for pr in prompts]
        assert sum(left) == 5 * 16 and left[3] == 32            # the newest chain is whole
        pool.check()
        # without a file the host arena's oldest pages are dropped instead
        pool.prefix_tiers(2 * slab)
        assert pool.prefix_tier_stats()[0] == (0, 0, 0)         # resizing drops what the tiers held
        for pr in prompts:
            publish(pool, pr)
        assert pool.prefix_evict(8) == 8
        nodes, _ = pool.prefix_tier_stats()
        assert nodes == (0, 2, 0)
        # tiers off: eviction drops again
        pool.prefix_tiers(0)
        publish(pool, prompts[0])
        assert pool.prefix_evict(2) == 2 and pool.prefix_stats()[0] == 0
        pool.check()


def test_reserve_demotes_and_a_republished_page_returns_without_a_transfer():
    with host_pool(n_pages=16) as pool:
        pool.prefix_tiers(64 * pool.swap_page_bytes())
        cached = toks(90, 160)                                  # 10 pages
        publish(pool, cached)
        big = pool.seq_create()
        pool.seq_reserve(big, 12 * 16)                          # 6 free + 6 demoted
        nodes, moved = pool.prefix_tier_stats()
        assert nodes[1] >= 6 and moved[0] == nodes[1] and pool.prefix_match(cached) == 160
        pool.seq_free(big)
        # a sequence that recomputed the whole prompt lists it again: its pages replace the host copies
        s = pool.seq_create()
        pool.seq_reserve(s, 160)
        assert pool.prefix_insert(s, cached) == 0
        nodes2, moved2 = pool.prefix_tier_stats()
        assert nodes2 == (10, 0, 0) and moved2[2] == 0          # nothing was promoted: no transfer
        # the pages that never left the device keep their first publisher's copies
        assert [pool.page_refcount(int(p)) for p in pool.block_table(s)[:10]] == \
            [1] * nodes[0] + [2] * (10 - nodes[0])
        pool.check()


def test_promotion_stops_where_the_device_has_no_page_left():
    with host_pool(n_pages=8, max_seqs=4, per_seq=8) as pool:
        pool.prefix_tiers(64 * pool.swap_page_bytes())
        a = toks(95, 96)                                        # 6 pages
        publish(pool, a)
        assert pool.prefix_evict(6) == 6
        hog = pool.seq_create()
        pool.seq_reserve(hog, 5 * 16)                           # 3 pages stay free
        s, m = pool.seq_create_from_prefix(a)
        assert m == 48                                          # 3 pages came back, the chain's head
        assert pool.prefix_tier_stats()[0] == (3, 3, 0)
        assert pool.prefix_match(a) == 96
        pool.check()


def test_prefetch_promotes_ahead_of_the_request():
    with host_pool(n_pages=16, max_seqs=4, per_seq=16) as pool:
        pool.prefix_tiers(64 * pool.swap_page_bytes())
        a, b = toks(96, 80), toks(97, 80)                       # 5 pages each
        publish(pool, a)
        publish(pool, b)
        assert pool.prefix_evict(10) == 10 and pool.prefix_tier_stats()[0] == (0, 10, 0)
        assert pool.prefix_prefetch(a) == 80                    # a is back on the device, nobody holds it
        assert pool.prefix_tier_stats()[0] == (5, 5, 0) and pool.prefix_stats()[1] == 5
        assert pool.prefix_prefetch(a[:40]) == 32               # already there: nothing moves
        assert pool.prefix_tier_stats()[1][2] == 5
        s, m = pool.seq_create_from_prefix(a)                   # the request finds it on the device
        assert m == 80 and pool.prefix_tier_stats()[1][2] == 5
        # with 11 pages held elsewhere only part of b can come back
        hog = pool.seq_create()
        pool.seq_reserve(hog, 9 * 16)
        assert pool.prefix_prefetch(b) == 32
        assert pool.prefix_match(b) == 80
        pool.check()


def test_randomised_tiered_tree_keeps_every_invariant(tmp_path):
    rng = np.random.Generator(np.random.PCG64(51))
    base = [toks(160 + i, 16 * 12) for i in range(5)]
    with host_pool(n_pages=48, max_seqs=12, per_seq=24) as pool:
        slab = pool.swap_page_bytes()
        pool.prefix_tiers(10 * slab, str(tmp_path / "t3.bin"), 12 * slab)
        live = []
        for step in range(600):
            op = rng.integers(0, 7)
            try:
                if op == 0 and len(live) < 10:
                    pr = base[rng.integers(0, 5)][:int(rng.integers(1, 12 * 16))].copy()
                    if rng.integers(0, 3) == 0:
                        pr[int(rng.integers(0, pr.size))] ^= 1
                    s, m = pool.seq_create_from_prefix(pr)
                    assert m % 16 == 0 and m <= pr.size
                    live.append((s, pr))
                    pool.seq_reserve(s, pr.size)
                elif op == 1 and live:
                    s, pr = live[rng.integers(0, len(live))]
                    if pool.seq_len(s) >= pr.size:
                        pool.prefix_insert(s, pr)
                elif op == 2 and live:
                    s, _ = live.pop(rng.integers(0, len(live)))
                    pool.seq_free(s)
                elif op == 3:
                    pool.prefix_evict(int(rng.integers(0, 8)))
                elif op == 4:
                    pool.prefix_pin(base[rng.integers(0, 5)][:64], pin=bool(rng.integers(0, 2)))
                elif op == 5 and live:
                    s, pr = live[rng.integers(0, len(live))]
                    pool.seq_reserve(s, min(pool.seq_len(s) + int(rng.integers(1, 40)), 24 * 16))
                elif op == 6 and step % 97 == 0:
                    pool.prefix_tiers(int(rng.integers(1, 12)) * slab, str(tmp_path / "t3.bin"),
                                      int(rng.integers(0, 12)) * slab)
            except BkvError as e:
                assert e.status in (L.ERR_NO_PAGES, L.ERR_RANGE), e
            pool.check()
            nodes, moved = pool.prefix_tier_stats()
            assert sum(nodes) == pool.prefix_stats()[0]
        nodes, moved = pool.prefix_tier_stats()
        assert moved[0] > 0 and moved[1] > 0 and moved[2] > 0


def test_a_very_long_chain_is_walked_without_recursion():
    # one node per page: a 480k-token prompt is a chain 30000 nodes deep
    n = 30000
    with host_pool(n_pages=n + 8, max_seqs=2, per_seq=n + 8) as pool:
        pool.prefix_tiers(n * pool.swap_page_bytes())
        prompt = toks(99, n * 16)
        publish(pool, prompt)
        assert pool.prefix_stats() == (n, n, 0)
        pool.check()
        assert pool.prefix_evict(n) == n
        assert pool.prefix_tier_stats()[0] == (0, n, 0)
        s, m = pool.seq_create_from_prefix(prompt)
        assert m == n * 16
        pool.seq_free(s)
        pool.check()
        pool.prefix_clear()
        assert pool.prefix_stats() == (0, 0, 0) and pool.free_pages() == n + 8
