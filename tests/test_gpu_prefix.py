"""End to end on the GPU: a request that adopts a cached prefix from the prefix tree and
appends only its own suffix attends exactly like a request that recomputed everything
(BASELINE configs[3]: shared prefix pages with refcounts, distinct chunks appended)."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, Stream
from gpu_common import Twin, check_attn

pytestmark = pytest.mark.gpu


def kv_of(tokens, pos0, seed):
    """Deterministic K/V rows of (token id, position): what a model would recompute."""
    out_k = np.empty((len(tokens), 2, 256), dtype=np.float32)
    out_v = np.empty((len(tokens), 2, 256), dtype=np.float32)
    for i, t in enumerate(tokens):
        g = np.random.Generator(np.random.PCG64([seed, int(t), pos0 + i]))
        out_k[i] = g.standard_normal((2, 256), dtype=np.float32)
        out_v[i] = g.standard_normal((2, 256), dtype=np.float32)
    return out_k, out_v


def test_adopted_prefix_attends_like_a_recomputed_one():
    rng = np.random.Generator(np.random.PCG64(900))
    prefix = rng.integers(0, 32000, size=2040).astype(np.int32)      # 127 pages + 8 tokens
    suffixes = [rng.integers(0, 32000, size=200).astype(np.int32) for _ in range(3)]
    with Twin(n_pages=1024, max_seqs=12) as tw:
        pool = tw.pool
        pool.set_free_order(rng.permutation(1024).astype(np.int32))
        # the first request computes the prefix and publishes it
        a = pool.seq_create()
        pool.seq_reserve(a, prefix.size)
        k, v = kv_of(prefix, 0, 7)
        tw.append(0, [a], [0], [k], [v])
        assert pool.prefix_insert(a, prefix) == 127
        pool.seq_free(a)
        adopted, fresh = [], []
        for sfx in suffixes:
            full = np.concatenate([prefix, sfx])
            # adopting request: shares 127 pages, appends tokens 2032.. only
            s, m = pool.seq_create_from_prefix(full)
            assert m == 2032
            assert pool.seq_reserve(s, full.size) == []              # page-aligned share: no COW copy
            k, v = kv_of(full[m:], m, 7)
            tw.append(0, [s], [m], [k], [v])
            adopted.append(s)
            # control: recomputes everything on its own pages
            c = pool.seq_create()
            pool.seq_reserve(c, full.size)
            k, v = kv_of(full, 0, 7)
            tw.append(0, [c], [0], [k], [v])
            fresh.append(c)
        tw.assert_pools_equal()
        shared = pool.block_table(adopted[0])[:127]
        assert all(np.array_equal(pool.block_table(s)[:127], shared) for s in adopted)
        assert all(pool.page_refcount(int(p)) == 4 for p in shared)   # tree + three requests
        pos = [prefix.size + 199] * 3
        q = rng.standard_normal((3, 16, 256)).astype(np.float32)
        out_adopted = tw.decode_attn(0, adopted, pos, q, 16)
        out_fresh = tw.decode_attn(0, fresh, pos, q, 16)
        assert np.array_equal(out_adopted.view(np.uint32), out_fresh.view(np.uint32))
        for i in range(3):
            check_attn(out_adopted[i], tw.oracle_attend(0, adopted[i], pos[i], q[i], 16), "adopted %d" % i)
        # the cache cannot be evicted from under its users; once they are gone it can
        assert pool.prefix_evict(1000) == 0
        before = tw.decode_attn(0, adopted[:1], pos[:1], q[:1], 16)
        for s in adopted:
            pool.seq_free(s)
        assert pool.prefix_evict(1000) == 127
        pool.check()
        assert np.array_equal(before, out_adopted[:1])


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V])
def test_demoted_prefix_comes_back_from_host_memory_and_from_disk_bit_for_bit(tmp_path, layout):
    # 50 cached pages of a two-layer pool leave the device (40 fit the host arena, 10 go on to the
    # file), the whole device pool is poisoned, and a request that adopts the prefix gets every
    # byte of both layers back: same pool bytes as a request that recomputed the prefix, and
    # bit-identical attention -- on a stream of the caller's, with no host synchronisation in
    # between (later calls wait for the transfers on the device)
    rng = np.random.Generator(np.random.PCG64(901 + layout))
    prefix = rng.integers(0, 32000, size=50 * 16 + 5).astype(np.int32)
    with Twin(n_layers=2, n_pages=128, max_seqs=8, layout=layout) as tw:
        pool = tw.pool
        pool.set_free_order(rng.permutation(128).astype(np.int32))
        slab = pool.swap_page_bytes()
        pool.prefix_tiers(40 * slab, str(tmp_path / "tier3.bin"), 64 * slab)
        a = pool.seq_create()
        pool.seq_reserve(a, prefix.size)
        for layer in range(2):
            k, v = kv_of(prefix, 0, 11 + layer)
            tw.append(layer, [a], [0], [k], [v])
        assert pool.prefix_insert(a, prefix) == 50
        pool.seq_free(a)
        assert pool.prefix_evict(50) == 50
        assert pool.prefix_tier_stats() == ((0, 40, 10), (50, 10, 0, 0))
        assert pool.free_pages() == 128
        pool.fill(0xFF)
        # control: recomputes everything; adopter: takes the 50 pages from the tiers
        c = pool.seq_create()
        pool.seq_reserve(c, prefix.size)
        for layer in range(2):
            k, v = kv_of(prefix, 0, 11 + layer)
            tw.append(layer, [c], [0], [k], [v])
        st = Stream()
        s, m = pool.seq_create_from_prefix(prefix)
        assert m == 800
        assert pool.prefix_tier_stats() == ((50, 0, 0), (50, 10, 50, 0))
        pool.seq_reserve(s, prefix.size)
        for layer in range(2):
            k, v = kv_of(prefix[800:], 800, 11 + layer)
            tw.append(layer, [s], [800], [k], [v], stream=st)
        q = rng.standard_normal((2, 16, 256)).astype(np.float32)
        for layer in range(2):
            out = tw.decode_attn(layer, [s, c], [prefix.size - 1] * 2, q[[0, 0]], 16, stream=st)
            assert np.all(np.isfinite(out))
            assert np.array_equal(out[0].view(np.uint32), out[1].view(np.uint32)), layer
        ts, tc = pool.block_table(s), pool.block_table(c)
        assert len(set(ts[:50].tolist()) & set(tc[:50].tolist())) == 0
        for layer in range(2):
            for which in range(2):
                img = pool.read_layer(layer, which)
                pb = img.size // 128
                for i in range(50):
                    ps, pc = int(ts[i]), int(tc[i])
                    assert np.array_equal(img[ps * pb:(ps + 1) * pb], img[pc * pb:(pc + 1) * pb]), (layer, which, i)
        pool.seq_free(s)
        pool.seq_free(c)
        pool.check()
        # once more through the tiers, with the host arena alone (a smaller one: 30 pages are dropped)
        pool.prefix_tiers(20 * slab)
        assert pool.prefix_evict(50) == 50
        nodes, _ = pool.prefix_tier_stats()
        assert nodes == (0, 20, 0) and pool.prefix_match(prefix) == 320
        pool.fill(0xEE)
        # promotion ahead of the request: the request then finds its pages on the device
        assert pool.prefix_prefetch(prefix) == 320
        promoted = pool.prefix_tier_stats()[1][2]
        s, m = pool.seq_create_from_prefix(prefix)
        assert m == 320 and pool.prefix_tier_stats()[1][2] == promoted
        c = pool.seq_create()
        pool.seq_reserve(c, 320)
        k, v = kv_of(prefix[:320], 0, 11)
        tw.append(0, [c], [0], [k], [v])
        out = tw.decode_attn(0, [s, c], [319, 319], q[[1, 1]], 16)
        assert np.array_equal(out[0].view(np.uint32), out[1].view(np.uint32))
        pool.check()


def test_randomised_requests_through_the_tiers_always_read_their_own_bytes(tmp_path):
    # Requests over a few prompts with shared heads come and go on a pool too small for them, with
    # a small host arena and a small file below it, so that pages are demoted, spilled, dropped,
    # promoted and republished in every order.  Whatever a request adopts must hold exactly the
    # K/V of its own tokens: every gathered row is compared with the rows the first computation of
    # that (token, position) stored.
    rng = np.random.Generator(np.random.PCG64(902))
    heads = [rng.integers(0, 32000, size=16 * 6).astype(np.int32) for _ in range(2)]
    prompts = []
    for i in range(6):
        tail = rng.integers(0, 32000, size=16 * int(rng.integers(4, 12)) + int(rng.integers(0, 16))).astype(np.int32)
        prompts.append(np.concatenate([heads[i % 2], tail]))
    with Twin(n_layers=2, n_pages=40, max_seqs=6, max_pages_per_seq=24) as tw:
        pool = tw.pool
        slab = pool.swap_page_bytes()
        pool.prefix_tiers(14 * slab, str(tmp_path / "tier3.bin"), 20 * slab)
        stored = {}                                    # (layer, prompt, page) -> (k rows, v rows) as gathered

        def serve(i):
            pr = prompts[i]
            s, m = pool.seq_create_from_prefix(pr)
            assert m % 16 == 0 and m <= pr.size
            try:
                pool.seq_reserve(s, pr.size)
            except BkvError:
                pool.seq_free(s)                       # no room for the rest of it: the request goes away
                raise
            for layer in range(2):
                if m < pr.size:
                    k, v = kv_of(pr[m:], m, 21 + layer)
                    tw.append(layer, [s], [m], [k], [v])
                gk, gv = pool.gather(layer, s, 0, pr.size - pr.size % 16)
                for pg in range(pr.size // 16):
                    rows = (gk[16 * pg:16 * pg + 16], gv[16 * pg:16 * pg + 16])
                    key = (layer, tuple(pr[:16 * pg + 16].tolist()))
                    if key not in stored:
                        assert pg * 16 >= m, "an adopted page nobody computed"
                        stored[key] = (rows[0].copy(), rows[1].copy())
                    else:
                        assert np.array_equal(rows[0], stored[key][0]) and np.array_equal(rows[1], stored[key][1]), \
                            (i, layer, pg, m)
            pool.prefix_insert(s, pr)
            return s

        live = []
        for step in range(80):
            op = int(rng.integers(0, 4))
            try:
                if op <= 1 and len(live) < 3:
                    live.append(serve(int(rng.integers(0, 6))))
                elif op == 2 and live:
                    pool.seq_free(live.pop(int(rng.integers(0, len(live)))))
                elif op == 3:
                    pool.prefix_evict(int(rng.integers(1, 12)))
            except BkvError as e:
                assert e.status == L.ERR_NO_PAGES, e
            pool.check()
        nodes, moved = pool.prefix_tier_stats()
        assert moved[0] > 20 and moved[1] > 0 and moved[2] > 20, moved
