"""End to end on the GPU: a request that adopts a cached prefix from the prefix tree and
appends only its own suffix attends exactly like a request that recomputed everything
(BASELINE configs[3]: shared prefix pages with refcounts, distinct chunks appended)."""
import numpy as np
import pytest

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
