"""GPU parity of a long randomised life of one pool: sequences are created, grown, forked, rolled
back, partly evicted to pinned host memory and restored, attended over and freed in a seeded random
order on a pool small enough to run out of pages.  A host-side model keeps the rows each sequence
should hold; after every few operations every live sequence's cells are read back through its block
table and compared with the model (bit for bit after the layout's storage rounding), the whole pool
is compared with the oracle's image of it, and decode attention is checked against the oracle."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, device_sync
from gpu_common import ORACLE_LAYOUT, Twin, check_attn

pytestmark = pytest.mark.gpu

N_LAYERS = 2


class Model:
    """What each live sequence should hold: per layer, the float32 rows as they were appended."""

    def __init__(self):
        self.rows = {}  # seq -> [ (k, v) per layer ], arrays [len, 2, 256]

    def length(self, s):
        return self.rows[s][0][0].shape[0]


def stored(tw, k, v):
    """Rows k, v as the layout stores them: appended to a scratch image through an identity table
    and read back (storage is per cell, so the place does not matter)."""
    n = k.shape[0]
    pages = (n + 15) // 16
    img = oracle.PoolImage(tw.g, max(pages, 1), ORACLE_LAYOUT[tw.layout])
    table = np.arange(max(pages, 1), dtype=np.int32)
    assert img.append(table, 0, k, v, capacity_cells=max(pages, 1) * 16) == 0
    return img.gather(table, 0, n)


def check_everything(tw, model, rng, n_head=16):
    tw.pool.check()
    for layer in range(N_LAYERS):
        tw.assert_pools_equal(layer)
    for s, per_layer in model.rows.items():
        n = model.length(s)
        assert tw.pool.seq_len(s) == n
        if n == 0:
            continue
        for layer in range(N_LAYERS):
            gk, gv = tw.pool.gather(layer, s, 0, n)
            wk, wv = stored(tw, *per_layer[layer])
            assert np.array_equal(gk.view(np.uint32), wk.view(np.uint32)), "K of seq %d layer %d" % (s, layer)
            assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32)), "V of seq %d layer %d" % (s, layer)
    live = [s for s in model.rows if model.length(s) > 0]
    if live:
        pick = [live[i] for i in rng.permutation(len(live))[:3]]
        pos = [model.length(s) - 1 for s in pick]
        layer = int(rng.integers(N_LAYERS))
        q = rng.standard_normal((len(pick), n_head, 256)).astype(np.float32)
        out = tw.decode_attn(layer, pick, pos, q, n_head)
        for i, s in enumerate(pick):
            check_attn(out[i], tw.oracle_attend(layer, s, pos[i], q[i], n_head), "seq %d" % s)


@pytest.mark.parametrize("layout,seed", [(L.LAYOUT_F16, 1), (L.LAYOUT_F16, 2), (L.LAYOUT_Q8V, 3),
                                         (L.LAYOUT_I8H, 4)])
def test_randomised_life_of_a_small_pool(layout, seed):
    rng = np.random.Generator(np.random.PCG64(9100 + seed))
    n_pages, max_seqs = 48, 8
    counts = dict(create=0, append=0, fork=0, truncate=0, free=0, evict=0, no_pages=0, cow=0)
    with Twin(n_layers=N_LAYERS, n_pages=n_pages, layout=layout, max_seqs=max_seqs + 2) as tw:
        host = tw.pool.host_alloc(8 * tw.pool.swap_page_bytes())
        model = Model()

        def empty():
            z = np.zeros((0, 2, 256), np.float32)
            return [(z, z) for _ in range(N_LAYERS)]

        for step in range(300):
            live = list(model.rows)
            op = rng.choice(["create", "append", "append", "append", "fork", "truncate", "free", "evict"])
            if op == "create" and len(live) < max_seqs:
                s = tw.pool.seq_create()
                assert s not in model.rows
                model.rows[s] = empty()
                counts["create"] += 1
            elif op == "append" and live:
                s = int(rng.choice(live))
                n = model.length(s)
                t = int(rng.choice([1, 1, 3, 16, 17, 40, 130]))
                try:
                    pairs = tw.pool.seq_reserve(s, n + t)
                except BkvError as e:
                    assert e.status == L.ERR_NO_PAGES
                    counts["no_pages"] += 1
                    # nothing may have changed; make room by freeing the longest sequence
                    tw.pool.check()
                    victim = max(live, key=model.length)
                    tw.pool.seq_free(victim)
                    del model.rows[victim]
                    continue
                counts["cow"] += len(pairs)
                if pairs:
                    tw.pool.page_copy(pairs)
                    for img in tw.images:
                        img.page_copy(pairs)
                for layer in range(N_LAYERS):
                    k = rng.standard_normal((t, 2, 256)).astype(np.float32)
                    v = (rng.standard_normal((t, 2, 256)) * (3.0 if layer else 0.25)).astype(np.float32)
                    tw.append(layer, [s], [n], [k], [v])
                    ok, ov = model.rows[s][layer]
                    model.rows[s][layer] = (np.concatenate([ok, k]), np.concatenate([ov, v]))
                counts["append"] += 1
            elif op == "fork" and live and len(live) < max_seqs:
                parent = int(rng.choice(live))
                n = int(rng.integers(0, model.length(parent) + 1))
                child = tw.pool.seq_fork(parent, n)
                model.rows[child] = [(k[:n].copy(), v[:n].copy()) for k, v in model.rows[parent]]
                counts["fork"] += 1
            elif op == "truncate" and live:
                s = int(rng.choice(live))
                n = int(rng.integers(max(0, model.length(s) - 40), model.length(s) + 1))
                tw.pool.seq_truncate(s, n)
                model.rows[s] = [(k[:n], v[:n]) for k, v in model.rows[s]]
                counts["truncate"] += 1
            elif op == "free" and len(live) > 5:
                s = int(rng.choice(live))
                tw.pool.seq_free(s)
                del model.rows[s]
                counts["free"] += 1
            elif op == "evict" and live:
                # complete pages held by this sequence alone go out and come back (to other ids)
                s = int(rng.choice(live))
                tab = tw.pool.block_table(s)
                full = model.length(s) // 16
                own = [i for i in range(full) if tw.pool.page_refcount(int(tab[i])) == 1]
                if not own:
                    continue
                lp0 = own[int(rng.integers(len(own)))]
                n = 1
                while n < 8 and lp0 + n in own:
                    n += 1
                free_before = tw.pool.free_pages()
                tw.pool.seq_evict(s, lp0, n, host)
                tw.pool.swap_wait()
                assert tw.pool.free_pages() == free_before + n
                # the freed pages are overwritten on the device before the bytes come back
                junk = tw.pool.seq_create()
                tw.pool.seq_reserve(junk, 16 * n)
                for layer in range(N_LAYERS):
                    k = rng.standard_normal((16 * n, 2, 256)).astype(np.float32)
                    tw.append(layer, [junk], [0], [k], [k])
                tw.pool.seq_free(junk)
                tw.pool.seq_restore(s, lp0, n, host)
                device_sync()
                new = tw.pool.block_table(s)[lp0:lp0 + n]
                # the oracle's image follows: the restored pages hold what the model says
                for layer in range(N_LAYERS):
                    k, v = model.rows[s][layer]
                    rows = slice(16 * lp0, 16 * (lp0 + n))
                    table = np.full(lp0 + n, -1, np.int32)
                    table[lp0:] = new
                    assert tw.images[layer].append(table, 16 * lp0, k[rows], v[rows],
                                                   capacity_cells=16 * (lp0 + n)) == 0
                counts["evict"] += 1
            if step % 20 == 19:
                check_everything(tw, model, rng)
        check_everything(tw, model, rng)
        for s in list(model.rows):
            tw.pool.seq_free(s)
        assert tw.pool.free_pages() == n_pages
        tw.pool.check()
        host.free()
    # the run exercised what it is meant to
    assert counts["append"] >= 30 and counts["fork"] >= 5 and counts["evict"] >= 3, counts
    assert counts["cow"] >= 1 and counts["no_pages"] >= 1, counts
