"""GPU parity of copy-on-write page copy, prefix sharing and the VRAM <-> pinned-host swap.
Byte moves: everything is compared bit for bit."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, Stream, device_sync
from gpu_common import Twin, check_attn
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu


def test_page_copy_moves_every_layer_and_leaves_the_rest_alone():
    rng = np.random.Generator(np.random.PCG64(51))
    with Twin(n_layers=3, n_pages=40, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 16 * 10)
        for layer in range(3):
            x = rng.standard_normal((160, 2, 256)).astype(np.float32)
            y = rng.standard_normal((160, 2, 256)).astype(np.float32)
            tw.append(layer, [s], [0], [x], [y])
        tab = tw.pool.block_table(s)
        used = set(tab.tolist())
        free = [p for p in range(40) if p not in used]
        pairs = [(int(tab[0]), free[0]), (int(tab[7]), free[5]), (int(tab[9]), free[2])]
        tw.pool.page_copy(pairs)
        device_sync()
        for img in tw.images:
            img.page_copy(pairs)
        for layer in range(3):
            tw.assert_pools_equal(layer)
        tw.pool.page_copy([])  # empty list is a no-op


@pytest.mark.parametrize("prefix", [2048, 2040])
def test_config4_shared_prefix_chunked_prefill_and_cow(prefix):
    """BASELINE config 4: four sequences share a prefix through shared page ids with refcounts;
    each appends a distinct 1024-token chunk.  A 2048-token prefix ends on a page boundary (no
    copy may happen); a 2040-token prefix leaves a shared partial page that each writer but the
    last must copy before its first append."""
    rng = np.random.Generator(np.random.PCG64(60 + prefix))
    with Twin(n_pages=512, max_seqs=8) as tw:
        root = tw.pool.seq_create()
        fill(tw, root, prefix, rng, chunk=512)
        kids = [tw.pool.seq_fork(root, prefix) for _ in range(3)]
        seqs = [root] + kids
        shared = tw.pool.block_table(root).copy()
        assert all(tw.pool.page_refcount(int(p)) == 4 for p in shared)
        before = [tw.pool.gather(0, s, 0, prefix) for s in seqs]
        n_copies = 0
        for s in seqs:
            pairs = tw.pool.seq_reserve(s, prefix + 1024)
            n_copies += len(pairs)
            tw.pool.page_copy(pairs)
            for img in tw.images:
                img.page_copy(pairs)
            k = rng.standard_normal((1024, 2, 256)).astype(np.float32)
            v = rng.standard_normal((1024, 2, 256)).astype(np.float32)
            tw.append(0, [s], [prefix], [k], [v])
        assert n_copies == (0 if prefix % 16 == 0 else 3)
        tw.assert_pools_equal()
        tw.pool.check()
        full = prefix // 16
        for s, (bk, bv) in zip(seqs, before):
            tab = tw.pool.block_table(s)
            assert np.array_equal(tab[:full], shared[:full])       # full prefix pages stay shared
            gk, gv = tw.pool.gather(0, s, 0, prefix)
            assert np.array_equal(gk, bk) and np.array_equal(gv, bv)  # nobody's prefix changed
        tails = [int(tw.pool.block_table(s)[full]) for s in seqs]
        assert len(set(tails)) == 4                                 # each writer has its own page
        q = rng.standard_normal((4, 16, 256)).astype(np.float32)
        pos = [prefix + 1023] * 4
        out = tw.decode_attn(0, seqs, pos, q, 16)
        for i, s in enumerate(seqs):
            check_attn(out[i], tw.oracle_attend(0, s, pos[i], q[i], 16), "shared-prefix seq %d" % i)


def test_swap_out_poison_swap_in_is_bit_exact():
    """Evict a seeded 25 % of cold pages to pinned host memory, overwrite them in VRAM, swap
    back: every pool byte must return."""
    rng = np.random.Generator(np.random.PCG64(71))
    with Twin(n_layers=2, n_pages=96, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 16 * 80)
        for layer in range(2):
            x = rng.standard_normal((1280, 2, 256)).astype(np.float32)
            y = rng.standard_normal((1280, 2, 256)).astype(np.float32)
            tw.append(layer, [s], [0], [x], [y])
        tab = tw.pool.block_table(s)
        cold = rng.choice(tab, size=20, replace=False).astype(np.int32)
        slab = tw.pool.swap_page_bytes()
        assert slab == 2 * 32768
        host = tw.pool.host_alloc(20 * slab)
        st = Stream()
        tw.pool.swap_out(cold, host, st)
        tw.pool.swap_wait()
        # host slab layout: [page][layer][K page | V page]
        hv = host.view().reshape(20, 2, 2, 16384)
        for i, p in enumerate(cold):
            for layer in range(2):
                assert np.array_equal(hv[i, layer, 0], tw.images[layer].k.reshape(-1, 16384)[p])
                assert np.array_equal(hv[i, layer, 1], tw.images[layer].v.reshape(-1, 16384)[p])
        # poison the evicted pages in VRAM by copying a garbage page over them
        junk = [p for p in range(96) if p not in set(tab.tolist())][0]
        tw.pool.page_copy([(junk, int(p)) for p in cold], st)
        st.sync()
        assert not np.array_equal(tw.pool.read_layer(0, 0), tw.images[0].k)
        tw.pool.swap_in(cold, host, st)
        tw.pool.swap_fence(st)
        st.sync()
        for layer in range(2):
            tw.assert_pools_equal(layer)
        host.free()
        st.close()


def test_evict_and_restore_through_the_allocator():
    rng = np.random.Generator(np.random.PCG64(73))
    with Twin(n_pages=64, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, 16 * 20 + 5, rng)
        kb, vb = tw.pool.gather(0, s, 0, 325)
        host = tw.pool.host_alloc(8 * tw.pool.swap_page_bytes())
        tw.pool.seq_evict(s, 4, 8, host)
        tw.pool.swap_wait()
        assert tw.pool.block_table(s)[4:12].tolist() == [-1] * 8 and tw.pool.free_pages() == 64 - 13
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        with pytest.raises(BkvError) as ei:
            tw.decode_attn(0, [s], [324], q, 16)
        assert ei.value.status == L.ERR_STATE
        # other sequences reuse the freed pages meanwhile
        other = tw.pool.seq_create()
        fill(tw, other, 16 * 30, rng)
        tw.pool.seq_restore(s, 4, 8, host)
        device_sync()
        ka, va = tw.pool.gather(0, s, 0, 325)
        assert np.array_equal(ka, kb) and np.array_equal(va, vb)
        tw.pool.check()
        host.free()


def test_two_streams_interleave_on_one_pool_without_host_synchronisation():
    # Two request streams share a pool: each grows its own sequence (2000 tokens to begin with) one
    # token at a time (a table update, an append and a decode attention per step) and forks it
    # every 16 steps (a copy-on-write page copy), 150 steps each, the calls of the two interleaved
    # and nothing synchronised on the host until the end -- the parameter ring and the block-table
    # uploads wrap around several times, and the attention calls of the two streams, which share
    # the pool's split-K workspace, would overlap on the device if the pool did not order them.
    # Every output and the final K/V rows equal what the same work gives when it is run on one
    # stream with a synchronisation after every call.
    from breccia_amd.kv import DeviceBuffer, Pool, Stream, device_sync

    def run(async_two_streams):
        rng = np.random.Generator(np.random.PCG64(444))
        pool = Pool(n_pages=400, max_seqs=40)
        pool.set_free_order(rng.permutation(400).astype(np.int32))
        streams = [Stream(), Stream()] if async_two_streams else [Stream()] * 2
        seqs = [pool.seq_create(), pool.seq_create()]
        steps, base = 150, 2000
        head = DeviceBuffer.from_numpy(rng.standard_normal((base, 2, 256), dtype=np.float32))
        for s in seqs:
            pool.seq_reserve(s, base)
            pool.append(0, [s], [0], [base], head, head, streams[0])
        streams[0].sync()
        k = [DeviceBuffer.from_numpy(rng.standard_normal((steps, 2, 256), dtype=np.float32)) for _ in range(2)]
        v = [DeviceBuffer.from_numpy(rng.standard_normal((steps, 2, 256), dtype=np.float32)) for _ in range(2)]
        q = [DeviceBuffer.from_numpy(rng.standard_normal((steps, 16, 256), dtype=np.float32)) for _ in range(2)]
        out = [DeviceBuffer(steps * 16 * 256 * 4) for _ in range(2)]
        row, qrow = 2 * 256 * 4, 16 * 256 * 4
        for t in range(steps):
            for i in range(2):
                st = streams[i]
                if t and t % 16 == 5:
                    # fork inside a page and drop the parent: the child's next write copies the page
                    child = pool.seq_fork(seqs[i], base + t)
                    old = seqs[i]
                    seqs[i] = child
                    pairs = pool.seq_reserve(child, base + t + 1)
                    assert len(pairs) == 1
                    pool.page_copy(pairs, st)
                    pool.seq_free(old)
                else:
                    pool.seq_reserve(seqs[i], base + t + 1)
                pool.append(0, [seqs[i]], [base + t], [1], k[i].at(t * row), v[i].at(t * row), st)
                pool.decode_attn(0, [seqs[i]], [base + t], 16, q[i].at(t * qrow), out[i].at(t * qrow), 1.0 / 16.0, stream=st)
                if not async_two_streams:
                    st.sync()
        for st in set(streams):
            st.sync()
        device_sync()
        res = [o.download(np.float32) for o in out]
        rows = [pool.gather(0, s, 0, base + steps) for s in seqs]
        pool.check()
        for b in k + v + q + out + [head]:
            b.free()
        pool.destroy()
        return res, rows

    a_out, a_rows = run(True)
    b_out, b_rows = run(False)
    for i in range(2):
        assert np.array_equal(a_out[i].view(np.uint32), b_out[i].view(np.uint32)), i
        assert np.array_equal(a_rows[i][0], b_rows[i][0]) and np.array_equal(a_rows[i][1], b_rows[i][1]), i
        assert np.abs(a_out[i]).max() > 0


def test_table_updates_flushed_on_one_stream_are_seen_on_another():
    # The block-table changes of two sequences are pushed to the device by whichever call comes
    # next -- here a call on stream 1, queued behind a long append -- and the other sequence's
    # append and attention follow at once on stream 0: they wait for that push on the device.
    from breccia_amd.kv import DeviceBuffer, Pool, Stream, device_sync
    rng = np.random.Generator(np.random.PCG64(445))
    s0, s1 = Stream(), Stream()
    with Pool(n_pages=1200, max_seqs=8, max_pages_per_seq=600) as pool:
        pool.set_free_order(rng.permutation(1200).astype(np.int32))
        big_rows = DeviceBuffer.from_numpy(rng.standard_normal((8192, 2, 256), dtype=np.float32))
        rows = rng.standard_normal((40, 2, 256), dtype=np.float32)
        rd = DeviceBuffer.from_numpy(rows)
        q = rng.standard_normal((1, 16, 256), dtype=np.float32)
        qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
        c = pool.seq_create()
        pool.seq_reserve(c, 8192)
        for rep in range(5):
            a, b = pool.seq_create(), pool.seq_create()
            pool.append(0, [c], [0], [8192], big_rows, big_rows, s1)     # long work on stream 1
            pool.seq_reserve(a, 40)
            pool.seq_reserve(b, 40)
            pool.append(0, [b], [0], [40], rd, rd, s1)                   # pushes both tables, on stream 1
            pool.append(0, [a], [0], [40], rd, rd, s0)                   # stream 0, nothing left to push
            pool.decode_attn(0, [a], [39], 16, qd, od, 1.0 / 16.0, stream=s0)
            s0.sync()
            out_a = od.download(np.float32, stream=s0).copy()
            s1.sync()
            ka, va = pool.gather(0, a, 0, 40)
            kb, vb = pool.gather(0, b, 0, 40)
            assert np.array_equal(ka, kb) and np.array_equal(va, vb) and np.abs(ka).max() > 1.0
            pool.decode_attn(0, [b], [39], 16, qd, od, 1.0 / 16.0, stream=s1)
            s1.sync()
            out_b = od.download(np.float32, stream=s1)
            assert np.array_equal(out_a.view(np.uint32), out_b.view(np.uint32))
            pool.seq_free(a)
            pool.seq_free(b)
            pool.check()
        device_sync()
        for x in (big_rows, rd, qd, od):
            x.free()


def test_bounded_waits_time_out_and_the_work_still_completes():
    """crates/breccia-vk/src/ctx.rs:1545-1553: the reference's device waits have a deadline and report
    instead of hanging.  A stream with a queue of bulk appends behind it: a wait with a deadline of 0 ms
    is a query and returns TIMEOUT (with what it waited for), nothing is cancelled, a wait with a real
    deadline then succeeds and the pool holds every appended byte.  The same on the pool's side stream
    with page transfers in flight."""
    from breccia_amd.kv import DeviceBuffer

    rng = np.random.Generator(np.random.PCG64(77))
    T = 8192
    with Twin(n_pages=T // 16 + 600, max_seqs=4, max_pages_per_seq=T // 16 + 8) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, T)
        k = rng.standard_normal((T, 2, 256)).astype(np.float32)
        v = rng.standard_normal((T, 2, 256)).astype(np.float32)
        kd, vd = DeviceBuffer.from_numpy(k), DeviceBuffer.from_numpy(v)
        st = Stream()
        st.wait(0)                                              # an idle stream: a query succeeds
        for _ in range(400):                                    # some 10 ms of device work, enqueued in less
            tw.pool.append(0, [s], [0], [T], kd, vd, st)
        with pytest.raises(BkvError) as ei:
            st.wait(0)
        assert ei.value.status == L.ERR_TIMEOUT and "caller stream" in ei.value.message
        assert "nothing was cancelled" in ei.value.message
        st.wait(10000)
        assert tw.images[0].append(tw.pool.block_table(s), 0, k, v) == 0
        tw.assert_pools_equal()
        # the side stream: 512 pages out to pinned host memory
        pages = tw.pool.block_table(s)[:512].astype(np.int32)
        host = tw.pool.host_alloc(512 * tw.pool.swap_page_bytes())
        for _ in range(200):                                    # the transfers queue up behind these
            tw.pool.append(0, [s], [0], [T], kd, vd, st)
        tw.pool.swap_out(pages, host, st)
        with pytest.raises(BkvError) as ei:
            tw.pool.swap_wait_for(0)
        assert ei.value.status == L.ERR_TIMEOUT and "side stream" in ei.value.message
        tw.pool.swap_wait()
        hv = host.view().reshape(512, 2, 16384)
        assert np.array_equal(hv[511, 0], tw.images[0].k.reshape(-1, 16384)[pages[511]])
        host.free()
        kd.free()
        vd.free()
