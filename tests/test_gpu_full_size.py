"""BASELINE.json's batched configurations at full size on the GPU.

configs[2] (batch 8, contexts 1k..32k, f16): parity against the oracle on every (sequence, head).
configs[4] (batch 16, contexts 8k..128k, int8 K/V with f16 scales): the oracle attends over the
rows read back through bkv_gather for a seeded subset of sequences (shortest, median, longest --
all 16 heads each; the full f64 oracle over all 16 sequences is ~10^10 MACs), plus
size-independent properties on all of them: the batched call equals the per-sequence call to
1e-6, and every output is a convex combination of V rows (bounded by the largest |v|).
configs[3] shape (4 sequences, 2048-token prefix + 1024-token chunk) through the chunk kernel on
all three layouts: sampled tokens against the oracle, the chunk's tail against the decode kernel.
The fused step (bkv_decode_step) on configs[2] (f16 and f16 K + q8_0 V) and on configs[4] at the same
sizes: outputs bit-identical to bkv_append + bkv_decode_attn, the new rows' pool bytes against the
oracle's encoders.  configs[3] end to end on one pool: shared 2040-token prefix, binary16 chunks
through bkv_append_f16, the copy-on-write copies, a seeded quarter of the pages out to pinned host
memory, poisoned, back, every pool byte against the oracle's image.
In the attention checks of this file the oracle attends over the rows read back through bkv_gather
(its own kernel and address arithmetic) unless a test says it keeps an oracle image: the appends
that stored those rows are compared byte for byte with the oracle's image elsewhere
(tests/test_gpu_append.py, the configs[1] and configs[3] tests below).
A 300k-page pool with a sequence on the highest page ids (byte offsets past 2^32): every kernel of the
path there against a twin on the lowest pages and the oracle."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import DeviceBuffer, Pool, device_sync
from gpu_common import REF_BAR_MAX_REL, check_attn
from helpers import max_abs

pytestmark = pytest.mark.gpu
N_Q, N_KV, HD = 16, 2, 256


def build(rng, n_seqs, lo, hi, layout, occupancy=0.6):
    ctx = []
    for _ in range(n_seqs):
        c = int(rng.integers(lo, hi + 1))
        if c % 16 == 0:
            c -= 3
        ctx.append(c)
    live = sum((c + 15) // 16 for c in ctx)
    n_pages = int(np.ceil(live / occupancy))
    pool = Pool(n_layers=1, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, layout=layout,
                max_seqs=n_seqs + 1, max_pages_per_seq=max(ctx) // 16 + 2)
    pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
    seqs = [pool.seq_create() for _ in ctx]
    grown = [0] * n_seqs
    while any(g < c for g, c in zip(grown, ctx)):   # deal pages round-robin: interleaved tables
        for i, s in enumerate(seqs):
            if grown[i] < ctx[i]:
                grown[i] = min(ctx[i], grown[i] + 16 * 8)
                pool.seq_reserve(s, grown[i])
    return pool, seqs, ctx


def fill_tiled(pool, seqs, ctx, rng, tile=8192):
    """Append N(0,1) rows; one random tile of `tile` tokens per sequence offset keeps the host
    side small while every sequence still holds distinct data (a different window per chunk)."""
    src_k = rng.standard_normal((3 * tile, N_KV, HD), dtype=np.float32)
    src_v = rng.standard_normal((3 * tile, N_KV, HD), dtype=np.float32)
    kd, vd = DeviceBuffer.from_numpy(src_k), DeviceBuffer.from_numpy(src_v)
    row = N_KV * HD * 4
    for i, (s, c) in enumerate(zip(seqs, ctx)):
        at = 0
        while at < c:
            n = min(tile, c - at)
            off = int(rng.integers(0, 2 * tile)) * row
            pool.append(0, [s], [at], [n], kd.at(off), vd.at(off))
            at += n
    device_sync()
    kd.free()
    vd.free()


def run_attn(pool, seqs, pos, q):
    qd = DeviceBuffer.from_numpy(q)
    od = DeviceBuffer(q.nbytes)
    pool.decode_attn(0, seqs, pos, N_Q, qd, od, 1.0 / 16.0)
    device_sync()
    out = od.download(np.float32).reshape(len(seqs), N_Q, HD)
    qd.free()
    od.free()
    return out


def oracle_for(pool, seq, pos, q):
    k, v = pool.gather(0, seq, 0, pos + 1)
    return oracle.attend(q, k, v, oracle.dense_cells(pos), pos, N_Q, N_KV, HD, threads=8), v


def test_config3_batch8_mixed_1k_32k_all_heads():
    rng = np.random.Generator(np.random.PCG64(20250003))
    pool, seqs, ctx = build(rng, 8, 1024, 32768, L.LAYOUT_F16)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        # the step: one more token per sequence, then attention at the new position
        for s, c in zip(seqs, ctx):
            pool.seq_reserve(s, c + 1)
        new = rng.standard_normal((8, N_KV, HD), dtype=np.float32)
        nd = DeviceBuffer.from_numpy(new)
        pool.append(0, seqs, ctx, [1] * 8, nd, nd)
        q = rng.standard_normal((8, N_Q, HD), dtype=np.float32)
        out = run_attn(pool, seqs, ctx, q)
        worst = 0.0
        for i, s in enumerate(seqs):
            want, _ = oracle_for(pool, s, ctx[i], q[i])
            _, rel = check_attn(out[i], want, "config3 seq %d (ctx %d)" % (i, ctx[i]))
            worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
        nd.free()
    finally:
        pool.destroy()


def read_page(pool, which, page):
    """Raw bytes of one page of layer 0's K (0) or V (1) pool."""
    import ctypes as C

    from breccia_amd.kv import check, lib

    base, _ = pool.layer_ptr(0, which)
    n = pool.page_bytes(which)
    out = np.empty(n, dtype=np.uint8)
    check(lib.bkv_memcpy_d2h(out.ctypes.data, C.c_void_p(base.value + page * n), n, None))
    check(lib.bkv_stream_sync(None))
    return out


def step_both_ways(pool, layout, seqs, ctx, rng):
    """One decode step at positions ctx, as bkv_append + bkv_decode_attn and then -- after the new
    cells have been overwritten with other rows -- as one bkv_decode_step.  Checks that the two forms
    return the same bits and leave the same pool bytes in the pages they wrote, and that the new
    rows' bytes are the oracle encoders'.  Returns (q, outputs)."""
    n = len(seqs)
    for s, c in zip(seqs, ctx):
        pool.seq_reserve(s, c + 1)
    new_k = rng.standard_normal((n, N_KV, HD), dtype=np.float32)
    new_v = rng.standard_normal((n, N_KV, HD), dtype=np.float32)
    junk = rng.standard_normal((n, N_KV, HD), dtype=np.float32)
    q = rng.standard_normal((n, N_Q, HD), dtype=np.float32)
    kd, vd, jd = DeviceBuffer.from_numpy(new_k), DeviceBuffer.from_numpy(new_v), DeviceBuffer.from_numpy(junk)
    qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
    try:
        pool.append(0, seqs, ctx, [1] * n, kd, vd)
        two = run_attn(pool, seqs, ctx, q)
        last_pages = [int(pool.block_table(s)[c // 16]) for s, c in zip(seqs, ctx)]
        pages_two = [(read_page(pool, 0, p), read_page(pool, 1, p)) for p in last_pages]
        pool.append(0, seqs, ctx, [1] * n, jd, jd)          # other rows in the new cells
        assert not np.array_equal(read_page(pool, 0, last_pages[0]), pages_two[0][0])
        pool.decode_step(0, seqs, ctx, kd, vd, N_Q, qd, od, 1.0 / 16.0)
        device_sync()
        fused = od.download(np.float32).reshape(n, N_Q, HD)
        assert np.array_equal(fused.view(np.uint32), two.view(np.uint32))
        g = oracle.Geom(N_KV, HD, 16)
        from gpu_common import ORACLE_LAYOUT
        for i, (p, c) in enumerate(zip(last_pages, ctx)):
            pk, pv = read_page(pool, 0, p), read_page(pool, 1, p)
            assert np.array_equal(pk, pages_two[i][0]) and np.array_equal(pv, pages_two[i][1]), i
            img = oracle.PoolImage(g, 1, ORACLE_LAYOUT[layout])
            assert img.append(np.zeros(1, dtype=np.int32), c % 16, new_k[i], new_v[i]) == 0
            for which, page, image in ((0, pk, img.k), (1, pv, img.v)):
                rb = image.size // (N_KV * 16)
                for kvh in range(N_KV):
                    at = (kvh * 16 + c % 16) * rb
                    assert np.array_equal(page[at:at + rb], image[at:at + rb]), (i, which, kvh)
    finally:
        for b in (kd, vd, jd, qd, od):
            b.free()
    return q, fused


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V])
def test_config3_batch8_fused_step_all_heads(layout):
    # the benchmark's headline call at the benchmark's size (and its q8_0-V variant): every (sequence,
    # head) pair of the fused step against the oracle at the reference's bar
    rng = np.random.Generator(np.random.PCG64(20250003))
    pool, seqs, ctx = build(rng, 8, 1024, 32768, layout)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        q, out = step_both_ways(pool, layout, seqs, ctx, rng)
        worst = 0.0
        for i, s in enumerate(seqs):
            want, _ = oracle_for(pool, s, ctx[i], q[i])
            _, rel = check_attn(out[i], want, "config3 fused step, layout %d, seq %d (ctx %d)" % (layout, i, ctx[i]))
            worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
    finally:
        pool.destroy()


def test_config5_batch16_int8_fused_step():
    # configs[4] through bkv_decode_step, the call the benchmark times on this layout: bit-identical to
    # append + attend on all 16 sequences, the oracle on the shortest, the median and the longest
    rng = np.random.Generator(np.random.PCG64(20250005))
    pool, seqs, ctx = build(rng, 16, 8192, 131072, L.LAYOUT_I8H)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        q, out = step_both_ways(pool, L.LAYOUT_I8H, seqs, ctx, rng)
        order = np.argsort(ctx)
        for i in (int(order[0]), int(order[8]), int(order[-1])):
            want, v = oracle_for(pool, seqs[i], ctx[i], q[i])
            _, rel = check_attn(out[i], want, "config5 fused step seq %d (ctx %d)" % (i, ctx[i]))
            assert rel <= REF_BAR_MAX_REL, rel
            assert np.abs(out[i]).max() <= np.abs(v).max()
    finally:
        pool.destroy()


def test_config4_end_to_end_shared_prefix_f16_chunks_cow_and_swap():
    """BASELINE configs[3] as worded, on one pool: four sequences share a prefix through shared page ids
    with refcounts (2040 tokens: 127 full pages and a partial one); each appends a distinct 1024-token
    chunk of binary16 K/V (bkv_append_f16), which makes all writers but the last copy the shared
    partial page first; then a seeded 25 % of the pages in use go to pinned host memory, are
    overwritten in VRAM, and come back.  The oracle keeps its own image of the pool throughout
    (append of the widened rows, page copies): every pool byte is compared after the appends and after
    the swap, and decode attention runs against the oracle over its own image."""
    from breccia_amd.kv import Stream
    from gpu_common import Twin

    rng = np.random.Generator(np.random.PCG64(20250004))
    prefix, chunk = 2040, 1024
    with Twin(n_pages=640, max_seqs=8) as tw:
        tw.pool.set_free_order(rng.permutation(640).astype(np.int32))
        root = tw.pool.seq_create()
        tw.pool.seq_reserve(root, prefix)
        pk = rng.standard_normal((prefix, N_KV, HD)).astype(np.float16).view(np.uint16)
        pv = rng.standard_normal((prefix, N_KV, HD)).astype(np.float16).view(np.uint16)
        tw.append(0, [root], [0], [pk], [pv], f16_rows=True)
        kids = [tw.pool.seq_fork(root, prefix) for _ in range(3)]
        seqs = [root] + kids
        shared = tw.pool.block_table(root).copy()
        assert shared.size == 128 and all(tw.pool.page_refcount(int(p)) == 4 for p in shared)
        n_copies = 0
        for s in seqs:
            pairs = tw.pool.seq_reserve(s, prefix + chunk)
            n_copies += len(pairs)
            tw.pool.page_copy(pairs)
            tw.images[0].page_copy(pairs)
            ck = rng.standard_normal((chunk, N_KV, HD)).astype(np.float16).view(np.uint16)
            cv = rng.standard_normal((chunk, N_KV, HD)).astype(np.float16).view(np.uint16)
            tw.append(0, [s], [prefix], [ck], [cv], f16_rows=True)
        assert n_copies == 3
        tw.assert_pools_equal()
        tw.pool.check()
        assert all(np.array_equal(tw.pool.block_table(s)[:127], shared[:127]) for s in seqs)
        assert len({int(tw.pool.block_table(s)[127]) for s in seqs}) == 4
        # a seeded quarter of the pages in use: out, poisoned, back
        used = np.unique(np.concatenate([tw.pool.block_table(s) for s in seqs]))
        cold = rng.choice(used, size=used.size // 4, replace=False).astype(np.int32)
        slab = tw.pool.swap_page_bytes()
        host = tw.pool.host_alloc(cold.size * slab)
        st = Stream()
        tw.pool.swap_out(cold, host, st)
        tw.pool.swap_wait()
        hv = host.view().reshape(cold.size, 2, 16384)
        for i, p in enumerate(cold):
            assert np.array_equal(hv[i, 0], tw.images[0].k.reshape(-1, 16384)[p])
            assert np.array_equal(hv[i, 1], tw.images[0].v.reshape(-1, 16384)[p])
        junk = int(np.setdiff1d(np.arange(640, dtype=np.int32), used)[0])
        tw.pool.page_copy([(junk, int(p)) for p in cold], st)
        st.sync()
        assert not np.array_equal(tw.pool.read_layer(0, 0), tw.images[0].k)
        tw.pool.swap_in(cold, host, st)
        tw.pool.swap_fence(st)
        st.sync()
        tw.assert_pools_equal()
        host.free()
        q = rng.standard_normal((4, N_Q, HD)).astype(np.float32)
        pos = [prefix + chunk - 1] * 4
        out = tw.decode_attn(0, seqs, pos, q, N_Q)
        worst = 0.0
        for i, s in enumerate(seqs):
            _, rel = check_attn(out[i], tw.oracle_attend(0, s, pos[i], q[i], N_Q, threads=8), "configs[3] seq %d" % i)
            worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst


def test_config5_batch16_int8_8k_128k():
    rng = np.random.Generator(np.random.PCG64(20250005))
    pool, seqs, ctx = build(rng, 16, 8192, 131072, L.LAYOUT_I8H)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        q = rng.standard_normal((16, N_Q, HD), dtype=np.float32)
        pos = [c - 1 for c in ctx]
        out = run_attn(pool, seqs, pos, q)
        assert np.all(np.isfinite(out))
        order = np.argsort(ctx)
        for i in (int(order[0]), int(order[8]), int(order[-1])):
            want, v = oracle_for(pool, seqs[i], pos[i], q[i])
            _, rel = check_attn(out[i], want, "config5 seq %d (ctx %d)" % (i, ctx[i]))
            assert rel <= REF_BAR_MAX_REL, rel
            assert np.abs(out[i]).max() <= np.abs(v).max()
        # batched == one at a time (different split plans), all 16 sequences
        for i in range(16):
            alone = run_attn(pool, [seqs[i]], [pos[i]], q[i:i + 1])
            assert max_abs(alone[0], out[i]) < 1e-6, i
    finally:
        pool.destroy()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_config4_shape_prefill_of_1024_token_chunks_on_2048_token_prefixes(layout):
    # BASELINE configs[3] at full size through the chunk kernel: 4 sequences, a 2048-token prefix in
    # the cache, a 1024-token chunk each, one call.  Sampled tokens of every sequence against the
    # oracle (over the rows read back through bkv_gather) at the reference's bar; the chunk's last 64
    # positions of one sequence against the decode kernel; every output bounded by the largest |v|.
    rng = np.random.Generator(np.random.PCG64(20250004 + layout))
    before, t = 2048, 1024
    ctx = [before + t] * 4
    live = sum((c + 15) // 16 for c in ctx)
    pool = Pool(n_layers=1, n_pages=int(np.ceil(live / 0.6)), n_kv_head=N_KV, head_dim=HD, layout=layout,
                max_seqs=5, max_pages_per_seq=ctx[0] // 16 + 2)
    pool.set_free_order(rng.permutation(pool.desc.n_pages).astype(np.int32))
    try:
        seqs = [pool.seq_create() for _ in ctx]
        for s in seqs:
            pool.seq_reserve(s, ctx[0])
        fill_tiled(pool, seqs, ctx, rng, tile=1024)
        q = rng.standard_normal((4 * t, N_Q, HD), dtype=np.float32)
        qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
        pool.prefill_attn(0, seqs, [before] * 4, [t] * 4, N_Q, qd, od, 1.0 / 16.0)
        device_sync()
        out = od.download(np.float32).reshape(4, t, N_Q, HD)
        assert np.all(np.isfinite(out))
        worst = 0.0
        for i, s in enumerate(seqs):
            k, v = pool.gather(0, s, 0, ctx[i])
            assert np.abs(out[i]).max() <= np.abs(v).max()
            for tok in sorted({0, t - 1, t // 2, int(rng.integers(0, t)), int(rng.integers(0, t))}):
                pos = before + tok
                want = oracle.attend(q[i * t + tok], k[:pos + 1], v[:pos + 1], oracle.dense_cells(pos), pos, N_Q,
                                     N_KV, HD, threads=8)
                _, rel = check_attn(out[i, tok], want, "config4 seq %d token %d" % (i, tok))
                worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
        tail = list(range(ctx[2] - 64, ctx[2]))
        dec = run_attn(pool, [seqs[2]] * 64, tail, q[2 * t + t - 64:3 * t])
        assert max_abs(dec, out[2, -64:]) < 5e-6
        qd.free()
        od.free()
    finally:
        pool.destroy()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_pages_beyond_4_gib_into_a_pool(layout):
    # A pool of 300k pages (4.9 GB of K and as much of V on the f16 layout): one sequence lives on
    # the highest page ids, byte offsets past 2^32 into either pool.  Append, decode attention,
    # chunk attention, the fused step and a copy-on-write page copy there, against the oracle over
    # the rows read back through bkv_gather (a separate kernel with its own address arithmetic) and
    # against a twin sequence on the lowest page ids that holds the same rows.
    rng = np.random.Generator(np.random.PCG64(20250009 + layout))
    n_pages, n = 300000, 517
    pool = Pool(n_layers=1, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, layout=layout, max_seqs=6,
                max_pages_per_seq=64)
    try:
        pool.set_free_order(np.arange(n_pages - 1, -1, -1, dtype=np.int32))          # highest first
        hi = pool.seq_create()
        pool.seq_reserve(hi, n + 1)                                                  # 33 pages
        assert int(pool.block_table(hi)[:33].min()) == n_pages - 33
        pool.set_free_order(np.arange(0, n_pages - 33, dtype=np.int32))              # lowest first
        lo = pool.seq_create()
        pool.seq_reserve(lo, n + 1)
        assert int(pool.block_table(lo)[:33].max()) == 32
        k = rng.standard_normal((n + 1, N_KV, HD), dtype=np.float32)
        v = rng.standard_normal((n + 1, N_KV, HD), dtype=np.float32)
        kd, vd = DeviceBuffer.from_numpy(k), DeviceBuffer.from_numpy(v)
        pool.append(0, [hi], [0], [n], kd, vd)
        pool.append(0, [lo], [0], [n], kd, vd)
        device_sync()
        ghk, ghv = pool.gather(0, hi, 0, n)
        glk, glv = pool.gather(0, lo, 0, n)
        assert np.array_equal(ghk, glk) and np.array_equal(ghv, glv)
        assert np.abs(ghk).max() > 1.0                           # not the zeros of an untouched pool
        q = rng.standard_normal((2, N_Q, HD), dtype=np.float32)
        out = run_attn(pool, [hi, lo], [n - 1, n - 1], q[[0, 0]])
        assert np.array_equal(out[0].view(np.uint32), out[1].view(np.uint32))
        want = oracle.attend(q[0], ghk, ghv, oracle.dense_cells(n - 1), n - 1, N_Q, N_KV, HD, threads=8)
        _, rel = check_attn(out[0], want, "decode on the highest pages")
        assert rel <= REF_BAR_MAX_REL, rel
        # chunk attention over the last 100 tokens of both
        qc = rng.standard_normal((100, N_Q, HD), dtype=np.float32)
        qd, od = DeviceBuffer.from_numpy(np.concatenate([qc, qc])), DeviceBuffer(2 * qc.nbytes)
        pool.prefill_attn(0, [hi, lo], [n - 100, n - 100], [100, 100], N_Q, qd, od, 1.0 / 16.0)
        device_sync()
        oc = od.download(np.float32).reshape(2, 100, N_Q, HD)
        assert np.array_equal(oc[0].view(np.uint32), oc[1].view(np.uint32))
        for t in (0, 99):
            p = n - 100 + t
            want = oracle.attend(qc[t], ghk[:p + 1], ghv[:p + 1], oracle.dense_cells(p), p, N_Q, N_KV, HD, threads=8)
            _, rel = check_attn(oc[0, t], want, "chunk on the highest pages, token %d" % t)
            assert rel <= REF_BAR_MAX_REL, rel
        qd.free()
        od.free()
        # the fused step appends row n on both and attends
        k1 = DeviceBuffer.from_numpy(np.ascontiguousarray(k[n:n + 1].repeat(2, 0)))
        v1 = DeviceBuffer.from_numpy(np.ascontiguousarray(v[n:n + 1].repeat(2, 0)))
        qd, od = DeviceBuffer.from_numpy(np.ascontiguousarray(q[[1, 1]])), DeviceBuffer(q.nbytes)
        pool.decode_step(0, [hi, lo], [n, n], k1, v1, N_Q, qd, od, 1.0 / 16.0)
        device_sync()
        os_ = od.download(np.float32).reshape(2, N_Q, HD)
        assert np.array_equal(os_[0].view(np.uint32), os_[1].view(np.uint32))
        ghk, ghv = pool.gather(0, hi, 0, n + 1)
        want = oracle.attend(q[1], ghk, ghv, oracle.dense_cells(n), n, N_Q, N_KV, HD, threads=8)
        _, rel = check_attn(os_[0], want, "step on the highest pages")
        assert rel <= REF_BAR_MAX_REL, rel
        for b in (k1, v1, qd, od):
            b.free()
        # selection lists (every block, ascending) through the list kernel
        n_ids = (n + 1 + 3) // 4
        ids = np.tile(np.arange(n_ids, dtype=np.uint32), (2, 1))
        idd, cd = DeviceBuffer.from_numpy(ids), DeviceBuffer.from_numpy(np.full(2, n_ids, dtype=np.uint32))
        qd, od = DeviceBuffer.from_numpy(np.ascontiguousarray(q[[1, 1]])), DeviceBuffer(q.nbytes)
        pool.decode_attn_select(0, [hi, lo], [n, n], N_Q, qd, od, 1.0 / 16.0, idd, n_ids, cd, n_ids)
        device_sync()
        osel = od.download(np.float32).reshape(2, N_Q, HD)
        assert np.array_equal(osel[0].view(np.uint32), osel[1].view(np.uint32))
        _, rel = check_attn(osel[0], want, "selection lists on the highest pages")
        assert rel <= REF_BAR_MAX_REL, rel
        for b in (idd, cd, qd, od):
            b.free()
        # the complete pages of `hi` go to host memory and come back onto other high pages
        pool.set_free_order(np.arange(n_pages - 34, 32, -1, dtype=np.int32))
        host = pool.host_alloc(32 * pool.swap_page_bytes())
        pool.seq_evict(hi, 0, 32, host)
        pool.swap_wait()
        pool.seq_restore(hi, 0, 32, host)
        device_sync()
        pool.swap_wait()
        assert int(pool.block_table(hi)[:32].min()) >= n_pages - 100
        grk, grv = pool.gather(0, hi, 0, n + 1)
        assert np.array_equal(grk, ghk) and np.array_equal(grv, ghv)
        host.free()
        # a fork of `hi` that writes copies the shared, partly filled last page to another high page
        child = pool.seq_fork(hi, n + 1)
        pairs = pool.seq_reserve(child, n + 2)
        assert len(pairs) == 1 and pairs[0][0] == n_pages - 33 and pairs[0][1] >= n_pages - 100
        pool.page_copy(pairs)
        device_sync()
        gck, gcv = pool.gather(0, child, 0, n + 1)
        assert np.array_equal(gck, ghk) and np.array_equal(gcv, ghv)
        kd.free()
        vd.free()
        pool.check()
    finally:
        pool.destroy()


def test_one_sequence_of_400k_tokens():
    # far past BASELINE's longest context (128k): 25000 pages in one block-table row, hundreds of
    # split-K ranges per head for the merge; decode attention and the fused step against the oracle
    rng = np.random.Generator(np.random.PCG64(20250010))
    ctx = [400003]
    pool, seqs, _ = build(rng, 1, ctx[0], ctx[0], L.LAYOUT_F16, occupancy=0.9)
    try:
        fill_tiled(pool, seqs, ctx, rng)
        q = rng.standard_normal((1, N_Q, HD), dtype=np.float32)
        out = run_attn(pool, seqs, [ctx[0] - 1], q)
        want, v = oracle_for(pool, seqs[0], ctx[0] - 1, q[0])
        _, rel = check_attn(out[0], want, "400k tokens")
        assert rel <= REF_BAR_MAX_REL, rel
        assert np.abs(out[0]).max() <= np.abs(v).max()
        # a T = 3 decode (three positions of the same sequence) equals three single calls
        pos = [ctx[0] - 1, ctx[0] // 2, 12345]
        q3 = rng.standard_normal((3, N_Q, HD), dtype=np.float32)
        together = run_attn(pool, seqs * 3, pos, q3)
        for i in range(3):
            alone = run_attn(pool, seqs, [pos[i]], q3[i:i + 1])
            assert max_abs(alone[0], together[i]) < 1e-6, i
    finally:
        pool.destroy()


def test_config2_single_stream_ctx4096_on_a_64k_page_pool_12_layers():
    """BASELINE configs[1]: one sequence of 4096 tokens on pages drawn by a seeded shuffle from a
    65 536-page pool (1 GiB K + 1 GiB V per layer), 12 layers with independent seeded K/V/q; the step
    of every layer is append-then-attend at position 4096 (the reference's per-layer loop,
    crates/breccia-engine/src/graph.rs:5899-5966 -> crates/breccia-kernels/src/qsa/mod.rs:1617-1641).
    The step runs in both forms -- one bkv_decode_step on the sequence, bkv_append + bkv_decode_attn on
    a fork that shares its 256 full pages -- and per layer the rows the sequence holds are compared bit
    for bit with the oracle's image (through bkv_gather, and the new row's raw pool bytes at the page
    the shuffle gave it), the outputs with the oracle at the reference's 1e-5 bar and with each other
    bit for bit."""
    n_layers, n_pages, ctx = 12, 65536, 4096
    rng = np.random.Generator(np.random.PCG64(20250002))
    pool = Pool(n_layers=n_layers, n_pages=n_pages, n_kv_head=N_KV, head_dim=HD, max_seqs=4,
                max_pages_per_seq=ctx // 16 + 2)
    bufs = []
    try:
        pool.set_free_order(rng.permutation(n_pages).astype(np.int32))
        seq = pool.seq_create()
        pool.seq_reserve(seq, ctx)
        g = oracle.Geom(N_KV, HD, 16)
        compact = np.arange(ctx // 16 + 1, dtype=np.int32)      # the oracle keeps the pages side by side
        images = []
        for layer in range(n_layers):
            k = rng.standard_normal((ctx, N_KV, HD), dtype=np.float32)
            v = rng.standard_normal((ctx, N_KV, HD), dtype=np.float32)
            kd, vd = DeviceBuffer.from_numpy(k), DeviceBuffer.from_numpy(v)
            pool.append(layer, [seq], [0], [ctx], kd, vd)
            device_sync()
            kd.free()
            vd.free()
            img = oracle.PoolImage(g, compact.size)
            assert img.append(compact, 0, k, v) == 0
            images.append(img)
        twin = pool.seq_fork(seq, ctx)                          # 256 full pages shared: no copy to make
        assert pool.seq_reserve(seq, ctx + 1) == [] and pool.seq_reserve(twin, ctx + 1) == []
        tab, tab2 = pool.block_table(seq), pool.block_table(twin)
        assert np.array_equal(tab[:256], tab2[:256]) and tab[256] != tab2[256]
        assert len(set(tab.tolist())) == 257 and tab.max() > n_pages // 2      # scattered over the pool
        worst = 0.0
        for layer in range(n_layers):
            k1 = rng.standard_normal((1, N_KV, HD), dtype=np.float32)
            v1 = rng.standard_normal((1, N_KV, HD), dtype=np.float32)
            q = rng.standard_normal((1, N_Q, HD), dtype=np.float32)
            kd, vd, qd = DeviceBuffer.from_numpy(k1), DeviceBuffer.from_numpy(v1), DeviceBuffer.from_numpy(q)
            o1, o2 = DeviceBuffer(q.nbytes), DeviceBuffer(q.nbytes)
            bufs = [kd, vd, qd, o1, o2]
            pool.decode_step(layer, [seq], [ctx], kd, vd, N_Q, qd, o1, 1.0 / 16.0)
            pool.append(layer, [twin], [ctx], [1], kd, vd)
            pool.decode_attn(layer, [twin], [ctx], N_Q, qd, o2, 1.0 / 16.0)
            device_sync()
            fused = o1.download(np.float32).reshape(N_Q, HD)
            twocall = o2.download(np.float32).reshape(N_Q, HD)
            img = images[layer]
            assert img.append(compact, ctx, k1, v1) == 0
            wk, wv = img.gather(compact, 0, ctx + 1)
            for s, t in ((seq, tab), (twin, tab2)):
                gk, gv = pool.gather(layer, s, 0, ctx + 1)
                assert np.array_equal(gk.view(np.uint32), wk.view(np.uint32)), (layer, s)
                assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32)), (layer, s)
                # the new row's bytes where the block table says they are: page t[256], cell 0, both kv heads
                for which, image in ((0, img.k), (1, img.v)):
                    base, _ = pool.layer_ptr(layer, which)
                    for kvh in range(N_KV):
                        row = np.empty(HD * 2, dtype=np.uint8)
                        off = ((int(t[256]) * N_KV + kvh) * 16) * HD * 2
                        from breccia_amd.kv import check, lib
                        import ctypes as C
                        check(lib.bkv_memcpy_d2h(row.ctypes.data, C.c_void_p(base.value + off), row.nbytes, None))
                        check(lib.bkv_stream_sync(None))
                        woff = ((256 * N_KV + kvh) * 16) * HD * 2
                        assert np.array_equal(row, image[woff:woff + HD * 2]), (layer, s, which, kvh)
            want = oracle.attend(q[0], wk, wv, oracle.dense_cells(ctx), ctx, N_Q, N_KV, HD, threads=8)
            _, rel = check_attn(fused, want, "configs[1] layer %d fused step" % layer)
            _, rel2 = check_attn(twocall, want, "configs[1] layer %d two calls" % layer)
            worst = max(worst, rel, rel2)
            assert np.array_equal(fused.view(np.uint32), twocall.view(np.uint32)), layer
            for b in bufs:
                b.free()
            bufs = []
        assert worst <= REF_BAR_MAX_REL, worst
        pool.check()
    finally:
        for b in bufs:
            b.free()
        pool.destroy()
