"""GPU parity of block selection (indexer score + top-k) against the CPU oracle: the emitted
id lists must be identical, element for element (crates/breccia-kernels/src/qsa/cpu.rs:93-152;
recipes of tests/qsa_topk.rs and tests/attn_conformance.rs:897-1004)."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, Pool, device_sync
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from test_gpu_attn import fill
from test_oracle_select import DEAD, lcg_scores

pytestmark = pytest.mark.gpu


def gpu_topk(pool, scores, pos, topk, max_ids, dense=False, id_stride=None):
    """scores: float32 [n, n_blocks] -> list of uint32 id arrays."""
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    n, nb = scores.shape
    id_stride = id_stride or max_ids
    sd = DeviceBuffer.from_numpy(scores if scores.size else np.zeros(4, np.float32))
    idd = DeviceBuffer.from_numpy(np.full((n, id_stride), 0xFFFFFFFF, dtype=np.uint32))
    cd = DeviceBuffer.from_numpy(np.full(n, 0xFFFFFFFF, dtype=np.uint32))
    try:
        pool.topk_blocks(pos, sd, nb, topk, idd, id_stride, cd, max_ids, dense=dense)
        device_sync()
        ids = idd.download(np.uint32, n * id_stride).reshape(n, id_stride)
        cnt = cd.download(np.uint32, n)
        after = sd.download(np.float32, max(scores.size, 4))[:scores.size].reshape(n, nb)
        assert np.array_equal(after.view(np.uint32), scores.view(np.uint32))    # scores untouched
        for i in range(n):
            assert np.all(ids[i, cnt[i]:] == 0xFFFFFFFF)                          # nothing past count
        return [ids[i, :cnt[i]].copy() for i in range(n)]
    finally:
        for b in (sd, idd, cd):
            b.free()


def oracle_topk_f32(scores_row, topk, own, max_ids):
    # the shaders' dead rule: a score <= -1e29 is never selected (shaders/qsa_topk.comp)
    s = np.asarray(scores_row, dtype=np.float64).copy()
    s[~(s > -1.0e29)] = -np.inf
    ids = oracle.topk_blocks(s, min(topk, max_ids), None)
    if own not in ids and ids.size < max_ids:
        ids = np.append(ids, np.uint32(own))
    return ids


@pytest.mark.parametrize("cells", [65536, 65521])
def test_reference_topk_recipes_are_exact(cells):
    # crates/breccia-kernels/tests/qsa_topk.rs:87-122, 16384 / 16380 blocks, 512 kept
    n, k, max_ids = cells // 4, 512, 513
    distinct = lcg_scores(n)
    tied = np.zeros(n, dtype=np.float32)
    tied[:100] = 1.0
    dead = distinct.copy()
    dead[::3] = DEAD
    rows = [distinct, tied, dead, np.full(n, 0.5, dtype=np.float32), distinct]
    pos = [0, 0, 0, 0, 4 * (n - 3)]
    with Pool(n_pages=4, max_seqs=2) as pool:
        got = gpu_topk(pool, np.stack(rows), pos, k, max_ids)
    for i, (row, p) in enumerate(zip(rows, pos)):
        want = oracle_topk_f32(row, k, p // 4, max_ids)
        assert np.array_equal(got[i], want), "recipe %d: first difference at %s" % (
            i, np.nonzero(got[i][:min(got[i].size, want.size)] != want[:min(got[i].size, want.size)])[0][:3])


def test_topk_edge_cases():
    rng = np.random.Generator(np.random.PCG64(700))
    with Pool(n_pages=4, max_seqs=2) as pool:
        # reference known answers (qsa/cpu.rs:517-536) on f32 scores
        s = np.array([[1.0, 3.0, 3.0, 2.0]], dtype=np.float32)
        assert list(gpu_topk(pool, s, [4 * 9], 2, 8)[0]) == [1, 2, 9]
        assert list(gpu_topk(pool, s, [4 * 9], 4, 8)[0]) == [1, 2, 3, 0, 9]
        assert list(gpu_topk(pool, s, [4 * 3 + 1], 3, 8)[0]) == [1, 2, 3]
        s = np.array([[-np.inf, -np.inf, 1.0]], dtype=np.float32)
        assert list(gpu_topk(pool, s, [8], 3, 8)[0]) == [2]
        # fewer live than k; NaN and the shaders' -1e30 marker are dead; -0 ties with +0 by index
        s = np.array([[0.25, -1e30, 0.75, np.nan, 0.5, -0.0, 0.0, -3.0]], dtype=np.float32)
        assert list(gpu_topk(pool, s, [4], 512, 16)[0]) == [2, 4, 0, 5, 6, 7, 1]
        # no room for the own block; max_ids caps the list
        assert list(gpu_topk(pool, s, [4 * 40], 3, 3)[0]) == [2, 4, 0]
        assert list(gpu_topk(pool, s, [4 * 40], 512, 2, id_stride=5)[0]) == [2, 4]
        # zero blocks: only the own block
        assert list(gpu_topk(pool, np.zeros((1, 0), np.float32), [21], 512, 4)[0]) == [5]
        # several lists of one call, random scores with many exact ties, k not a power of two
        sc = rng.integers(0, 50, size=(7, 3000)).astype(np.float32) / 8 - 2
        pos = [int(p) for p in rng.integers(0, 4 * 3000, size=7)]
        got = gpu_topk(pool, sc, pos, 300, 301)
        for i in range(7):
            assert np.array_equal(got[i], oracle_topk_f32(sc[i], 300, pos[i] // 4, 301)), i
        # negative scores order correctly (key transform of negative floats)
        sc = -np.abs(rng.standard_normal((2, 1000))).astype(np.float32) * 1e3
        got = gpu_topk(pool, sc, [0, 3999], 2048, 2049)
        for i, p in enumerate([0, 3999]):
            assert np.array_equal(got[i], oracle_topk_f32(sc[i], 2048, p // 4, 2049)), i
        # lists longer than the work-group (more than one candidate per thread in the sort): 1500 and
        # 2048 kept, scores with ties
        sc = (rng.integers(0, 4000, size=(2, 6000)).astype(np.float32) - 1000) / 16
        for keep in (1500, 2048):
            got = gpu_topk(pool, sc, [4 * 6000, 4 * 6000], keep, keep + 1)
            for i in range(2):
                assert np.array_equal(got[i], oracle_topk_f32(sc[i], keep, 6000, keep + 1)), (keep, i)
        # dense: every visible block ascending, own appended when it lies beyond n_blocks
        d = gpu_topk(pool, np.zeros((3, 515), np.float32), [2061, 100, 2059], 512, 600, dense=True)
        assert list(d[0]) == list(range(515)) + [515]
        assert list(d[1]) == list(range(26))
        assert list(d[2]) == list(range(515))


def test_topk_orders_through_buckets_and_through_the_sorting_network():
    # The kernel selects and orders through one histogram over equal slices of the score range when the
    # slices at and above the threshold are thinly filled; otherwise by a radix select on the key bits,
    # then slices of the selected keys' range or, when those are crowded too, a sorting network.  Smooth
    # scores (thin slices), one outlier far above the rest (every other key in the lowest slice), 200
    # equal scores above the threshold, a threshold inside a run of equal scores, denormal scores, an
    # outlier far below (a stretched range, but a tight one among the selected), infinities, a selection
    # that spans both signs, and lists whose keys are re-read from memory on every pass.
    rng = np.random.Generator(np.random.PCG64(701))
    n, k = 5003, 512
    smooth = rng.standard_normal(n).astype(np.float32)
    outlier = smooth.copy()
    outlier[1234] = 1e30
    both_signs = smooth.copy()
    many_equal = smooth.copy()
    many_equal[rng.permutation(n)[:200]] = 2.5
    run_at_threshold = smooth.copy()
    order = np.argsort(-smooth, kind="stable")
    run_at_threshold[order[480:560]] = smooth[order[480]]          # 80 equal scores around rank 512
    tiny = (rng.standard_normal(n) * 1e-42).astype(np.float32)     # denormal scores of both signs
    low_outlier = smooth.copy()
    low_outlier[77] = -1e25                                        # live, and far below: stretches the range
    with_inf = smooth.copy()
    with_inf[[5, 4000]] = np.inf                                   # never selected (qsa/cpu.rs:139-143)
    with_inf[6] = 3.0e38                                           # live: the range overflows f32, not f64
    rows = [smooth, outlier, many_equal, run_at_threshold, tiny, low_outlier, with_inf]
    pos = [int(p) for p in rng.integers(0, 4 * n, size=len(rows))]
    with Pool(n_pages=4, max_seqs=2) as pool:
        got = gpu_topk(pool, np.stack(rows), pos, k, k + 1)
        for i, row in enumerate(rows):
            assert np.array_equal(got[i], oracle_topk_f32(row, k, pos[i] // 4, k + 1)), i
        got = gpu_topk(pool, both_signs[None, :], [0], 2048, 2049)  # below and above zero
        assert np.array_equal(got[0], oracle_topk_f32(both_signs, 2048, 0, 2049))
        big = rng.standard_normal((2, 30011)).astype(np.float32)    # keys re-read from memory per pass
        big[1, ::7] = 0.125
        got = gpu_topk(pool, big, [5, 4 * 30011], 2000, 2001)
        for i, p in enumerate([5, 4 * 30011]):
            assert np.array_equal(got[i], oracle_topk_f32(big[i], 2000, p // 4, 2001)), i


def gpu_select(pool, pos, idx_q, pooled_list, topk, max_ids):
    n = len(pos)
    qd = DeviceBuffer.from_numpy(np.ascontiguousarray(idx_q, dtype=np.float32))
    pds = [DeviceBuffer.from_numpy(np.ascontiguousarray(p, dtype=np.float32)) for p in pooled_list]
    idd = DeviceBuffer.from_numpy(np.full((n, max_ids), 0xFFFFFFFF, dtype=np.uint32))
    cd = DeviceBuffer.from_numpy(np.zeros(n, dtype=np.uint32))
    pool.select_blocks(pos, qd, pds, [p.shape[0] for p in pooled_list], idx_q.shape[1], idx_q.shape[2], topk,
                       idd, max_ids, cd, max_ids)
    device_sync()
    ids = idd.download(np.uint32, n * max_ids).reshape(n, max_ids)
    cnt = cd.download(np.uint32, n)
    for b in [qd, cd] + pds:
        b.free()
    return idd, ids, cnt


def test_reference_selection_and_attention_at_2062_cells():
    # crates/breccia-kernels/tests/attn_conformance.rs:897-1004: 515 whole blocks + 2 tail cells,
    # indexer queries 0xE1, pooled keys 0xE2, K/V 0xE3/0xE4 appended in 256-cell chunks, q 0xE5,
    # gate in place from q_full 0xE6, 24 heads; selection list, then attention over exactly it
    cells, n_blocks, pos = 2062, 515, 2061
    idx_q = oracle.normalish(0xE1, 4 * 128).reshape(1, 4, 128)
    pooled = oracle.normalish(0xE2, (n_blocks + 1) * 128).reshape(n_blocks + 1, 128)
    k_all = oracle.normalish(0xE3, cells * 512).reshape(cells, 2, 256)
    v_all = oracle.normalish(0xE4, cells * 512).reshape(cells, 2, 256)
    q = oracle.normalish(0xE5, 24 * 256).reshape(1, 24, 256)
    q_full = oracle.normalish(0xE6, 24 * 512)
    with Twin(n_pages=129, max_seqs=2) as tw:
        s = tw.pool.seq_create_identity(129)
        tw.pool.seq_reserve(s, cells)
        for at in range(0, cells, 256):
            tw.append(0, [s], [at], [k_all[at:at + 256]], [v_all[at:at + 256]])
        idd, ids, cnt = gpu_select(tw.pool, [pos], idx_q, [pooled[:n_blocks]], 512, 513)
        want_ids = oracle.topk_blocks(oracle.indexer_score(idx_q[0], pooled, n_blocks, pos), 512, pos // 4)
        assert cnt[0] == want_ids.size == 513
        assert np.array_equal(ids[0, :cnt[0]], want_ids)      # order and set, tail block last
        # attention over exactly those cells, lists left on the device
        cd = DeviceBuffer.from_numpy(cnt)
        qd = DeviceBuffer.from_numpy(q)
        gd = DeviceBuffer.from_numpy(q_full)
        od = DeviceBuffer(q.nbytes)
        tw.pool.decode_attn_select(0, [s], [pos], 24, qd, od, 0.0625, idd, 513, cd, 513, gate_dev=gd.at(256 * 4),
                                   gate_seq_stride=24 * 512, gate_head_stride=512)
        out = od.download(np.float32, q.size).reshape(24, 256)
        kk, vv = tw.images[0].gather(tw.pool.block_table(s), 0, cells)
        gate = np.ascontiguousarray(q_full.reshape(24, 512)[:, 256:])
        want = oracle.attend(q[0], kk, vv, oracle.cells_of(want_ids), pos, 24, 2, 256, gate=gate, threads=4)
        _, rel = check_attn(out, want, "2062-cell sparse")
        assert rel <= REF_BAR_MAX_REL, rel
        for b in (idd, cd, qd, gd, od):
            b.free()


def test_score_and_select_batched_lists_are_exact():
    # several sequences of different lengths in one call; scores are dense in value (many near
    # ties), which is where an f32 score would reorder the list
    rng = np.random.Generator(np.random.PCG64(710))
    n_blocks = [8192, 515, 3, 0, 12001, 64]
    pos = [4 * 8192 + 2, 2061, 9, 1, 48007, 130]       # entry 5: only blocks 0..32 are visible
    idx_q = rng.standard_normal((6, 4, 128)).astype(np.float32)
    pooled = [rng.standard_normal((nb, 128)).astype(np.float32) * 0.05 for nb in n_blocks]
    with Pool(n_pages=4, max_seqs=2) as pool:
        idd, ids, cnt = gpu_select(pool, pos, idx_q, pooled, 512, 513)
        idd.free()
    for i in range(6):
        sc = oracle.indexer_score(idx_q[i], pooled[i], n_blocks[i], pos[i]) if n_blocks[i] else np.zeros(0)
        want = oracle.topk_blocks(sc, 512, pos[i] // 4)
        assert cnt[i] == want.size, (i, cnt[i], want.size)
        assert np.array_equal(ids[i, :cnt[i]], want), i
    assert cnt[5] == 33 and 32 in ids[5, :33]


@pytest.mark.parametrize("heads,dim", [(2, 96), (8, 64), (1, 2), (3, 128)])
def test_score_and_select_other_indexer_shapes(heads, dim):
    # widths other than 128 take the score kernel's element-by-element path; the lists stay exact
    rng = np.random.Generator(np.random.PCG64(711 + heads * 131 + dim))
    n_blocks = [3000, 65, 700]
    pos = [4 * 3000 + 1, 259, 2000]
    idx_q = rng.standard_normal((3, heads, dim)).astype(np.float32)
    pooled = [rng.standard_normal((nb, dim)).astype(np.float32) * 0.05 for nb in n_blocks]
    with Pool(n_pages=4, max_seqs=2) as pool:
        idd, ids, cnt = gpu_select(pool, pos, idx_q, pooled, 128, 129)
        idd.free()
    for i in range(3):
        sc = oracle.indexer_score(idx_q[i], pooled[i], n_blocks[i], pos[i], idx_n_head=heads, idx_dim=dim)
        want = oracle.topk_blocks(sc, 128, pos[i] // 4)
        assert cnt[i] == want.size, (i, cnt[i], want.size)
        assert np.array_equal(ids[i, :cnt[i]], want), i


def test_select_errors_come_before_any_launch():
    with Pool(n_pages=4, max_seqs=2) as pool:
        z = DeviceBuffer(1 << 16)
        for kw, status in [(dict(topk_blocks=0), L.ERR_INVALID), (dict(topk_blocks=4096), L.ERR_INVALID),
                           (dict(max_ids=0), L.ERR_INVALID), (dict(id_stride=4), L.ERR_INVALID),
                           (dict(ids_dev=None), L.ERR_INVALID), (dict(pos=[-1]), L.ERR_RANGE)]:
            a = dict(pos=[5], scores_dev=z, n_blocks=16, topk_blocks=8, ids_dev=z, id_stride=16, counts_dev=z,
                     max_ids=9)
            a.update(kw)
            with pytest.raises(BkvError) as ei:
                pool.topk_blocks(**a)
            assert ei.value.status == status, kw
        with pytest.raises(BkvError) as ei:
            pool.select_blocks([5], z, [z], [16], 9, 128, 8, z, 16, z, 9)       # too many indexer heads
        assert ei.value.status == L.ERR_INVALID
        with pytest.raises(BkvError) as ei:
            pool.select_blocks([5], z, [None], [16], 4, 128, 8, z, 16, z, 9)    # NULL pooled keys
        assert ei.value.status == L.ERR_INVALID
        z.free()


def test_pooled_indexer_keys_in_ragged_chunks_are_bit_exact():
    # Qsa::idx_pool + Qsa::idx_tail over a sequence fed in chunks of every residue mod 4: the pooled
    # rows must equal the oracle's pool_keys over the whole sequence, and feed the same selection
    from breccia_amd.kv import rope_table
    rng = np.random.Generator(np.random.PCG64(720))
    cells, max_blocks = 1203, 320
    raw = (rng.standard_normal((cells, 128)) * rng.uniform(0.1, 4.0, size=(cells, 1))).astype(np.float32)
    gamma = (1.0 + 0.2 * rng.standard_normal(128)).astype(np.float32)
    table = rope_table(1e7, 64, 2048)
    want = oracle.pool_keys(raw, gamma, table)
    with Pool(n_pages=4, max_seqs=2) as pool:
        pooled = DeviceBuffer.from_numpy(np.full((max_blocks, 128), np.nan, dtype=np.float32))
        tail = DeviceBuffer.from_numpy(np.full((3, 128), np.nan, dtype=np.float32))
        gd, td = DeviceBuffer.from_numpy(gamma), DeviceBuffer.from_numpy(table)
        at = 0
        chunks = [1, 1, 1, 1, 2, 3, 5, 7, 4, 8, 1, 2, 300, 6, 1, 1, 3, 512]
        while at < cells:
            n = min(chunks.pop(0) if chunks else 97, cells - at)
            kd = DeviceBuffer.from_numpy(raw[at:at + n])
            pool.idx_pool(pooled, max_blocks, tail, kd, at, n, gd, 1e-6, td, 64, 2048)
            device_sync()
            kd.free()
            at += n
        got = pooled.download(np.float32, max_blocks * 128).reshape(max_blocks, 128)
        assert np.array_equal(got[:cells // 4].view(np.uint32), want.view(np.uint32))
        assert np.all(np.isnan(got[cells // 4:]))                       # nothing past the completed blocks
        t = tail.download(np.float32, 3 * 128).reshape(3, 128)
        assert np.array_equal(t[:3], raw[1200:1203])                    # the incomplete block's rows
        # selection over the device-pooled keys == selection over the oracle's
        idx_q = rng.standard_normal((1, 4, 128)).astype(np.float32)
        qd = DeviceBuffer.from_numpy(idx_q)
        idd = DeviceBuffer.from_numpy(np.zeros((1, 129), dtype=np.uint32))
        cd = DeviceBuffer.from_numpy(np.zeros(1, dtype=np.uint32))
        pool.select_blocks([cells - 1], qd, [pooled], [cells // 4], 4, 128, 128, idd, 129, cd, 129)
        device_sync()
        n = int(cd.download(np.uint32, 1)[0])
        ids = idd.download(np.uint32, 129)[:n]
        ref = oracle.topk_blocks(oracle.indexer_score(idx_q[0], want, cells // 4, cells - 1), 128, (cells - 1) // 4)
        assert np.array_equal(ids, ref)
        with pytest.raises(BkvError) as ei:
            pool.idx_pool(pooled, 10, tail, gd, 36, 8, gd, 1e-6, td, 64, 2048)     # would write block 10
        assert ei.value.status == L.ERR_RANGE
        for b in (pooled, tail, gd, td, qd, idd, cd):
            b.free()
