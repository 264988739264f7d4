"""GPU parity of decode attention over selection lists (device-resident block ids / counts,
4 cells per block) against the CPU oracle's attend over cells_of(ids) -- the reference's
sparse form (crates/breccia-kernels/src/qsa/cpu.rs:197-257, qsa/mod.rs:1382-1462).
Tolerances as in test_gpu_attn.py."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from helpers import max_abs
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu


def select_attn(tw, layer, seqs, pos, q, n_head, id_lists, max_ids=None, id_stride=None, gate=None,
                gate_strides=None, counts=None, pad=0xDEADBEEF):
    """q: [n, n_head, 256]; id_lists: one list of block ids per entry.  The unused tail of every
    ids row is filled with `pad` (never read as a live block)."""
    n = len(seqs)
    max_ids = max_ids or max(1, max(len(l) for l in id_lists))
    id_stride = id_stride or max_ids
    ids = np.full((n, id_stride), pad, dtype=np.uint32)
    for i, l in enumerate(id_lists):
        ids[i, :len(l)] = np.asarray(l, dtype=np.uint32)
    cnt = np.asarray([len(l) for l in id_lists] if counts is None else counts, dtype=np.uint32)
    q = np.ascontiguousarray(q, dtype=np.float32)
    qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
    idd, cd = DeviceBuffer.from_numpy(ids), DeviceBuffer.from_numpy(cnt)
    gd, ss, hs = None, 0, 0
    if gate is not None:
        gd = DeviceBuffer.from_numpy(np.ascontiguousarray(gate, dtype=np.float32))
        ss, hs = gate_strides if gate_strides else (n_head * 256, 256)
    try:
        tw.pool.decode_attn_select(layer, seqs, pos, n_head, qd, od, 1.0 / 16.0, idd, id_stride, cd, max_ids,
                                   gate_dev=gd, gate_seq_stride=ss, gate_head_stride=hs)
        return od.download(np.float32, q.size).reshape(n, n_head, 256)
    finally:
        for b in (qd, od, idd, cd, gd):
            if b is not None:
                b.free()


def oracle_select(tw, layer, seq, pos, q, n_head, ids, gate=None):
    table = tw.pool.block_table(seq)
    k, v = tw.images[layer].gather(table, 0, pos + 1)
    # a block that starts past `pos` has no live cell; it is dropped here so that ids whose
    # cell index would not fit 32 bits never reach the oracle's u32 arithmetic
    cells = oracle.cells_of(np.asarray([b for b in ids if 4 * int(b) <= pos], dtype=np.uint32))
    return oracle.attend(q, k, v, cells, pos, n_head, 2, 256, gate=gate, threads=4)


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V])
def test_reference_sparse_recipe_blocks_0_5_9_15(layout):
    # attn_conformance.rs:1355-1452: 64 cells from normalish 0xF1/0xF2, 24 heads, q 0xF3, gate
    # in place from q_full 0xF4, selection ids [0, 5, 9, 15], query at the last cell
    k_all = oracle.normalish(0xF1, 64 * 512).reshape(64, 2, 256)
    v_all = oracle.normalish(0xF2, 64 * 512).reshape(64, 2, 256)
    q = oracle.normalish(0xF3, 24 * 256).reshape(1, 24, 256)
    q_full = oracle.normalish(0xF4, 24 * 512)
    gate = np.ascontiguousarray(q_full.reshape(24, 512)[:, 256:])
    ids = [0, 5, 9, 15]
    with Twin(n_pages=4, max_seqs=2, layout=layout) as tw:
        s = tw.pool.seq_create_identity(4)
        tw.pool.seq_reserve(s, 64)
        tw.append(0, [s], [0], [k_all], [v_all])
        out = select_attn(tw, 0, [s], [63], q, 24, [ids], max_ids=513, gate=q_full[256:],
                          gate_strides=(24 * 512, 512))
        want = oracle_select(tw, 0, s, 63, q[0], 24, ids, gate=gate)
        _, rel = check_attn(out[0], want, "ids 0,5,9,15")
        assert rel <= REF_BAR_MAX_REL, rel


@pytest.mark.parametrize("n_q", [16, 24])
def test_full_list_equals_the_dense_kernel_and_the_oracle(n_q):
    # the reference's dense selection: blocks 0..=pos/4 ascending (qsa/mod.rs:1363-1376)
    rng = np.random.Generator(np.random.PCG64(600 + n_q))
    lens = [2062, 37, 1, 517]
    with Twin(n_pages=256, max_seqs=8) as tw:
        tw.pool.set_free_order(rng.permutation(256).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=512)
        pos = [n - 1 for n in lens]
        q = rng.standard_normal((4, n_q, 256)).astype(np.float32)
        lists = [list(range(p // 4 + 1)) for p in pos]
        out = select_attn(tw, 0, seqs, pos, q, n_q, lists, max_ids=516)
        dense = tw.decode_attn(0, seqs, pos, q, n_q, scale=1.0 / 16.0)
        assert max_abs(out, dense) < 2e-6
        for i, s in enumerate(seqs):
            want = oracle_select(tw, 0, s, pos[i], q[i], n_q, lists[i])
            _, rel = check_attn(out[i], want, "full list, seq %d" % i)
            assert rel <= REF_BAR_MAX_REL, rel


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_sparse_lists_ragged_batch_with_duplicates_and_future_blocks(layout):
    rng = np.random.Generator(np.random.PCG64(610 + layout))
    lens = [4099, 1000, 70, 9, 2500]
    with Twin(n_pages=600, max_seqs=8, layout=layout) as tw:
        tw.pool.set_free_order(rng.permutation(600).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=1024)
        # T = 2 decode on the first sequence: two entries, different positions and lists
        ent_seq = [seqs[0], seqs[0], seqs[1], seqs[2], seqs[3], seqs[4]]
        pos = [4098, 4000, 999, 69, 8, 2499]
        lists = []
        for p in pos:
            nb = p // 4 + 1
            k = min(nb, int(rng.integers(1, 140)))
            l = list(rng.choice(nb, size=k, replace=False))
            if nb - 1 not in l:
                l.append(nb - 1)                      # own block last, as the top-k leaves it
            lists.append(l)
        lists[1] = lists[1] + lists[1][:3]            # blocks listed twice count twice
        lists[2] = [nb_future for nb_future in (260, 10**6, 2**31)] + lists[2]   # past pos: dead
        lists[3] = [17]                               # one block, the query's own, 2 live cells
        lists[4] = [2, 0, 1]                          # 9 cells: block 2 has one live cell
        q = rng.standard_normal((6, 16, 256)).astype(np.float32)
        gate = rng.standard_normal((6, 16, 256)).astype(np.float32)
        out = select_attn(tw, 0, ent_seq, pos, q, 16, lists, max_ids=160, id_stride=200, gate=gate)
        for i in range(6):
            want = oracle_select(tw, 0, ent_seq[i], pos[i], q[i], 16, lists[i], gate=gate[i])
            _, rel = check_attn(out[i], want, "layout %d entry %d" % (layout, i))
            assert rel <= REF_BAR_MAX_REL, (i, rel)


def test_empty_and_capped_lists_and_poisoned_cells():
    rng = np.random.Generator(np.random.PCG64(620))
    with Twin(n_pages=64, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, 300, rng, chunk=300)
        # cells past the end of the sequence hold NaN patterns: they must never reach the output
        kp = tw.pool.read_layer(0, 0).view(np.uint16).copy()
        vp = tw.pool.read_layer(0, 1).view(np.uint16).copy()
        t = tw.pool.block_table(s)
        for c in range(300, 304):
            for h in range(2):
                row = ((int(t[c // 16]) * 2 + h) * 16 + c % 16) * 256
                kp[row:row + 256] = 0x7E00
                vp[row:row + 256] = 0xFE01
        tw.pool.write_layer(0, 0, kp.view(np.uint8))
        tw.pool.write_layer(0, 1, vp.view(np.uint8))
        q = rng.standard_normal((3, 16, 256)).astype(np.float32)
        lists = [[], [74, 3, 40], list(range(75))]
        # entry 0: empty list -> zeros; entry 1: own block 74 holds cells 296..299 live + the NaN
        # neighbours are in block 75 (not listed); entry 2: counts says 75 but max_ids caps at 60
        out = select_attn(tw, 0, [s, s, s], [299, 297, 299], q, 16, lists, max_ids=60, id_stride=80,
                          counts=[0, 3, 75])
        assert np.all(out[0] == 0.0)
        assert np.all(np.isfinite(out))
        want1 = oracle_select(tw, 0, s, 297, q[1], 16, lists[1])
        check_attn(out[1], want1, "own block with cells past pos")
        want2 = oracle_select(tw, 0, s, 299, q[2], 16, lists[2][:60])
        check_attn(out[2], want2, "list capped at max_ids")
        # a list that also names block 75 (cells 300..303, all past pos and all NaN): the block is
        # dead as a whole, so the result is that of its live neighbour alone
        out3 = select_attn(tw, 0, [s], [299], q[:1], 16, [[75, 74]], max_ids=8)
        want3 = oracle_select(tw, 0, s, 299, q[0], 16, [74])
        check_attn(out3[0], want3, "future block listed")


def test_select_errors_come_before_any_launch():
    with Twin(n_pages=8, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 40)
        z = DeviceBuffer(1 << 16)

        def call(**kw):
            a = dict(layer=0, seqs=[s], pos=[39], n_q_head=16, q_dev=z, out_dev=z, scale=0.0625, ids_dev=z,
                     id_stride=16, counts_dev=z, max_ids=16)
            a.update(kw)
            tw.pool.decode_attn_select(**a)

        for kw, status in [(dict(max_ids=0), L.ERR_INVALID), (dict(id_stride=8), L.ERR_INVALID),
                           (dict(ids_dev=None), L.ERR_INVALID), (dict(counts_dev=None), L.ERR_INVALID),
                           (dict(pos=[48]), L.ERR_RANGE), (dict(n_q_head=15), L.ERR_INVALID),
                           (dict(layer=1), L.ERR_RANGE)]:
            with pytest.raises(BkvError) as ei:
                call(**kw)
            assert ei.value.status == status, kw
        z.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_kv,n_q", [(1, 16), (3, 12), (8, 32), (5, 60)])
def test_selection_lists_with_other_head_counts(layout, n_kv, n_q):
    rng = np.random.Generator(np.random.PCG64(950 + 13 * n_kv + n_q + layout))
    with Twin(n_pages=64, n_kv=n_kv, layout=layout, max_seqs=4) as tw:
        tw.pool.set_free_order(rng.permutation(64).astype(np.int32))
        n = 413
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, n)
        k = rng.standard_normal((n, n_kv, 256)).astype(np.float32)
        v = rng.standard_normal((n, n_kv, 256)).astype(np.float32)
        tw.append(0, [s], [0], [k], [v])
        pos = [n - 1, 200]
        lists = [sorted(rng.choice((p + 1 + 3) // 4, size=min(37, (p + 4) // 4), replace=False).tolist()) for p in pos]
        q = rng.standard_normal((2, n_q, 256)).astype(np.float32)
        out = select_attn(tw, 0, [s, s], pos, q, n_q, lists)
        table = tw.pool.block_table(s)
        for i in range(2):
            kk, vv = tw.images[0].gather(table, 0, pos[i] + 1)
            cells = oracle.cells_of(np.asarray(lists[i], dtype=np.uint32))
            want = oracle.attend(q[i], kk, vv, cells, pos[i], n_q, n_kv, 256, threads=4)
            _, rel = check_attn(out[i], want, "list %d" % i)
            assert rel <= REF_BAR_MAX_REL, rel
