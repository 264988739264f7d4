"""GPU parity of paged decode attention against the f64 CPU oracle
(crates/breccia-kernels/src/qsa/cpu.rs:197-246).  Tolerance: north_star's 2e-3 max-abs /
1e-3 relative (relative = the reference's max|g-w|/max(|w|,1)); the reference's own
1e-5 bar is asserted too wherever the f32 kernel is expected to meet it."""
import json
import os

import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import DeviceBuffer, device_sync
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from helpers import max_abs

pytestmark = pytest.mark.gpu


GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def fill(tw, seq, n, rng, layer=0, chunk=256, gen=None):
    """Grow `seq` to n cells of N(0,1) K/V (or gen(count) values) in append chunks."""
    pos = tw.pool.seq_len(seq)
    while pos < n:
        t = min(chunk, n - pos)
        tw.pool.seq_reserve(seq, pos + t)
        if gen is None:
            k = rng.standard_normal((t, 2, 256)).astype(np.float32)
            v = rng.standard_normal((t, 2, 256)).astype(np.float32)
        else:
            k, v = gen(t)
        tw.append(layer, [seq], [pos], [k], [v])
        pos += t


def test_config1_four_sequences_append_then_decode():
    """BASELINE config 1: 16 q / 2 kv heads, d 256, page 16, 512-page pool, sequences of
    37/512/1000/2048 tokens on a seeded permutation of the pool; step = append one token per
    sequence, then decode attention with scale 1/16."""
    rng = np.random.Generator(np.random.PCG64(20240001))
    lens = [37, 512, 1000, 2048]
    with Twin(n_pages=512, max_seqs=8) as tw:
        # seeded permutation of the pool: interleave reservations so that physical pages of
        # the four sequences are shuffled among each other
        seqs = [tw.pool.seq_create() for _ in lens]
        order = rng.permutation(sum((n + 15) // 16 for n in lens))
        owner = np.concatenate([[i] * ((n + 15) // 16) for i, n in enumerate(lens)])[order]
        for i in owner:
            s = seqs[i]
            tw.pool.seq_reserve(s, min(lens[i], tw.pool.seq_len(s) + 16))
        for s, n in zip(seqs, lens):
            assert tw.pool.seq_len(s) == n
            tw.pool.seq_truncate(s, 0)
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng)
        # the step
        for s in seqs:
            tw.pool.seq_reserve(s, tw.pool.seq_len(s) + 1)
        k1 = [rng.standard_normal((1, 2, 256)).astype(np.float32) for _ in seqs]
        v1 = [rng.standard_normal((1, 2, 256)).astype(np.float32) for _ in seqs]
        tw.append(0, seqs, lens, k1, v1)
        tw.assert_pools_equal()
        q = rng.standard_normal((4, 16, 256)).astype(np.float32)
        out = tw.decode_attn(0, seqs, lens, q, 16, scale=1.0 / 16.0)
        worst = 0.0
        for i, (s, n) in enumerate(zip(seqs, lens)):
            want = tw.oracle_attend(0, s, n, q[i], 16)
            a, r = check_attn(out[i], want, "config1 seq %d" % i)
            worst = max(worst, r)
        assert worst <= REF_BAR_MAX_REL, worst


def test_reference_recipe_2062_cells_24_heads_gated():
    # crates/breccia-kernels/tests/attn_conformance.rs:897-1164 with the dense selection:
    # normalish inputs, 256-cell append chunks (last chunk 14), 24 q heads, gate read in place
    # from q_full at h*512 + 256 + d
    r = GOLD["dense_2062_recipe"]
    cells = r["cells"]
    k_all = oracle.normalish(int(r["seeds"]["k"], 16), cells * 512).reshape(cells, 2, 256)
    v_all = oracle.normalish(int(r["seeds"]["v"], 16), cells * 512).reshape(cells, 2, 256)
    q = oracle.normalish(int(r["seeds"]["q"], 16), 24 * 256).reshape(1, 24, 256)
    q_full = oracle.normalish(int(r["seeds"]["q_full"], 16), 24 * 512)
    with Twin(n_pages=(cells + 15) // 16, max_seqs=2) as tw:
        s = tw.pool.seq_create_identity((cells + 15) // 16)
        tw.pool.seq_reserve(s, cells)
        for at in range(0, cells, r["append_chunk"]):
            n = min(r["append_chunk"], cells - at)
            tw.append(0, [s], [at], [k_all[at:at + n]], [v_all[at:at + n]])
        tw.assert_pools_equal()
        gate_view = q_full.reshape(24, 512)[:, 256:]
        out = tw.decode_attn(0, [s], [r["pos"]], q, 24, gate=q_full[256:],
                             gate_strides=(24 * 512, 512))
        want = tw.oracle_attend(0, s, r["pos"], q[0], 24, gate=np.ascontiguousarray(gate_view))
        a, rel = check_attn(out[0], want, "2062-cell recipe")
        assert rel <= r["bar_max_rel"], rel


def test_reference_recipe_64_cells_is_dense_when_all_blocks_are_listed():
    # crates/breccia-kernels/tests/attn_conformance.rs:1355-1452 inputs (seeds 0xF1..0xF4); the
    # sparse id list [0,5,9,15] is outside the dense path, so this checks the full 64 cells
    r = GOLD["q8_recipe"]
    k_all = oracle.normalish(0xF1, 64 * 512).reshape(64, 2, 256)
    v_all = oracle.normalish(0xF2, 64 * 512).reshape(64, 2, 256)
    q = oracle.normalish(0xF3, 24 * 256).reshape(1, 24, 256)
    q_full = oracle.normalish(0xF4, 24 * 512)
    with Twin(n_pages=4, max_seqs=2) as tw:
        s = tw.pool.seq_create_identity(4)
        tw.pool.seq_reserve(s, 64)
        tw.append(0, [s], [0], [k_all], [v_all])
        out = tw.decode_attn(0, [s], [63], q, 24, gate=q_full[256:], gate_strides=(24 * 512, 512))
        gate = np.ascontiguousarray(q_full.reshape(24, 512)[:, 256:])
        want = tw.oracle_attend(0, s, 63, q[0], 24, gate=gate)
        _, rel = check_attn(out[0], want, "64-cell recipe")
        assert rel <= r["bar_max_rel"]


def test_closed_forms_on_the_gpu():
    rng = np.random.Generator(np.random.PCG64(17))
    with Twin(n_pages=64, max_seqs=8) as tw:
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        gate = rng.standard_normal((1, 16, 256)).astype(np.float32)
        # one live cell: out = v * sigmoid(gate)
        a = tw.pool.seq_create()
        fill(tw, a, 1, rng)
        out = tw.decode_attn(0, [a], [0], q, 16, gate=gate)
        _, v = tw.images[0].gather(tw.pool.block_table(a), 0, 1)
        want = np.repeat(v[0].astype(np.float64), 8, axis=0) / (1.0 + np.exp(-gate[0].astype(np.float64)))
        assert max_abs(out[0], want) < 1e-6
        # identical K rows: mean of V
        b = tw.pool.seq_create()
        krow = rng.standard_normal((1, 2, 256)).astype(np.float32)
        fill(tw, b, 100, rng, gen=lambda t: (np.repeat(krow, t, axis=0),
                                              rng.standard_normal((t, 2, 256)).astype(np.float32)))
        out = tw.decode_attn(0, [b], [99], q, 16)
        _, v = tw.images[0].gather(tw.pool.block_table(b), 0, 100)
        want = np.repeat(v.astype(np.float64).mean(axis=0), 8, axis=0)
        assert max_abs(out[0], want) < 1e-6
        # gate = 0: exactly half of the ungated output
        half = tw.decode_attn(0, [b], [99], q, 16, gate=np.zeros_like(gate))
        assert np.array_equal(half, out * np.float32(0.5))
        # a position inside the sequence: later cells contribute nothing
        c = tw.pool.seq_create()
        fill(tw, c, 77, rng)
        out40 = tw.decode_attn(0, [c], [40], q, 16)
        check_attn(out40[0], tw.oracle_attend(0, c, 40, q[0], 16), "pos inside the sequence")
        # scale is honoured (a dropped or doubled scale changes the result)
        out_s = tw.decode_attn(0, [c], [76], q, 16, scale=0.03)
        kk, vv = tw.images[0].gather(tw.pool.block_table(c), 0, 77)
        want = oracle.attend(q[0] * np.float32(0.03 * 16.0), kk, vv, np.arange(77), 76, 16, 2, 256)
        assert max_abs(out_s[0], want) < 1e-5


def score_spread_case(loud_rows, layout=0):
    # The running maximum of a head must be the maximum over all 16 rows of a page, whichever
    # lanes hold them: cells at page rows [lo, hi) carry scores some 40 (base-2: 58) above the
    # rest, so a maximum taken over part of the rows only would overflow the probabilities.
    rng = np.random.Generator(np.random.PCG64(640 + loud_rows[0]))
    n = 16 * 23 + 7
    with Twin(n_pages=40, max_seqs=2, layout=layout) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, n)
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        k = rng.standard_normal((n, 2, 256)).astype(np.float32)
        v = rng.standard_normal((n, 2, 256)).astype(np.float32)
        rows = np.arange(n) % 16
        loud = (rows >= loud_rows[0]) & (rows < loud_rows[1])
        # loud cells: k = a multiple of the mean query of the kv head's group, so that every head
        # of the group scores them high
        for h in range(2):
            qm = q[0, 8 * h:8 * h + 8].mean(axis=0)
            k[loud, h] = (40.0 * 16.0 / float(qm @ qm)) * qm + 0.1 * k[loud, h]
        tw.append(0, [s], [0], [k], [v])
        out = tw.decode_attn(0, [s], [n - 1], q, 16)
        want = tw.oracle_attend(0, s, n - 1, q[0], 16)
        check_attn(out[0], want, "loud rows %d..%d" % loud_rows)


@pytest.mark.parametrize("loud_rows", [(0, 4), (4, 16), (9, 10), (12, 16)])
def test_score_spread_across_the_rows_of_a_page(loud_rows):
    score_spread_case(loud_rows)


def test_unwritten_and_poisoned_cells_are_never_read_as_values():
    # the reference's BRECCIA_FAULT_POISON_QSA check (crates/breccia-kernels/src/qsa/mod.rs:
    # 509-523): with the pool NaN-filled, nothing past `pos` may reach the output
    rng = np.random.Generator(np.random.PCG64(19))
    with Twin(n_pages=32, max_seqs=4) as tw:
        tw.pool.fill(0xFF)
        device_sync()
        for img in tw.images:
            img.k[:] = 0xFF
            img.v[:] = 0xFF
        s = tw.pool.seq_create()
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        for n in (1, 15, 16, 17, 37, 250):
            fill(tw, s, n, rng, chunk=64)
            out = tw.decode_attn(0, [s], [n - 1], q, 16)
            assert np.all(np.isfinite(out)), n
            check_attn(out[0], tw.oracle_attend(0, s, n - 1, q[0], 16), "poisoned pool, len %d" % n)


def test_physical_page_placement_does_not_change_a_bit():
    rng = np.random.Generator(np.random.PCG64(23))
    k = rng.standard_normal((900, 2, 256)).astype(np.float32)
    v = rng.standard_normal((900, 2, 256)).astype(np.float32)
    q = rng.standard_normal((1, 16, 256)).astype(np.float32)
    outs = []
    for shift in (0, 5, 40):
        with Twin(n_pages=128, max_seqs=4) as tw:
            pad = tw.pool.seq_create()
            if shift:
                tw.pool.seq_reserve(pad, 16 * shift)
            s = tw.pool.seq_create()
            tw.pool.seq_reserve(s, 900)
            tw.append(0, [s], [0], [k], [v])
            outs.append(tw.decode_attn(0, [s], [899], q, 16))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_several_positions_of_one_sequence_in_one_call():
    # T > 1 decode: the reference's attend takes T tokens at pos0..pos0+T
    # (crates/breccia-kernels/src/qsa/mod.rs:1382-1462)
    rng = np.random.Generator(np.random.PCG64(29))
    with Twin(n_pages=64, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, 600, rng)
        pos = [590, 591, 592, 599, 15, 16, 0]
        q = rng.standard_normal((len(pos), 16, 256)).astype(np.float32)
        out = tw.decode_attn(0, [s] * len(pos), pos, q, 16)
        for i, p in enumerate(pos):
            _, rel = check_attn(out[i], tw.oracle_attend(0, s, p, q[i], 16), "pos %d" % p)
            assert rel <= REF_BAR_MAX_REL


def test_split_count_does_not_matter_beyond_rounding():
    """The same sequence alone and inside a batch gets different split-K plans; both must sit
    within 1e-6 of each other and of the oracle's bar."""
    rng = np.random.Generator(np.random.PCG64(37))
    with Twin(n_pages=1400, max_seqs=8) as tw:
        seqs = [tw.pool.seq_create() for _ in range(4)]
        lens = [5000, 333, 8111, 4096]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=1024)
        q = rng.standard_normal((4, 16, 256)).astype(np.float32)
        pos = [n - 1 for n in lens]
        batch = tw.decode_attn(0, seqs, pos, q, 16)
        for i in range(4):
            alone = tw.decode_attn(0, [seqs[i]], [pos[i]], q[i:i + 1], 16)
            assert max_abs(alone[0], batch[i]) < 1e-6
            _, rel = check_attn(batch[i], tw.oracle_attend(0, seqs[i], pos[i], q[i], 16), "seq %d" % i)
            assert rel <= REF_BAR_MAX_REL


@pytest.mark.parametrize("n_q", [2, 4, 8, 24, 32])
def test_other_head_groupings(n_q):
    rng = np.random.Generator(np.random.PCG64(41 + n_q))
    with Twin(n_pages=64, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, 300, rng)
        q = rng.standard_normal((1, n_q, 256)).astype(np.float32)
        gate = rng.standard_normal((1, n_q, 256)).astype(np.float32)
        out = tw.decode_attn(0, [s], [299], q, n_q, gate=gate)
        _, rel = check_attn(out[0], tw.oracle_attend(0, s, 299, q[0], n_q, gate=gate[0]), "n_q %d" % n_q)
        assert rel <= REF_BAR_MAX_REL


def test_layers_are_independent():
    rng = np.random.Generator(np.random.PCG64(43))
    with Twin(n_layers=3, n_pages=32, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 200)
        for layer in range(3):
            k = rng.standard_normal((200, 2, 256)).astype(np.float32)
            v = rng.standard_normal((200, 2, 256)).astype(np.float32)
            tw.append(layer, [s], [0], [k], [v])
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        for layer in range(3):
            tw.assert_pools_equal(layer)
            out = tw.decode_attn(layer, [s], [199], q, 16)
            check_attn(out[0], tw.oracle_attend(layer, s, 199, q[0], 16), "layer %d" % layer)


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_kv,n_q", [(1, 16), (3, 12), (8, 32), (4, 4), (5, 60)])
def test_other_head_counts(layout, n_kv, n_q):
    # kv head counts other than the model's 2, groups of 1, 4, 12 and 16 q heads per kv head: decode
    # attention, the fused step and the chunk kernel against the oracle
    rng = np.random.Generator(np.random.PCG64(150 + 17 * n_kv + n_q + layout))
    with Twin(n_pages=96, n_kv=n_kv, layout=layout, max_seqs=4) as tw:
        tw.pool.set_free_order(rng.permutation(96).astype(np.int32))
        lens = [333, 70]
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            tw.pool.seq_reserve(s, n + 1)
            k = rng.standard_normal((n, n_kv, 256)).astype(np.float32)
            v = rng.standard_normal((n, n_kv, 256)).astype(np.float32)
            tw.append(0, [s], [0], [k], [v])
        q = rng.standard_normal((2, n_q, 256)).astype(np.float32)
        pos = [n - 1 for n in lens]
        out = tw.decode_attn(0, seqs, pos, q, n_q)
        for i in range(2):
            _, rel = check_attn(out[i], tw.oracle_attend(0, seqs[i], pos[i], q[i], n_q), "decode %d" % i)
            assert rel <= REF_BAR_MAX_REL, rel
        # the chunk kernel over the last 40 tokens of the first sequence
        qc = rng.standard_normal((40, n_q, 256)).astype(np.float32)
        qd, od = DeviceBuffer.from_numpy(qc), DeviceBuffer(qc.nbytes)
        tw.pool.prefill_attn(0, [seqs[0]], [lens[0] - 40], [40], n_q, qd, od, 1.0 / 16.0)
        device_sync()
        oc = od.download(np.float32).reshape(40, n_q, 256)
        qd.free()
        od.free()
        for t in (0, 17, 39):
            _, rel = check_attn(oc[t], tw.oracle_attend(0, seqs[0], lens[0] - 40 + t, qc[t], n_q), "chunk %d" % t)
            assert rel <= REF_BAR_MAX_REL, rel
        # the fused step (one more token per sequence): pool bytes as an append would leave them,
        # outputs against the oracle
        k1 = rng.standard_normal((2, n_kv, 256)).astype(np.float32)
        v1 = rng.standard_normal((2, n_kv, 256)).astype(np.float32)
        kd, vd = DeviceBuffer.from_numpy(k1), DeviceBuffer.from_numpy(v1)
        qd, od = DeviceBuffer.from_numpy(q), DeviceBuffer(q.nbytes)
        tw.pool.decode_step(0, seqs, lens, kd, vd, n_q, qd, od, 1.0 / 16.0)
        device_sync()
        os_ = od.download(np.float32).reshape(2, n_q, 256)
        for b in (kd, vd, qd, od):
            b.free()
        for i, s in enumerate(seqs):
            assert tw.images[0].append(tw.pool.block_table(s), lens[i], k1[i:i + 1], v1[i:i + 1],
                                       capacity_cells=tw.pool.seq_capacity(s)) == 0
        tw.assert_pools_equal()
        for i in range(2):
            _, rel = check_attn(os_[i], tw.oracle_attend(0, seqs[i], lens[i], q[i], n_q), "step %d" % i)
            assert rel <= REF_BAR_MAX_REL, rel


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_batches_that_need_more_than_one_generation_of_work_groups(layout):
    # 64 entries x 9 kv heads = 576 units even with one range per entry: more than the 512 work-groups
    # that are resident at once.  Planned as one range per entry (the host used to spin on this shape),
    # run in two generations, and still the oracle's answer.
    n_kv, n_q = 9, 18
    rng = np.random.Generator(np.random.PCG64(9100 + layout))
    with Twin(n_pages=64 * 6, n_kv=n_kv, layout=layout, max_seqs=64, max_pages_per_seq=8) as tw:
        tw.pool.set_free_order(rng.permutation(64 * 6).astype(np.int32))
        lens = [int(x) for x in rng.integers(1, 90, size=64)]
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            tw.pool.seq_reserve(s, n)
        ks = [rng.standard_normal((n, n_kv, 256)).astype(np.float32) for n in lens]
        vs = [rng.standard_normal((n, n_kv, 256)).astype(np.float32) for n in lens]
        tw.append(0, seqs, [0] * 64, ks, vs)
        q = rng.standard_normal((64, n_q, 256)).astype(np.float32)
        pos = [n - 1 for n in lens]
        out = tw.decode_attn(0, seqs, pos, q, n_q)
        for i in range(64):
            _, rel = check_attn(out[i], tw.oracle_attend(0, seqs[i], pos[i], q[i], n_q), "entry %d" % i)
            assert rel <= REF_BAR_MAX_REL, (i, rel)


def test_foreign_f16_subnormals_attend_with_their_ieee_value_and_gather_as_zero():
    """The append path never stores an f16 code with exponent field 0; bytes written behind its
    back (bkv_pool_layer_ptr, a restored foreign dump) may hold them.  The documented split: the
    attention kernels multiply such codes as the IEEE subnormals they are, bkv_gather reads them
    as zero (the reference's load rule, crates/breccia-kernels/shaders/f16_storage.glsl:58-69).
    kv head 0 gets subnormal V rows (outputs of the size of a subnormal, not zero), kv head 1
    subnormal K rows under a large q (logits that move the weights by about a percent)."""
    rng = np.random.Generator(np.random.PCG64(6060))
    n, n_q = 45, 16
    with Twin(n_pages=8) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, n, rng)
        table = tw.pool.block_table(s)
        kb = tw.pool.read_layer(0, 0).view(np.uint16).copy()
        vb = tw.pool.read_layer(0, 1).view(np.uint16).copy()
        k_img, v_img = tw.images[0].gather(table, 0, n)
        k_ieee, v_ieee = k_img.copy().reshape(n, 2, 256), v_img.copy().reshape(n, 2, 256)
        for cell in range(n):
            for buf, kvh, img in ((vb, 0, v_ieee), (kb, 1, k_ieee)):
                row = (int(table[cell // 16]) * 2 + kvh) * 16 + cell % 16
                c = (rng.integers(1, 0x400, size=256) | (rng.integers(0, 2, size=256) << 15)).astype(np.uint16)
                buf[row * 256:(row + 1) * 256] = c
                img[cell, kvh] = c.view(np.float16).astype(np.float32)
        tw.pool.write_layer(0, 0, kb)
        tw.pool.write_layer(0, 1, vb)
        q = rng.standard_normal((1, n_q, 256)).astype(np.float32)
        q[0, 8:] *= 300.0
        got = tw.decode_attn(0, [s], [n - 1], q, n_q)[0]
        want = oracle.attend(q[0], k_ieee, v_ieee, oracle.dense_cells(n - 1), n - 1, n_q, 2, 256)
        # heads of kv head 0: weighted means of subnormals
        top = float(np.max(np.abs(want[:8])))
        assert 1e-6 < top < 1e-4, top
        assert max_abs(got[:8], want[:8]) <= 1e-3 * top
        # heads of kv head 1: the reference bar, and visibly not the uniform weights of an all-zero K
        _, rel = check_attn(got[8:], want[8:], "subnormal K rows as IEEE values")
        assert rel <= REF_BAR_MAX_REL, rel
        uniform = v_ieee[:, 1, :].astype(np.float64).mean(axis=0)
        assert max_abs(got[8:], np.broadcast_to(uniform, (8, 256))) > 1e-4
        gk, gv = tw.pool.gather(0, s, 0, n)
        assert not np.any(gv[:, 0]) and not np.any(gk[:, 1])
        assert np.array_equal(gk[:, 0], k_img.reshape(n, 2, 256)[:, 0])


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_repeated_launches_of_one_batch_return_identical_bits(layout):
    """The cut into page ranges and the order in which the partial results are combined are a
    function of the batch alone: 100 launches of one batch (ranges of 1 to 40 pages per
    work-group, 1 to 33 of them per head) return identical bits, and those are the oracle's answer."""
    rng = np.random.Generator(np.random.PCG64(8800 + layout))
    lens = [5000, 16, 2100, 333, 90, 1]
    n_q = 16
    with Twin(n_pages=520, layout=layout, max_seqs=8, max_pages_per_seq=320) as tw:
        tw.pool.set_free_order(rng.permutation(520).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=1024)
        pos = [n - 1 for n in lens]
        q = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
        gate = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
        qd, gd = DeviceBuffer.from_numpy(q), DeviceBuffer.from_numpy(gate)
        od = DeviceBuffer(q.nbytes)
        first = None
        for it in range(100):
            tw.pool.decode_attn(0, seqs, pos, n_q, qd, od, 1.0 / 16.0, gate_dev=gd, gate_seq_stride=n_q * 256,
                                gate_head_stride=256)
            out = od.download(np.float32).reshape(len(lens), n_q, 256)
            if first is None:
                first = out.copy()
                for i in range(len(lens)):
                    _, rel = check_attn(out[i], tw.oracle_attend(0, seqs[i], pos[i], q[i], n_q, gate=gate[i]), "entry %d" % i)
                    assert rel <= REF_BAR_MAX_REL, (i, rel)
            else:
                assert np.array_equal(first.view(np.uint32), out.view(np.uint32)), "launch %d differs" % it
        for b in (qd, gd, od):
            b.free()
