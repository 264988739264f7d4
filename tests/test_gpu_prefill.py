"""GPU parity of the MFMA prefill attention (causal attention of whole chunks over the paged
cache) against the CPU oracle, token by token, and against the decode kernel.  Tolerances as in
test_gpu_attn.py, including the reference's own 1e-5 bar."""
import numpy as np
import pytest

from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from helpers import max_abs
from test_gpu_attn import fill

pytestmark = pytest.mark.gpu


def prefill(tw, layer, seqs, pos0, q_list, n_head, gate_list=None):
    """q_list[i]: [T_i, n_head, 256] -> list of outputs of the same shapes (one call)."""
    n_tok = [q.shape[0] for q in q_list]
    qcat = np.ascontiguousarray(np.concatenate([q.reshape(-1) for q in q_list] + [np.zeros(4, np.float32)]),
                                dtype=np.float32)
    qd, od = DeviceBuffer.from_numpy(qcat), DeviceBuffer(qcat.nbytes)
    gd = None
    if gate_list is not None:
        gd = DeviceBuffer.from_numpy(np.concatenate([g.reshape(-1) for g in gate_list] + [np.zeros(4, np.float32)]))
    try:
        tw.pool.prefill_attn(layer, seqs, pos0, n_tok, n_head, qd, od, 1.0 / 16.0, gate_dev=gd,
                             gate_tok_stride=n_head * 256 if gd else 0, gate_head_stride=256 if gd else 0)
        flat = od.download(np.float32, qcat.size)
    finally:
        for b in (qd, od, gd):
            if b is not None:
                b.free()
    outs, at = [], 0
    for t in n_tok:
        outs.append(flat[at:at + t * n_head * 256].reshape(t, n_head, 256))
        at += t * n_head * 256
    return outs


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_q", [16, 24])
def test_chunks_match_the_oracle_token_by_token(n_q, layout):
    rng = np.random.Generator(np.random.PCG64(1000 + n_q))
    # (cells before the chunk, chunk length): from scratch, on a prefix, single token, page edges
    cases = [(0, 100), (517, 300), (64, 1), (15, 17), (2048, 130)]
    with Twin(n_pages=400, max_seqs=8, layout=layout) as tw:
        tw.pool.set_free_order(rng.permutation(400).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in cases]
        for s, (before, t) in zip(seqs, cases):
            fill(tw, s, before + t, rng, chunk=1024)            # the chunk's own K/V are in the cache
        qs = [rng.standard_normal((t, n_q, 256)).astype(np.float32) for _, t in cases]
        gates = [rng.standard_normal((t, n_q, 256)).astype(np.float32) for _, t in cases]
        outs = prefill(tw, 0, seqs, [b for b, _ in cases], qs, n_q, gates)
        worst = 0.0
        for s, (before, t), q, g, out in zip(seqs, cases, qs, gates, outs):
            picks = sorted(set([0, t - 1, t // 2] + [int(x) for x in rng.integers(0, t, size=6)] +
                               [i for i in range(t) if (before + i) % 16 in (0, 15)][:6]))
            for i in picks:
                want = tw.oracle_attend(0, s, before + i, q[i], n_q, gate=g[i])
                _, rel = check_attn(out[i], want, "chunk at %d, token %d" % (before, i))
                worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
        # the decode kernel on the same positions agrees to f32 noise
        s, (before, t) = seqs[1], cases[1]
        pos = list(range(before + t - 40, before + t))
        dec = tw.decode_attn(0, [s] * 40, pos, qs[1][-40:], n_q, scale=1.0 / 16.0, gate=gates[1][-40:])
        assert max_abs(dec, outs[1][-40:]) < 5e-6


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("v_mag", [1.2e-2, 1.0, 900.0])
def test_quantised_chunks_across_the_scale_range(v_mag, layout):
    # quantised V with block scales from near 2^-14 up to 7, blocks of one row and rows of one page
    # on different scales (the quietest rows of the int8 layout have scales below 2^-14, which pool
    # and oracle alike read as zero): the result stays at the reference's bar relative to the
    # largest output
    rng = np.random.Generator(np.random.PCG64(1020))
    with Twin(n_pages=80, max_seqs=2, layout=layout) as tw:
        s = tw.pool.seq_create()
        n = 1203
        tw.pool.seq_reserve(s, n)
        k = rng.standard_normal((n, 2, 256)).astype(np.float32)
        v = (rng.standard_normal((n, 2, 256)) * v_mag).astype(np.float32)
        v[:, :, 64:96] *= 0.37
        v[5::7] *= 0.11
        v[40:60] *= 1.0e-3      # a page and a half of very quiet rows
        tw.append(0, [s], [0], [k], [v])
        q = rng.standard_normal((203, 16, 256)).astype(np.float32)
        out = prefill(tw, 0, [s], [1000], [q], 16)[0]
        for i in (0, 57, 101, 202):
            want = tw.oracle_attend(0, s, 1000 + i, q[i], 16)
            rel = max_abs(out[i], want) / float(np.max(np.abs(want)))
            assert rel <= REF_BAR_MAX_REL, (i, rel)
        # a short context made of the quiet rows and their neighbours only
        q2 = rng.standard_normal((30, 16, 256)).astype(np.float32)
        out2 = prefill(tw, 0, [s], [35], [q2], 16)[0]
        for i in (0, 10, 29):
            want = tw.oracle_attend(0, s, 35 + i, q2[i], 16)
            rel = max_abs(out2[i], want) / float(np.max(np.abs(want)))
            assert rel <= REF_BAR_MAX_REL, (i, rel)


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_quantised_prefill_ignores_poisoned_cells(layout):
    # every unwritten byte of the pools is 0xFF (NaN scales, NaN K): chunks that end inside a page
    rng = np.random.Generator(np.random.PCG64(1021))
    with Twin(n_pages=32, max_seqs=2, layout=layout) as tw:
        tw.pool.fill(0xFF)
        for img in tw.images:
            img.k[:] = 0xFF
            img.v[:] = 0xFF
        s = tw.pool.seq_create()
        for n, t in ((1, 1), (17, 16), (40, 23), (200, 130), (203, 3)):
            fill(tw, s, n, rng, chunk=64)
            q = rng.standard_normal((t, 16, 256)).astype(np.float32)
            out = prefill(tw, 0, [s], [n - t], [q], 16)[0]
            assert np.all(np.isfinite(out))
            for i in sorted({0, t // 2, t - 1}):
                check_attn(out[i], tw.oracle_attend(0, s, n - t + i, q[i], 16), "len %d token %d" % (n, i))


def test_prefill_ignores_poisoned_cells_and_future_tokens():
    rng = np.random.Generator(np.random.PCG64(1010))
    with Twin(n_pages=64, max_seqs=4) as tw:
        s = tw.pool.seq_create()
        fill(tw, s, 200, rng, chunk=200)
        # attend a chunk that ends before the cache does (tokens 100..149): cells 150..199 are real
        # but in the future; cells 200..207 of the last page hold NaN patterns
        kp = tw.pool.read_layer(0, 0).view(np.uint16).copy()
        vp = tw.pool.read_layer(0, 1).view(np.uint16).copy()
        t = tw.pool.block_table(s)
        for c in range(200, 208):
            for h in range(2):
                row = ((int(t[c // 16]) * 2 + h) * 16 + c % 16) * 256
                kp[row:row + 256] = 0x7E00
                vp[row:row + 256] = 0xFE01
        tw.pool.write_layer(0, 0, kp.view(np.uint8))
        tw.pool.write_layer(0, 1, vp.view(np.uint8))
        q = rng.standard_normal((50, 16, 256)).astype(np.float32)
        out = prefill(tw, 0, [s], [100], [q], 16)[0]
        assert np.all(np.isfinite(out))
        for i in (0, 11, 27, 49):
            check_attn(out[i], tw.oracle_attend(0, s, 100 + i, q[i], 16), "token %d" % i)
        # a chunk that ends exactly at the poisoned page's last live cell
        q2 = rng.standard_normal((9, 16, 256)).astype(np.float32)
        out2 = prefill(tw, 0, [s], [191], [q2], 16)[0]
        assert np.all(np.isfinite(out2))
        check_attn(out2[8], tw.oracle_attend(0, s, 199, q2[8], 16), "last cell")


def test_prefill_errors_come_before_any_launch():
    with Twin(n_pages=8, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 40)
        z = DeviceBuffer(1 << 20)
        for kw, status in [(dict(pos0=[30], n_tokens=[19]), L.ERR_RANGE), (dict(n_q_head=15), L.ERR_INVALID),
                           (dict(q_dev=None), L.ERR_INVALID), (dict(layer=2), L.ERR_RANGE),
                           (dict(seqs=[1]), L.ERR_RANGE)]:
            a = dict(layer=0, seqs=[s], pos0=[0], n_tokens=[40], n_q_head=16, q_dev=z, out_dev=z, scale=0.0625)
            a.update(kw)
            with pytest.raises(BkvError) as ei:
                tw.pool.prefill_attn(**a)
            assert ei.value.status == status, kw
        z.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_the_largest_batch_of_chunks_in_one_call(layout):
    # 64 chunks (the limit of one call) over 8 sequences, lengths 0..70 tokens, several chunks of
    # one sequence in the same call: every token agrees with the decode kernel at its position, and
    # a sample with the oracle; 65 chunks are refused
    rng = np.random.Generator(np.random.PCG64(1030 + layout))
    with Twin(n_pages=300, max_seqs=10, layout=layout) as tw:
        tw.pool.set_free_order(rng.permutation(300).astype(np.int32))
        lens = [int(x) for x in rng.integers(200, 520, size=8)]
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=256)
        ent_seq, pos0, n_tok = [], [], []
        for i in range(64):
            j = i % 8
            t = [0, 1, 15, 16, 17, 33, 64, 70][(i // 8 + j) % 8]
            p0 = int(rng.integers(0, lens[j] - t + 1))
            ent_seq.append(seqs[j])
            pos0.append(p0)
            n_tok.append(t)
        qs = [rng.standard_normal((t, 16, 256)).astype(np.float32) for t in n_tok]
        outs = prefill(tw, 0, ent_seq, pos0, qs, 16)
        checked = 0
        for i in range(64):
            t = n_tok[i]
            if t == 0:
                assert outs[i].shape[0] == 0
                continue
            for at in range(0, t, 64):
                m = min(64, t - at)
                dec = tw.decode_attn(0, [ent_seq[i]] * m, list(range(pos0[i] + at, pos0[i] + at + m)),
                                     qs[i][at:at + m], 16, scale=1.0 / 16.0)
                assert max_abs(dec, outs[i][at:at + m]) < 5e-6, (i, at)
            if i % 9 == 0:
                tok = t - 1
                want = tw.oracle_attend(0, ent_seq[i], pos0[i] + tok, qs[i][tok], 16)
                _, rel = check_attn(outs[i][tok], want, "chunk %d" % i)
                assert rel <= REF_BAR_MAX_REL, (i, rel)
                checked += 1
        assert checked >= 5
        z = DeviceBuffer(1 << 16)
        with pytest.raises(BkvError) as ei:
            tw.pool.prefill_attn(0, ent_seq + [seqs[0]], pos0 + [0], [1] * 65, 16, z, z, 0.0625)
        assert ei.value.status == L.ERR_INVALID
        z.free()


def test_work_group_width_does_not_change_a_bit():
    # On f16 pools a call whose chunks fill the chip runs work-groups of eight waves (128 query rows
    # share each page image), a smaller one work-groups of four.  A wave's sixteen rows are computed
    # the same way in both, so three chunks in one call (566 work-groups of 64 rows: eight waves) and
    # the same chunks one call each (four waves) must agree in every bit; the oracle checks a sample.
    rng = np.random.Generator(np.random.PCG64(1234))
    cases = [(100, 700), (37, 650), (515, 900)]
    with Twin(n_pages=200, max_seqs=4) as tw:
        tw.pool.set_free_order(rng.permutation(200).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in cases]
        for s, (before, t) in zip(seqs, cases):
            fill(tw, s, before + t, rng, chunk=1024)
        qs = [rng.standard_normal((t, 16, 256)).astype(np.float32) for _, t in cases]
        gates = [rng.standard_normal((t, 16, 256)).astype(np.float32) for _, t in cases]
        together = prefill(tw, 0, seqs, [b for b, _ in cases], qs, 16, gates)
        for i, (s, (before, t)) in enumerate(zip(seqs, cases)):
            alone = prefill(tw, 0, [s], [before], [qs[i]], 16, [gates[i]])[0]
            assert np.array_equal(alone.view(np.uint32), together[i].view(np.uint32)), i
            for tok in (0, t - 1, int(rng.integers(0, t))):
                want = tw.oracle_attend(0, s, before + tok, qs[i][tok], 16, gate=gates[i][tok])
                check_attn(together[i][tok], want, "chunk %d, token %d" % (i, tok))
