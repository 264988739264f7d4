"""GPU parity of decode attention over quantised K/V pools against the CPU oracle, which
dequantises the same stored codes (crates/breccia-kernels/src/qsa/cpu.rs:65-82 for q8_0 V) and
attends in f64.  Tolerances as in test_gpu_attn.py; the quantisation loss itself is measured
separately against the f16 path, as the reference does
(crates/breccia-kernels/tests/attn_conformance.rs:1288-1452)."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer
from gpu_common import REF_BAR_MAX_REL, Twin, check_attn
from helpers import max_abs, max_rel
from test_gpu_attn import fill, score_spread_case

pytestmark = pytest.mark.gpu


def test_reference_q8v_recipe_64_cells():
    # attn_conformance.rs:1355-1452: normalish seeds 0xF1..0xF4, one append of 64 cells, 24 heads,
    # gate from q_full; dense list instead of the reference's sparse ids [0,5,9,15]
    k_all = oracle.normalish(0xF1, 64 * 512).reshape(64, 2, 256)
    v_all = oracle.normalish(0xF2, 64 * 512).reshape(64, 2, 256)
    q = oracle.normalish(0xF3, 24 * 256).reshape(1, 24, 256)
    q_full = oracle.normalish(0xF4, 24 * 512)
    gate = np.ascontiguousarray(q_full.reshape(24, 512)[:, 256:])
    outs = {}
    for layout in (L.LAYOUT_F16, L.LAYOUT_Q8V):
        with Twin(n_pages=4, max_seqs=2, layout=layout) as tw:
            s = tw.pool.seq_create_identity(4)
            tw.pool.seq_reserve(s, 64)
            tw.append(0, [s], [0], [k_all], [v_all])
            tw.assert_pools_equal()
            out = tw.decode_attn(0, [s], [63], q, 24, gate=q_full[256:], gate_strides=(24 * 512, 512))
            want = tw.oracle_attend(0, s, 63, q[0], 24, gate=gate)
            _, rel = check_attn(out[0], want, "layout %d" % layout)
            assert rel <= REF_BAR_MAX_REL, rel     # vs the same-quantised CPU reference: 1e-5 bar
            outs[layout] = out[0]
    # quantisation loss against the f16 path: the reference measured 1.1e-2 (attn_conformance.rs
    # :1430-1452, docs/phase-4/01-forward-pass.md:4614-4617); it must be small but not zero
    loss = max_rel(outs[L.LAYOUT_Q8V], outs[L.LAYOUT_F16])
    assert 0.0 < loss < 3e-2, loss


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("n_q", [16, 24])
def test_quantised_pools_ragged_batch(layout, n_q):
    rng = np.random.Generator(np.random.PCG64(90 + layout + n_q))
    with Twin(n_pages=700, max_seqs=8, layout=layout) as tw:
        seqs = [tw.pool.seq_create() for _ in range(4)]
        lens = [1, 37, 1000, 4099]
        order = rng.permutation(700).astype(np.int32)
        tw.pool.set_free_order(order)
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=1024)
        tw.assert_pools_equal()
        q = rng.standard_normal((4, n_q, 256)).astype(np.float32)
        gate = rng.standard_normal((4, n_q, 256)).astype(np.float32)
        pos = [n - 1 for n in lens]
        out = tw.decode_attn(0, seqs, pos, q, n_q, gate=gate)
        for i, s in enumerate(seqs):
            want = tw.oracle_attend(0, s, pos[i], q[i], n_q, gate=gate[i])
            _, rel = check_attn(out[i], want, "layout %d seq %d" % (layout, i))
            assert rel <= REF_BAR_MAX_REL, rel


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("v_mag", [1.2e-2, 3e-3, 1.0, 900.0])
def test_quantised_values_across_the_scale_range(layout, v_mag):
    # block scales from just above 2^-14 (dequantised values and their low-order parts in the f16
    # subnormal range) up to 7: the result must stay at the same-quantised-reference bar, relative
    # to the largest output.  v_mag 3e-3 puts some blocks' scales below 2^-14: those are stored,
    # and read, as zero by pool and oracle alike.
    rng = np.random.Generator(np.random.PCG64(97 + layout))
    with Twin(n_pages=80, max_seqs=2, layout=layout) as tw:
        s = tw.pool.seq_create()
        n = 1203
        tw.pool.seq_reserve(s, n)
        k = rng.standard_normal((n, 2, 256)).astype(np.float32)
        v = (rng.standard_normal((n, 2, 256)) * v_mag).astype(np.float32)
        v[:, :, 64:96] *= 0.37      # blocks of one row differ in scale
        v[5::7] *= 0.11
        tw.append(0, [s], [0], [k], [v])
        tw.assert_pools_equal()
        q = rng.standard_normal((2, 16, 256)).astype(np.float32)
        pos = [n - 1, 700]
        out = tw.decode_attn(0, [s, s], pos, q, 16)
        for i in range(2):
            want = tw.oracle_attend(0, s, pos[i], q[i], 16)
            assert np.max(np.abs(want)) > 0.0
            rel = max_abs(out[i], want) / float(np.max(np.abs(want)))
            assert rel <= REF_BAR_MAX_REL, (i, rel)


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
@pytest.mark.parametrize("loud_rows", [(4, 16), (9, 10)])
def test_quantised_score_spread_across_the_rows_of_a_page(layout, loud_rows):
    score_spread_case(loud_rows, layout)


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_largest_batch_of_entries_and_the_empty_call(layout):
    # 64 entries (the limit of one call): 16 sequences, 4 positions each (T = 4 decode), lengths
    # from 1 cell to several pages; then 65 entries and 0 entries
    rng = np.random.Generator(np.random.PCG64(98 + layout))
    lens = [1, 2, 15, 16, 17, 31, 33, 64, 65, 100, 129, 200, 255, 256, 257, 300]
    with Twin(n_pages=200, max_seqs=20, layout=layout) as tw:
        tw.pool.set_free_order(rng.permutation(200).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=128)
        ent_seq, pos = [], []
        for s, n in zip(seqs, lens):
            for back in range(4):
                ent_seq.append(s)
                pos.append(max(n - 1 - back, 0))
        assert len(ent_seq) == L.MAX_BATCH
        q = rng.standard_normal((64, 16, 256)).astype(np.float32)
        out = tw.decode_attn(0, ent_seq, pos, q, 16)
        for i in range(64):
            want = tw.oracle_attend(0, ent_seq[i], pos[i], q[i], 16)
            _, rel = check_attn(out[i], want, "layout %d entry %d" % (layout, i))
            assert rel <= REF_BAR_MAX_REL, (i, rel)
        with pytest.raises(BkvError) as ei:
            tw.decode_attn(0, ent_seq + [seqs[0]], pos + [0], np.concatenate([q, q[:1]]), 16)
        assert ei.value.status == L.ERR_INVALID
        # an empty call is a no-op that succeeds
        z = DeviceBuffer(64)
        tw.pool.decode_attn(0, [], [], 16, z, z, 0.0625)
        z.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_quantised_pools_ignore_poisoned_cells(layout):
    # a NaN scale in an unwritten row must not reach the output through 0 * NaN
    rng = np.random.Generator(np.random.PCG64(95 + layout))
    with Twin(n_pages=16, max_seqs=2, layout=layout) as tw:
        tw.pool.fill(0xFF)
        for img in tw.images:
            img.k[:] = 0xFF
            img.v[:] = 0xFF
        s = tw.pool.seq_create()
        q = rng.standard_normal((1, 16, 256)).astype(np.float32)
        for n in (1, 17, 40):
            fill(tw, s, n, rng, chunk=32)
            out = tw.decode_attn(0, [s], [n - 1], q, 16)
            assert np.all(np.isfinite(out))
            check_attn(out[0], tw.oracle_attend(0, s, n - 1, q[0], 16), "poisoned, len %d" % n)


def test_config5_int8_long_context_sample():
    """BASELINE config 5 geometry at a reduced batch: int8 K/V with f16 scales quantised on append
    from N(0,1), contexts up to 40k, 16 q / 2 kv heads; parity on every (sequence, head)."""
    rng = np.random.Generator(np.random.PCG64(20250005))
    lens = [8192 + 5, 40000 + 11, 20000 + 3]
    with Twin(n_pages=sum((n + 15) // 16 for n in lens) + 8, max_seqs=4, layout=L.LAYOUT_I8H) as tw:
        tw.pool.set_free_order(rng.permutation(tw.pool.desc.n_pages).astype(np.int32))
        seqs = [tw.pool.seq_create() for _ in lens]
        for s, n in zip(seqs, lens):
            fill(tw, s, n, rng, chunk=4096)
        q = rng.standard_normal((3, 16, 256)).astype(np.float32)
        pos = [n - 1 for n in lens]
        out = tw.decode_attn(0, seqs, pos, q, 16)
        worst = 0.0
        for i, s in enumerate(seqs):
            want = tw.oracle_attend(0, s, pos[i], q[i], 16, threads=8)
            _, rel = check_attn(out[i], want, "config5 seq %d" % i)
            worst = max(worst, rel)
        assert worst <= REF_BAR_MAX_REL, worst
