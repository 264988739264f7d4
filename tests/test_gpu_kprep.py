"""GPU parity of the fused K preparation + append (RMSNorm * gamma -> partial NEOX rotary ->
cache store) against the CPU oracle's restatement of the reference chain
Qsa::k_norm -> Qsa::rope_k -> Qsa::kv_append.  Bit-exact: every pool byte is compared."""
import numpy as np
import pytest

import oracle
from breccia_amd import lib as L
from breccia_amd.kv import BkvError, DeviceBuffer, device_sync, rope_table
from gpu_common import Twin

pytestmark = pytest.mark.gpu

N_KV, HD, N_ROT, EPS = 2, 256, 64, 1e-6      # the model's geometry, ops/mod.rs:316, :452-454


class Prep:
    """Device copies of gamma / table / positions and the oracle's view of the same."""

    def __init__(self, gamma, max_pos=4096, freq_base=1e7, n_rot=N_ROT, positions=None):
        self.gamma = np.ascontiguousarray(gamma, dtype=np.float32)
        self.table = rope_table(freq_base, n_rot, max_pos)
        self.n_rot, self.max_pos = n_rot, max_pos
        self.positions = None if positions is None else np.ascontiguousarray(positions, dtype=np.int32)
        self.gd = DeviceBuffer.from_numpy(self.gamma)
        self.td = DeviceBuffer.from_numpy(self.table)
        self.pd = None if positions is None else DeviceBuffer.from_numpy(self.positions)

    def free(self):
        for b in (self.gd, self.td, self.pd):
            if b is not None:
                b.free()

    def oracle_k(self, k, pos0, eps=EPS):
        k = np.asarray(k, dtype=np.float32).reshape(-1, N_KV, HD)
        cells = pos0 + np.arange(k.shape[0])
        token_pos = cells if self.positions is None else self.positions[cells]
        return oracle.k_prep(k, N_KV, HD, self.gamma, eps, self.table, self.n_rot, token_pos)


def fused_append(tw, prep, layer, seqs, pos0, ks, vs, eps=EPS):
    """One bkv_append_kprep call on the device; the oracle chain + plain append in the image."""
    n_tok = [np.asarray(k).reshape(-1, N_KV, HD).shape[0] for k in ks]
    kcat = np.concatenate([np.asarray(k, dtype=np.float32).reshape(-1) for k in ks] + [np.zeros(4, np.float32)])
    vcat = np.concatenate([np.asarray(v, dtype=np.float32).reshape(-1) for v in vs] + [np.zeros(4, np.float32)])
    kd, vd = DeviceBuffer.from_numpy(kcat), DeviceBuffer.from_numpy(vcat)
    try:
        tw.pool.append_kprep(layer, seqs, pos0, n_tok, kd, vd, prep.gd, eps, prep.td, prep.n_rot,
                             prep.max_pos, prep.pd)
        device_sync()
    finally:
        kd.free()
        vd.free()
    for s, p0, k, v, t in zip(seqs, pos0, ks, vs, n_tok):
        if t:
            rc = tw.images[layer].append(tw.pool.block_table(s), p0, prep.oracle_k(k, p0, eps), v,
                                         capacity_cells=tw.pool.seq_capacity(s))
            assert rc == 0


@pytest.mark.parametrize("layout", [L.LAYOUT_F16, L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_decode_step_and_ragged_prefill_are_bit_exact(layout):
    rng = np.random.Generator(np.random.PCG64(300 + layout))
    gamma = (1.0 + 0.3 * rng.standard_normal(HD)).astype(np.float32)
    prep = Prep(gamma, max_pos=2048)
    with Twin(n_pages=256, layout=layout, max_seqs=12) as tw:
        seqs = [tw.pool.seq_create() for _ in range(8)]
        lens = [37, 0, 300, 16, 1, 517, 64, 129]
        for step in range(0, 560, 48):                  # interleave so tables are not contiguous
            for s, n in zip(seqs, lens):
                tgt = min(n, step + 48)
                if tgt > tw.pool.seq_len(s):
                    tw.pool.seq_reserve(s, tgt)
        scale = rng.uniform(0.05, 30.0, size=(8,))
        ks = [(rng.standard_normal((n, N_KV, HD)) * sc).astype(np.float32) for n, sc in zip(lens, scale)]
        vs = [rng.standard_normal((n, N_KV, HD)).astype(np.float32) for n in lens]
        fused_append(tw, prep, 0, seqs, [0] * 8, ks, vs)    # one ragged call, one empty sequence
        tw.assert_pools_equal()
        # decode step: one token per sequence at its current length, crossing page edges
        for s in seqs:
            tw.pool.seq_reserve(s, tw.pool.seq_len(s) + 1)
        k1 = [rng.standard_normal((1, N_KV, HD)).astype(np.float32) for _ in seqs]
        v1 = [rng.standard_normal((1, N_KV, HD)).astype(np.float32) for _ in seqs]
        fused_append(tw, prep, 0, seqs, lens, k1, v1)
        tw.assert_pools_equal()
        tw.pool.check()
    prep.free()


@pytest.mark.parametrize("layout", [L.LAYOUT_Q8V, L.LAYOUT_I8H])
def test_bulk_quantised_rows_with_rounding_ties_are_bit_exact(layout):
    # The quantised stores take their codes from a reciprocal of the scale where that provably gives
    # the rule's round-half-away(clamp(x / scale)) (qsa/cpu.rs:65-82) and from the division elsewhere.
    # 2000 tokens in one call; V rows pass through unprepared, so they can carry exact ties (scale 1
    # and 1/4), values one ulp either side of a tie, tiny blocks, a zero block and a lone large value;
    # the prepared K rows are whatever the normalisation makes of rows of very different magnitude.
    rng = np.random.Generator(np.random.PCG64(500 + layout))
    T = 2000
    gamma = (1.0 + 0.3 * rng.standard_normal(HD)).astype(np.float32)
    prep = Prep(gamma, max_pos=2048)
    k = (rng.standard_normal((T, N_KV, HD)) * rng.uniform(1e-3, 300, size=(T, N_KV, 1))).astype(np.float32)
    k[40, 0, :] = 0.0
    k[41, 1, 5:] = 0.0
    v = (rng.standard_normal((T, N_KV, HD)) * rng.uniform(0.05, 30, size=(T, N_KV, 1))).astype(np.float32)
    halves = (np.arange(32, dtype=np.float32) * 7.0) % 126.0 + 0.5
    halves[::2] *= -1.0
    v[10, 0, 0:32] = halves
    v[10, 0, 0] = 127.0
    v[11, 1, 64:96] = halves / 4.0
    v[11, 1, 64] = -127.0 / 4.0
    v[12, 0, 32:64] = np.nextafter(halves, np.float32(1000.0))
    v[12, 0, 32] = 127.0
    v[13, 1, 32:64] = np.nextafter(halves, np.float32(-1000.0))
    v[13, 1, 32] = 127.0
    v[14, 0, 96:128] = rng.standard_normal(32).astype(np.float32) * 1e-3
    v[15, 1, 0:32] = rng.standard_normal(32).astype(np.float32) * 1e-30
    v[16, 0, 128:160] = 0.0
    v[17, 1, 160:192] = 1e-4
    v[17, 1, 161] = 5e4
    with Twin(n_pages=T // 16 + 8, layout=layout, max_seqs=4) as tw:
        tw.pool.set_free_order(rng.permutation(T // 16 + 8).astype(np.int32))
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, T + 3)
        fused_append(tw, prep, 0, [s], [3], [k], [v])
        tw.assert_pools_equal()
    prep.free()


def test_fused_call_equals_the_unfused_chain_on_the_device():
    # bkv_append of the oracle-prepared K rows must land on the same bytes as the fused call
    rng = np.random.Generator(np.random.PCG64(41))
    prep = Prep(rng.standard_normal(HD).astype(np.float32), max_pos=512)
    k = oracle.normalish(0x1234_5678 ^ 256, 200 * N_KV * HD).reshape(200, N_KV, HD)   # ops_conformance.rs:155
    v = oracle.normalish(0xFEED, 200 * N_KV * HD).reshape(200, N_KV, HD)
    with Twin(n_pages=64, max_seqs=4) as tw:
        a, b = tw.pool.seq_create(), tw.pool.seq_create()
        tw.pool.seq_reserve(a, 207)
        tw.pool.seq_reserve(b, 207)
        fused_append(tw, prep, 0, [a], [7], [k], [v])
        tw.append(0, [b], [7], [prep.oracle_k(k, 7)], [v])
        ga, gb = tw.pool.gather(0, a, 0, 207), tw.pool.gather(0, b, 0, 207)
        assert np.array_equal(ga[0].view(np.uint32), gb[0].view(np.uint32))
        assert np.array_equal(ga[1].view(np.uint32), gb[1].view(np.uint32))
        tw.assert_pools_equal()
        # chunked fused appends == one fused append (positions follow the cells)
        c = tw.pool.seq_create()
        tw.pool.seq_reserve(c, 207)
        for at in range(0, 200, 33):
            fused_append(tw, prep, 0, [c], [7 + at], [k[at:at + 33]], [v[at:at + 33]])
        gc = tw.pool.gather(0, c, 0, 207)
        assert np.array_equal(ga[0].view(np.uint32), gc[0].view(np.uint32))
    prep.free()


def test_positions_buffer_clamping_and_edge_rows():
    rng = np.random.Generator(np.random.PCG64(43))
    T = 70
    # an explicit positions buffer indexed by cell, with entries below 0 and past the table
    positions = rng.integers(0, 40, size=128).astype(np.int32)
    positions[[3, 9]] = [-5, -1]
    positions[[20, 33]] = [40, 2**31 - 1]
    prep = Prep(np.ones(HD, dtype=np.float32), max_pos=40, positions=positions)
    k = rng.standard_normal((T, N_KV, HD)).astype(np.float32)
    k[4] = 0.0                                   # a zero row stays zero (eps keeps it finite)
    k[5] *= 1e-20                                # far below sqrt(eps): eps wins, the row stores as zeros
    k[9] *= 0.05                                 # small rows are normalised up to unit RMS
    k[6] *= 1e18                                 # huge rows: squares beyond f32, fine in f64
    k[7, 0, :] = 0.0
    k[7, 0, 200] = -3.0                          # a one-hot in the unrotated tail
    k[8, 1, :] = 0.0
    k[8, 1, 1] = 1.0                             # the reference's NEOX one-hot (ops/cpu.rs:400-421)
    v = rng.standard_normal((T, N_KV, HD)).astype(np.float32)
    with Twin(n_pages=16, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 2 + T)
        fused_append(tw, prep, 0, [s], [2], [k], [v])
        tw.assert_pools_equal()
        gk, _ = tw.pool.gather(0, s, 2, T)
        assert np.all(gk[4] == 0.0) and np.all(np.isfinite(gk))
        assert np.all(gk[5] == 0.0)
        rms = np.sqrt(np.mean(gk[[6, 9]].astype(np.float64) ** 2, axis=-1))
        assert np.all(np.abs(rms - 1.0) < 2e-3)
        # one-hot at dim 1, unit gamma: normalised to sqrt(256) = 16, rotated into dims 1 and 33
        c, sn = prep.table[min(max(int(positions[2 + 8]), 0), 39), 1]
        assert gk[8, 1, 1] == oracle.to_f16(np.float32(np.float32(16.0) * c)) or abs(gk[8, 1, 1] - 16 * c) < 8e-3
        assert abs(gk[8, 1, 33] - 16 * sn) < 8e-3 and gk[8, 1, 2] == 0.0
    prep.free()


def test_errors_come_before_any_launch():
    prep = Prep(np.ones(HD, dtype=np.float32), max_pos=64)
    z = DeviceBuffer(1 << 16)
    with Twin(n_pages=8, max_seqs=2) as tw:
        s = tw.pool.seq_create()
        tw.pool.seq_reserve(s, 20)
        before = tw.pool.read_layer(0, 0).copy()

        def call(**kw):
            a = dict(layer=0, seqs=[s], pos0=[0], n_tokens=[4], k_dev=z, v_dev=z, gamma_dev=prep.gd, eps=EPS,
                     table_dev=prep.td, n_rot=N_ROT, max_pos=64)
            a.update(kw)
            tw.pool.append_kprep(**a)

        for kw, status in [(dict(n_rot=63), L.ERR_INVALID), (dict(n_rot=0), L.ERR_INVALID),
                           (dict(n_rot=258), L.ERR_INVALID), (dict(max_pos=0), L.ERR_INVALID),
                           (dict(gamma_dev=None), L.ERR_INVALID), (dict(table_dev=None), L.ERR_INVALID),
                           (dict(eps=-1.0), L.ERR_INVALID), (dict(k_dev=None), L.ERR_INVALID),
                           (dict(pos0=[30]), L.ERR_RANGE), (dict(layer=3), L.ERR_RANGE),
                           (dict(seqs=[5]), L.ERR_RANGE)]:
            with pytest.raises(BkvError) as ei:
                call(**kw)
            assert ei.value.status == status, kw
        device_sync()
        assert np.array_equal(before, tw.pool.read_layer(0, 0))
        call()                                     # and the well-formed call goes through
        device_sync()
    z.free()
    prep.free()
